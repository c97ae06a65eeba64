// What stands between an attention layer's fused projection and its attention kernel, for layers whose queries,
// keys and values pass a short causal convolution and / or a weighted norm before they are scored:
//
//   convolution   y[t, c] = sum_a taps[c, a] * x[t - (n - 1 - a), c] over the n taps (oldest first), x before a request's
//                 first token of the step from the request's tail (the last n - 1 rows that earlier steps projected,
//                 zeros before the sequence's start); no activation, no bias.  n == 0: no convolution (n == 1: a factor
//                 per channel).
//   norm          of queries and of keys: none; head by head, x / sqrt(mean(x^2) + eps) * w[d] with w shared by the
//                 heads; or over the whole row (all heads at once) with a weight per entry.
//   rotation      the first rot_dims entries of every head turn, entry i with entry i + rot_dims / 2, by the angle
//                 position * inv_freq[i]; after the norm.
//   temperature   queries at position p times 1 + coef * ln(floor((p + 1) / every) + 1)  (every == 0: none), and times
//                 q_mult (the scores' factor, for an attention kernel that has none of its own).
//   bias          (without a convolution) a bias per column of the projection, added as the row is read.
//   values        their own columns of the projection (convolved, otherwise as they are), or the keys' columns as they
//                 stand before norm and rotation.
//
// Queries go to q_out [T, H * dk], keys into key pages [pages, K, P, dk] (operand blocks where the sizes allow),
// values into value pages [pages, K, dv, P].  A layer that reads another layer's keys and values has queries only.
// Everything between the loads and the stores is 32-bit.  A workgroup takes one of the three sections of one token's
// row; the section's convolved entries lie in LDS between the passes.
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kInputThreads = 256;
constexpr int kInputMaxTaps = 16;

struct AttentionInputs {
  int H, K, dk, dv;
  int k_at, v_at;          // first column of the keys and of the values in a projection row (queries start at 0)
  int values_are_keys;     // the keys' columns, as projected, are the values too (then there are no value columns)
  int taps;                // of the convolution; 0: none
  int conv_channels;       // channels that pass the convolution: a tail row's length
  int norm;                // 0 none, 1 head by head, 2 over the whole row
  int rot_dims;
  int temp_every;
  float temp_coef, eps;
  const void* in_bias;      // (or null) added to the projection's columns as they are read; without a convolution only
  int bias_dtype;
  int own_tails;            // every request brings one token: the thread that reads a channel's tail also moves it on
  float q_mult;             // a factor on the queries (the scores' factor, for an attention kernel that has none)
  int page_size;
};

template <typename T>
__global__ __launch_bounds__(kInputThreads) void attention_inputs_kernel(
    const T* __restrict__ proj, int64_t row_stride, AttentionInputs p, const void* __restrict__ taps, int taps_dtype,
    float* __restrict__ tails, int64_t tail_stride, const void* __restrict__ q_w, const void* __restrict__ k_w,
    int w_dtype, const float* __restrict__ inv_freq, const int* __restrict__ seq_meta,
    const int64_t* __restrict__ slot_mapping, T* __restrict__ q_out, int64_t q_stride, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int stage_len) {
  extern __shared__ float smem[];
  float* stage = smem;                 // [stage_len] the section after the convolution
  float* head_r = stage + stage_len;   // [heads] 1 / rms of every head (norm 1)
  float* rot_s = head_r + (p.H > p.K ? p.H : p.K);   // [rot_dims] the token's cosines, then its sines
  __shared__ float red_s[16];
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2], pos0 = meta[3];
  const int j = blockIdx.x;
  if (j >= count) return;
  const int sec = blockIdx.z;          // 0 queries, 1 keys, 2 values
  const int t = first + j, pos = pos0 + j, tid = threadIdx.x;
  const int heads = sec == 0 ? p.H : p.K, size = sec == 2 ? p.dv : p.dk;
  const int col0 = sec == 0 ? 0 : sec == 1 ? p.k_at : p.v_at;
  const int len = heads * size;
  const T* row = proj + static_cast<size_t>(t) * row_stride;

  for (int i = tid; i < len; i += kInputThreads) {
    const int c = col0 + i;
    float v;
    if (p.taps >= 1) {
      float* tail = tails + static_cast<size_t>(slot) * tail_stride;
      v = 0.f;
      for (int a = 0; a < p.taps; ++a) {
        const int jj = j - (p.taps - 1 - a);   // the request's token of this step under tap a; negative: an earlier step's
        const float u = jj >= 0 ? to_float(proj[static_cast<size_t>(first + jj) * row_stride + c])
                                : tail[static_cast<size_t>(p.taps - 1 + jj) * p.conv_channels + c];
        v = fmaf(load_f(taps, taps_dtype, static_cast<size_t>(c) * p.taps + a), u, v);
        // (one token a request: what tap a read is the tail's entry a - 1 from now on; entry a - 1 has been read)
        if (p.own_tails && a >= 1) tail[static_cast<size_t>(a - 1) * p.conv_channels + c] = u;
      }
    } else {
      v = to_float(row[c]);
      if (p.in_bias != nullptr) v += load_f(p.in_bias, p.bias_dtype, c);
    }
    stage[i] = v;
  }
  // the token's angles once for all heads (every head turns by the same ones)
  for (int i = tid; i < p.rot_dims / 2; i += kInputThreads)
    sincosf(static_cast<float>(pos) * inv_freq[i], &rot_s[p.rot_dims / 2 + i], &rot_s[i]);
  __syncthreads();

  const int64_t kv_slot = sec > 0 ? slot_mapping[t] : -1;
  if (sec > 0 && kv_slot < 0) return;
  const int koff = sec > 0 ? static_cast<int>(kv_slot % p.page_size) : 0;
  const int64_t page = sec > 0 ? kv_slot / p.page_size : 0;
  if (sec == 2 || (sec == 1 && p.values_are_keys)) {
    // values as they stand: [page, head, dv, page_size]
    const int dv = sec == 2 ? p.dv : p.dk;
    T* dst = v_pages + page * p.K * dv * p.page_size + koff;
    for (int i = tid; i < len; i += kInputThreads) dst[static_cast<size_t>(i) * p.page_size] = from_float<T>(stage[i]);
    if (sec == 2) return;
  }

  const void* w = sec == 0 ? q_w : k_w;
  float r_all = 1.f;
  if (p.norm == 1) {
    // a wave per head in turn
    const int wave = tid / kWave, lane = tid % kWave;
    for (int h = wave; h < heads; h += kInputThreads / kWave) {
      float ss = 0.f;
      for (int d = lane; d < size; d += kWave) ss = fmaf(stage[h * size + d], stage[h * size + d], ss);
      ss = wave_sum(ss);
      if (lane == 0) head_r[h] = 1.f / sqrtf(ss / static_cast<float>(size) + p.eps);
    }
    __syncthreads();
  } else if (p.norm == 2) {
    float ss = 0.f;
    for (int i = tid; i < len; i += kInputThreads) ss = fmaf(stage[i], stage[i], ss);
    r_all = 1.f / sqrtf(block_sum(ss, red_s) / static_cast<float>(len) + p.eps);
  }
  const float temp = (sec == 0 && p.temp_every > 0)
                         ? (1.f + p.temp_coef * logf(static_cast<float>((pos + 1) / p.temp_every) + 1.f)) * p.q_mult
                         : p.q_mult;
  const int half = p.rot_dims / 2;
  const bool tiled = keys_tiled(p.page_size, p.dk);
  T* kdst = sec == 1 ? k_pages + (page * p.K) * p.page_size * p.dk : nullptr;
  auto normed = [&](int h, int d) -> float {
    const float v = stage[h * size + d];
    if (p.norm == 1) return v * head_r[h] * load_f(w, w_dtype, d);
    if (p.norm == 2) return v * r_all * load_f(w, w_dtype, h * size + d);
    return v;
  };
  for (int i = tid; i < len; i += kInputThreads) {
    const int h = i / size, d = i % size;
    float v = normed(h, d);
    if (d < p.rot_dims) {
      const float o = normed(h, d < half ? d + half : d - half);
      const float cs = rot_s[d < half ? d : d - half], sn = rot_s[half + (d < half ? d : d - half)];
      v = d < half ? v * cs - o * sn : v * cs + o * sn;
    }
    if (sec == 0)
      q_out[static_cast<size_t>(t) * q_stride + i] = from_float<T>(v * temp);
    else
      kdst[static_cast<size_t>(h) * p.page_size * p.dk + key_index(tiled, p.page_size, p.dk, koff, d)] = from_float<T>(v);
  }
}

// The same for bfloat16 rows whose sections are whole pieces of eight entries (key and value sizes that are multiples of
// 8, rows and pages aligned to 16 bytes): a workgroup takes a token's whole row, a thread eight neighbouring channels at
// a time, with 16-byte loads of the projection's rows and of the taps and 16-byte stores of queries and keys (a page's
// key row, in either layout, holds eight neighbouring entries side by side).  The arithmetic, and the order of the
// convolution's sum, are those of the kernel above; a head's sum of squares is added up from its pieces' sums in their
// order.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8v;

__global__ __launch_bounds__(kInputThreads) void attention_inputs_rows_kernel(
    const bf16* __restrict__ proj, int64_t row_stride, AttentionInputs p, const void* __restrict__ taps, int taps_dtype,
    float* __restrict__ tails, int64_t tail_stride, const void* __restrict__ q_w, const void* __restrict__ k_w,
    int w_dtype, const float* __restrict__ inv_freq, const int* __restrict__ seq_meta,
    const int64_t* __restrict__ slot_mapping, bf16* __restrict__ q_out, int64_t q_stride, bf16* __restrict__ k_pages,
    bf16* __restrict__ v_pages, int channels, const bf16* __restrict__ taps_by_tap) {
  // taps_by_tap (or null): the taps once more as [taps][channels], so that a piece's eight weights of a tap are one load
  extern __shared__ float smem[];
  float* stage = smem;                      // [channels] the row after the convolution
  float* piece_ss = stage + channels;       // [channels / 8] sum of squares of every piece
  float* rot_s = piece_ss + channels / 8;   // [rot_dims] the token's cosines, then its sines
  __shared__ float red_s[16];
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2], pos0 = meta[3];
  const int j = blockIdx.x;
  if (j >= count) return;
  const int t = first + j, pos = pos0 + j, tid = threadIdx.x;
  const int q_len = p.H * p.dk, k_end = p.k_at + p.K * p.dk;   // (without keys of its own: channels == q_len)
  const int pieces = channels / 8;

  float ss_q = 0.f, ss_k = 0.f;
  for (int o = tid; o < pieces; o += kInputThreads) {
    const int c = o * 8;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.f;
    if (p.taps >= 1) {
      float* tail = tails + static_cast<size_t>(slot) * tail_stride;
      for (int a = 0; a < p.taps; ++a) {
        const int jj = j - (p.taps - 1 - a);
        float u[8];
        if (jj >= 0) {
          const bf16x8v x = *reinterpret_cast<const bf16x8v*>(proj + static_cast<size_t>(first + jj) * row_stride + c);
#pragma unroll
          for (int e = 0; e < 8; ++e) u[e] = static_cast<float>(x[e]);
        } else {
          const float* tp = tail + static_cast<size_t>(p.taps - 1 + jj) * p.conv_channels + c;
#pragma unroll
          for (int e = 0; e < 8; ++e) u[e] = tp[e];
        }
        if (p.own_tails && a >= 1) {   // (one token a request: what tap a read is the tail's entry a - 1 from now on)
          float* tw = tail + static_cast<size_t>(a - 1) * p.conv_channels + c;
#pragma unroll
          for (int e = 0; e < 8; ++e) tw[e] = u[e];
        }
        if (taps_by_tap != nullptr) {
          const bf16x8v wv = *reinterpret_cast<const bf16x8v*>(taps_by_tap + static_cast<size_t>(a) * p.conv_channels + c);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = fmaf(static_cast<float>(wv[e]), u[e], v[e]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = fmaf(load_f(taps, taps_dtype, static_cast<size_t>(c + e) * p.taps + a), u[e], v[e]);
        }
      }
    } else {
      const bf16x8v x = *reinterpret_cast<const bf16x8v*>(proj + static_cast<size_t>(t) * row_stride + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = static_cast<float>(x[e]);
      if (p.in_bias != nullptr) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += load_f(p.in_bias, p.bias_dtype, c + e);
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      stage[c + e] = v[e];
      ss = fmaf(v[e], v[e], ss);
    }
    piece_ss[o] = ss;
    if (c < q_len) ss_q += ss;
    else if (c < k_end) ss_k += ss;
  }
  for (int i = tid; i < p.rot_dims / 2; i += kInputThreads)
    sincosf(static_cast<float>(pos) * inv_freq[i], &rot_s[p.rot_dims / 2 + i], &rot_s[i]);
  float r_q = 1.f, r_k = 1.f;
  if (p.norm == 2) {
    r_q = 1.f / sqrtf(block_sum(ss_q, red_s) / static_cast<float>(q_len) + p.eps);
    if (channels > q_len) r_k = 1.f / sqrtf(block_sum(ss_k, red_s) / static_cast<float>(p.K * p.dk) + p.eps);
  }
  __syncthreads();

  const bool own = channels > q_len;
  const int64_t kv_slot = own ? slot_mapping[t] : -1;
  const int koff = kv_slot >= 0 ? static_cast<int>(kv_slot % p.page_size) : 0;
  const int64_t page = kv_slot >= 0 ? kv_slot / p.page_size : 0;
  const float temp = (p.temp_every > 0 ? 1.f + p.temp_coef * logf(static_cast<float>((pos + 1) / p.temp_every) + 1.f) : 1.f) *
                     p.q_mult;
  const int half = p.rot_dims / 2;
  const bool tiled = keys_tiled(p.page_size, p.dk);
  for (int o = tid; o < pieces; o += kInputThreads) {
    const int c = o * 8;
    if (c >= k_end || (c >= q_len && p.values_are_keys)) {
      // values as they stand (of a layer whose keys are its values: the keys' pieces, before norm and rotation)
      if (kv_slot >= 0) {
        const int i = c - (c >= k_end ? p.v_at : p.k_at);
        const int dv = c >= k_end ? p.dv : p.dk;
        bf16* dst = v_pages + page * p.K * dv * p.page_size + koff;
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[static_cast<size_t>(i + e) * p.page_size] = float_to_bf16(stage[c + e]);
      }
      if (c >= k_end) continue;
    }
    const bool is_q = c < q_len;
    if (!is_q && kv_slot < 0) continue;
    const int base = is_q ? 0 : p.k_at;
    const int i = c - base, h = i / p.dk, d0 = i % p.dk;
    const void* w = is_q ? q_w : k_w;
    float r = 1.f;
    if (p.norm == 1) {
      float ss = 0.f;
      const int po = (base + h * p.dk) / 8;
      for (int k = 0; k < p.dk / 8; ++k) ss += piece_ss[po + k];
      r = 1.f / sqrtf(ss / static_cast<float>(p.dk) + p.eps);
    } else if (p.norm == 2) {
      r = is_q ? r_q : r_k;
    }
    bf16x8v out;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = d0 + e;
      auto normed = [&](int dd) -> float {
        const float x = stage[base + h * p.dk + dd];
        if (p.norm == 1) return x * r * load_f(w, w_dtype, dd);
        if (p.norm == 2) return x * r * load_f(w, w_dtype, h * p.dk + dd);
        return x;
      };
      float x = normed(d);
      if (d < p.rot_dims) {
        const float other = normed(d < half ? d + half : d - half);
        const float cs = rot_s[d < half ? d : d - half], sn = rot_s[half + (d < half ? d : d - half)];
        x = d < half ? x * cs - other * sn : x * cs + other * sn;
      }
      out[e] = static_cast<__bf16>(is_q ? x * temp : x);
    }
    if (is_q)
      *reinterpret_cast<bf16x8v*>(q_out + static_cast<size_t>(t) * q_stride + i) = out;
    else
      *reinterpret_cast<bf16x8v*>(k_pages + (page * p.K + h) * p.page_size * p.dk +
                                  key_index(tiled, p.page_size, p.dk, koff, d0)) = out;
  }
}

// The tails after the step: the last n - 1 projected rows of every request, from this step's rows and, where the
// step brought fewer than n - 1 tokens, from the old tail.  A thread takes one channel of one request; it reads old
// entries only at places that it has not written yet.
template <typename T>
__global__ __launch_bounds__(kWave) void attention_inputs_tails_kernel(const T* __restrict__ proj, int64_t row_stride,
                                                                       int n, int C, float* __restrict__ tails,
                                                                       int64_t tail_stride,
                                                                       const int* __restrict__ seq_meta) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int c = blockIdx.x * kWave + threadIdx.x;
  if (c >= C || count <= 0) return;
  float* tail = tails + static_cast<size_t>(slot) * tail_stride;
  for (int i = 0; i < n - 1; ++i) {
    const int jj = count - (n - 1) + i;   // token of this step that becomes entry i; negative: an old entry
    tail[static_cast<size_t>(i) * C + c] = jj >= 0 ? to_float(proj[static_cast<size_t>(first + jj) * row_stride + c])
                                                    : tail[static_cast<size_t>(n - 1 + jj) * C + c];
  }
}

}  // namespace sa

using namespace sa;

extern "C" int sa_attention_inputs(const void* proj, int dtype, int64_t row_stride, int H, int K, int dk, int dv,
                                   int k_at, int v_at, int values_are_keys, const void* taps, int taps_dtype,
                                   int num_taps, float* tails, int64_t tail_stride, int norm, const void* q_w,
                                   const void* k_w, int w_dtype, float eps, const float* inv_freq, int rot_dims,
                                   float temp_coef, int temp_every, float q_mult, const int* seq_meta, int num_seqs,
                                   int max_q_len,
                                   const int64_t* slot_mapping, void* q_out, int64_t q_stride, void* k_pages,
                                   void* v_pages, int page_size, const void* taps_by_tap, const void* in_bias,
                                   int bias_dtype, hipStream_t stream) {
  if (num_seqs == 0 || max_q_len == 0) return 0;
  const bool own = k_pages != nullptr;   // keys and values of its own (else: queries only)
  SA_REQUIRE(dtype == kF32 || dtype == kBF16, "attention_inputs: unknown dtype %d", dtype);
  SA_REQUIRE(num_seqs > 0 && max_q_len > 0 && H > 0 && K > 0 && dk > 0 && dv > 0 && page_size > 0 && num_seqs <= 65535,
             "attention_inputs: bad sizes S=%d q=%d H=%d K=%d dk=%d dv=%d P=%d", num_seqs, max_q_len, H, K, dk, dv,
             page_size);
  SA_REQUIRE(proj != nullptr && q_out != nullptr && seq_meta != nullptr && q_stride >= static_cast<int64_t>(H) * dk,
             "attention_inputs: a null pointer, or query rows that are too short");
  SA_REQUIRE(norm >= 0 && norm <= 2 && eps >= 0.f && (norm == 0 || (q_w != nullptr && (!own || k_w != nullptr))),
             "attention_inputs: norm %d (0 none, 1 head by head, 2 the whole row) with its weights", norm);
  SA_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk && (rot_dims == 0 || inv_freq != nullptr),
             "attention_inputs: %d rotated entries of %d (an even number, with their frequencies)", rot_dims, dk);
  SA_REQUIRE(temp_every >= 0, "attention_inputs: the temperature's period must not be negative");
  SA_REQUIRE(!values_are_keys || dv == dk, "attention_inputs: keys that are the values too have the values' size");
  SA_REQUIRE(in_bias == nullptr || (num_taps == 0 && (bias_dtype == kF32 || bias_dtype == kBF16)),
             "attention_inputs: a bias is added here only where no convolution follows (else: before the call)");
  int C = H * dk;
  if (own) {
    SA_REQUIRE(v_pages != nullptr && slot_mapping != nullptr, "attention_inputs: key pages come with value pages and slots");
    SA_REQUIRE(k_at == H * dk && (values_are_keys || v_at == (H + K) * dk),
               "attention_inputs: a projection row holds queries, keys and values in this order, without gaps");
    C = (H + K) * dk + (values_are_keys ? 0 : K * dv);
  }
  SA_REQUIRE(row_stride >= C, "attention_inputs: row stride %lld is below the %d columns", (long long)row_stride, C);
  if (num_taps >= 1)
    SA_REQUIRE(num_taps <= kInputMaxTaps && taps != nullptr &&
                   (num_taps == 1 || (tails != nullptr && tail_stride >= static_cast<int64_t>(num_taps - 1) * C)),
               "attention_inputs: %d taps (at most %d) with their weights and tails of %d rows of %d channels", num_taps,
               kInputMaxTaps, num_taps - 1, C);
  const int max_heads = H > K ? H : K;
  int stage_len = H * dk;
  if (own && K * dk > stage_len) stage_len = K * dk;
  if (own && !values_are_keys && K * dv > stage_len) stage_len = K * dv;
  const size_t smem = sizeof(float) * (static_cast<size_t>(stage_len) + max_heads + rot_dims);
  SA_REQUIRE(smem <= 64 * 1024, "attention_inputs: rows of %d entries do not fit a workgroup's LDS", stage_len);
  AttentionInputs p;
  p.H = H, p.K = K, p.dk = dk, p.dv = dv, p.k_at = k_at, p.v_at = v_at, p.values_are_keys = values_are_keys;
  p.taps = num_taps, p.conv_channels = C, p.norm = norm, p.rot_dims = rot_dims, p.temp_every = temp_every;
  p.temp_coef = temp_coef, p.eps = eps, p.page_size = page_size, p.q_mult = q_mult;
  p.in_bias = in_bias, p.bias_dtype = bias_dtype;
  // with one token a request a channel's tail has one reader, who moves it on; else a second launch does, behind all readers
  p.own_tails = max_q_len == 1 && num_taps > 1;
  const bool tails_launch = num_taps > 1 && !p.own_tails;
  const dim3 grid(max_q_len, num_seqs, own ? (values_are_keys ? 2 : 3) : 1);
  const dim3 tail_grid((C + kWave - 1) / kWave, num_seqs);
  if (dtype == kF32) {
    attention_inputs_kernel<float><<<grid, kInputThreads, smem, stream>>>(
        static_cast<const float*>(proj), row_stride, p, taps, taps_dtype, tails, tail_stride, q_w, k_w, w_dtype, inv_freq,
        seq_meta, slot_mapping, static_cast<float*>(q_out), q_stride, static_cast<float*>(k_pages),
        static_cast<float*>(v_pages), stage_len);
    if (tails_launch)
      attention_inputs_tails_kernel<float><<<tail_grid, kWave, 0, stream>>>(static_cast<const float*>(proj), row_stride,
                                                                            num_taps, C, tails, tail_stride, seq_meta);
  } else if (dk % 8 == 0 && dv % 8 == 0 && row_stride % 8 == 0 && q_stride % 8 == 0 &&
             reinterpret_cast<uintptr_t>(proj) % 16 == 0 && reinterpret_cast<uintptr_t>(q_out) % 16 == 0 &&
             reinterpret_cast<uintptr_t>(k_pages) % 16 == 0 &&
             sizeof(float) * (static_cast<size_t>(C) + C / 8 + rot_dims) <= 64 * 1024) {
    // whole pieces of eight entries, aligned: a workgroup per token, 16-byte accesses
    attention_inputs_rows_kernel<<<dim3(max_q_len, num_seqs), kInputThreads, sizeof(float) * (C + C / 8 + rot_dims),
                                   stream>>>(
        static_cast<const bf16*>(proj), row_stride, p, taps, taps_dtype, tails, tail_stride, q_w, k_w, w_dtype, inv_freq,
        seq_meta, slot_mapping, static_cast<bf16*>(q_out), q_stride, static_cast<bf16*>(k_pages),
        static_cast<bf16*>(v_pages), C,
        (taps_dtype == kBF16 && reinterpret_cast<uintptr_t>(taps_by_tap) % 16 == 0) ? static_cast<const bf16*>(taps_by_tap)
                                                                                    : nullptr);
    if (tails_launch)
      attention_inputs_tails_kernel<bf16><<<tail_grid, kWave, 0, stream>>>(static_cast<const bf16*>(proj), row_stride,
                                                                           num_taps, C, tails, tail_stride, seq_meta);
  } else {
    attention_inputs_kernel<bf16><<<grid, kInputThreads, smem, stream>>>(
        static_cast<const bf16*>(proj), row_stride, p, taps, taps_dtype, tails, tail_stride, q_w, k_w, w_dtype, inv_freq,
        seq_meta, slot_mapping, static_cast<bf16*>(q_out), q_stride, static_cast<bf16*>(k_pages),
        static_cast<bf16*>(v_pages), stage_len);
    if (tails_launch)
      attention_inputs_tails_kernel<bf16><<<tail_grid, kWave, 0, stream>>>(static_cast<const bf16*>(proj), row_stride,
                                                                           num_taps, C, tails, tail_stride, seq_meta);
  }
  return check_launch("attention_inputs");
}
