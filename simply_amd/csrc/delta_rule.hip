// A recurrent mixer with a matrix state per head (the gated delta rule) over a ragged batch of requests:
//
//   short causal convolution per channel, then silu          short_conv_silu_kernel (+ conv_tail_update_kernel)
//   q, k to unit length, q / sqrt(size); beta and decay      delta_prepare_kernel
//   S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q   delta_rule_kernel
//
// A request's tokens of this step are rows first .. first + count - 1 of the step (seq_meta [S, 4]: state slot,
// first row, count, position of the first); what earlier steps left is the slot's state: the matrix S per head and
// the last taps - 1 inputs of the convolution.  Everything is 32-bit; sums run in a fixed order that depends on
// nothing but the sizes, so a token's result is the same however the tokens are cut into steps and whatever else
// is in the batch.
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kMaxTaps = 8;
constexpr int kConvTokens = 16;  // tokens that one thread of the convolution walks through

// y[t, c] = act(sum_j taps[c, j] * x[t - (n - 1 - j), c] + out_bias[c]) with x before the step's first token taken
// from the request's tail [n - 1][C] (oldest first); act is silu (kSilu) or nothing.  With in_bias, x stands for
// x + in_bias[c] (a projection's bias that has not been added yet; the tails hold the sums).  A thread takes one
// channel and kConvTokens consecutive tokens.
template <bool kSilu>
__global__ __launch_bounds__(kWave) void short_conv_kernel(
    const void* __restrict__ x, int x_dtype, int64_t x_stride, const void* __restrict__ taps, int taps_dtype, int n,
    const float* __restrict__ tails, int64_t tail_stride, const int* __restrict__ seq_meta, float* __restrict__ y,
    int C, const void* __restrict__ in_bias, const void* __restrict__ out_bias, int bias_dtype) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int j0 = blockIdx.x * kConvTokens;
  const int c = blockIdx.z * kWave + threadIdx.x;
  if (j0 >= count || c >= C) return;
  float w[kMaxTaps], win[kMaxTaps];   // win[i]: input at token j - (n - 1 - i)
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i) w[i] = i < n ? load_f(taps, taps_dtype, static_cast<size_t>(c) * n + i) : 0.f;
  const float* tail = tails + static_cast<size_t>(slot) * tail_stride;
  const float b_in = in_bias != nullptr ? load_f(in_bias, bias_dtype, c) : 0.f;
  const float b_out = out_bias != nullptr ? load_f(out_bias, bias_dtype, c) : 0.f;
  auto input = [&](int j) -> float {   // j: token of the request in this step; negative: before the step
    if (j >= 0) {
      const float v = load_f(x, x_dtype, static_cast<size_t>(first + j) * x_stride + c);
      return in_bias != nullptr ? v + b_in : v;
    }
    return tail[static_cast<size_t>(n - 1 + j) * C + c];
  };
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i) win[i] = (i >= 1 && i < n) ? input(j0 - (n - i)) : 0.f;   // win[1..n-1]: the n - 1 before j0
  const int jn = count - j0 < kConvTokens ? count - j0 : kConvTokens;
  for (int j = 0; j < jn; ++j) {
#pragma unroll
    for (int i = 0; i + 1 < kMaxTaps; ++i) win[i] = win[i + 1];
    // (the newest sits at win[n - 1]: entries from n on are never read)
    const float cur = input(j0 + j);
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i)
      if (i == n - 1) win[i] = cur;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i)
      if (i < n) acc = fmaf(w[i], win[i], acc);
    if (out_bias != nullptr) acc += b_out;
    y[static_cast<size_t>(first + j0 + j) * C + c] = kSilu ? acc / (1.f + expf(-acc)) : acc;
  }
}

// The tails after the step: the last n - 1 inputs of every request, from this step's rows and, where the step brought
// fewer than n - 1 tokens, from the old tail.  A thread takes one channel of one request; it reads old entries only
// at places that it has not written yet.
__global__ __launch_bounds__(kWave) void conv_tail_update_kernel(const void* __restrict__ x, int x_dtype,
                                                                 int64_t x_stride, int n, float* __restrict__ tails,
                                                                 int64_t tail_stride, const int* __restrict__ seq_meta,
                                                                 int C, const void* __restrict__ in_bias = nullptr,
                                                                 int bias_dtype = 0) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int c = blockIdx.x * kWave + threadIdx.x;
  if (c >= C || count <= 0) return;
  float* tail = tails + static_cast<size_t>(slot) * tail_stride;
  for (int i = 0; i < n - 1; ++i) {
    const int j = count - (n - 1) + i;   // token of this step that becomes entry i; negative: an old entry
    float v;
    if (j >= 0) {
      v = load_f(x, x_dtype, static_cast<size_t>(first + j) * x_stride + c);
      if (in_bias != nullptr) v += load_f(in_bias, bias_dtype, c);
    } else {
      v = tail[static_cast<size_t>(n - 1 + j) * C + c];
    }
    tail[static_cast<size_t>(i) * C + c] = v;
  }
}

// Per (token, unit): units 0 .. 2 G - 1 are the q and k heads of qkv [T, C] (q heads first), each made a unit vector
// x / sqrt(sum(x^2) + 1e-6), the queries also times size^(-1/2); unit 2 G computes, for every value head h,
// beta = sigmoid(b) and g = exp(-exp(A_log) * softplus(a + dt_bias)) into gates [T, 2 H] (beta first).
__global__ __launch_bounds__(kWave) void delta_prepare_kernel(float* __restrict__ qkv, int C, int G, int dk,
                                                              const void* __restrict__ ab, int ab_dtype,
                                                              int64_t ab_stride, const void* __restrict__ a_log,
                                                              const void* __restrict__ dt_bias, int vec_dtype, int H,
                                                              float* __restrict__ gates) {
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  if (unit < 2 * G) {
    float* head = qkv + static_cast<size_t>(t) * C + static_cast<size_t>(unit) * dk;
    float ss = 0.f;
    for (int i = lane; i < dk; i += kWave) ss = fmaf(head[i], head[i], ss);
    ss = wave_sum(ss);
    float r = 1.f / sqrtf(ss + 1e-6f);
    if (unit < G) r *= 1.f / sqrtf(static_cast<float>(dk));
    for (int i = lane; i < dk; i += kWave) head[i] *= r;
    return;
  }
  for (int h = lane; h < H; h += kWave) {
    const float a = load_f(ab, ab_dtype, static_cast<size_t>(t) * ab_stride + h);
    const float b = load_f(ab, ab_dtype, static_cast<size_t>(t) * ab_stride + H + h);
    const float z = a + load_f(dt_bias, vec_dtype, h);
    const float sp = z > 30.f ? z : log1pf(expf(z));
    gates[static_cast<size_t>(t) * 2 * H + h] = 1.f / (1.f + expf(-b));
    gates[static_cast<size_t>(t) * 2 * H + H + h] = expf(-expf(load_f(a_log, vec_dtype, h)) * sp);
  }
}

// For steps in which every request brings few tokens (decoding): the convolution with silu, the new tails, the
// unit norms of q and k and the gates in one launch.  A wave per (request, unit); units 0 .. 2 G - 1 are the q and
// k heads (the wave walks the request's tokens in order with each lane's channels' last inputs in registers, norms
// each token's head across its lanes, and leaves the tails), the next ones are pieces of 256 value channels, the
// last one computes beta and g for the request's tokens.  The arithmetic per element is that of the separate
// kernels, in the same order.
constexpr int kFewTokens = 16;
constexpr int kFewChannels = 4;   // channels per lane: key sizes up to 256, value pieces of 256
template <typename XT>   // the element type of the inputs and of the taps
__global__ __launch_bounds__(kWave) void delta_inputs_few_kernel(
    const XT* __restrict__ x, int64_t x_stride, const XT* __restrict__ taps, int n,
    float* __restrict__ tails, int64_t tail_stride, const int* __restrict__ seq_meta, float* __restrict__ y, int C, int G,
    int dk, const void* __restrict__ ab, int ab_dtype, int64_t ab_stride, const void* __restrict__ a_log,
    const void* __restrict__ dt_bias, int vec_dtype, int H, float* __restrict__ gates) {
  const int* meta = seq_meta + 4 * blockIdx.x;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int unit = blockIdx.y, lane = threadIdx.x;
  const int value_units = (C - 2 * G * dk + kFewChannels * kWave - 1) / (kFewChannels * kWave);
  if (unit == 2 * G + value_units) {
    for (int idx = lane; idx < count * H; idx += kWave) {
      const int t = first + idx / H, h = idx % H;
      const float a = load_f(ab, ab_dtype, static_cast<size_t>(t) * ab_stride + h);
      const float b = load_f(ab, ab_dtype, static_cast<size_t>(t) * ab_stride + H + h);
      const float z = a + load_f(dt_bias, vec_dtype, h);
      const float sp = z > 30.f ? z : log1pf(expf(z));
      gates[static_cast<size_t>(t) * 2 * H + h] = 1.f / (1.f + expf(-b));
      gates[static_cast<size_t>(t) * 2 * H + H + h] = expf(-expf(load_f(a_log, vec_dtype, h)) * sp);
    }
    return;
  }
  const bool head = unit < 2 * G;
  const int c0 = head ? unit * dk : 2 * G * dk + (unit - 2 * G) * kFewChannels * kWave;
  const int c1 = head ? c0 + dk : (c0 + kFewChannels * kWave < C ? c0 + kFewChannels * kWave : C);
  float* tail = tails + static_cast<size_t>(slot) * tail_stride;
  float w[kFewChannels][kMaxTaps], win[kFewChannels][kMaxTaps];
#pragma unroll
  for (int k = 0; k < kFewChannels; ++k) {
    const int c = c0 + lane + k * kWave;
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
      w[k][i] = (c < c1 && i < n) ? to_float(taps[static_cast<size_t>(c) * n + i]) : 0.f;
      win[k][i] = (c < c1 && i >= 1 && i < n) ? tail[static_cast<size_t>(i - 1) * C + c] : 0.f;   // the n - 1 before the step
    }
  }
  const float q_scale = unit < G ? 1.f / sqrtf(static_cast<float>(dk)) : 1.f;
  for (int j = 0; j < count; ++j) {
    float v[kFewChannels];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < kFewChannels; ++k) {
      const int c = c0 + lane + k * kWave;
      v[k] = 0.f;
      if (c < c1) {
#pragma unroll
        for (int i = 0; i + 1 < kMaxTaps; ++i) win[k][i] = win[k][i + 1];
        const float cur = to_float(x[static_cast<size_t>(first + j) * x_stride + c]);
#pragma unroll
        for (int i = 0; i < kMaxTaps; ++i)
          if (i == n - 1) win[k][i] = cur;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < kMaxTaps; ++i)
          if (i < n) acc = fmaf(w[k][i], win[k][i], acc);
        v[k] = acc / (1.f + expf(-acc));
        ss = fmaf(v[k], v[k], ss);
      }
    }
    float r = 1.f;
    if (head) {   // (uniform over the wave)
      // the sum runs over a lane's channels first and then across the lanes; the separate kernel's runs in the same order
      ss = wave_sum(ss);
      r = (1.f / sqrtf(ss + 1e-6f)) * q_scale;
    }
#pragma unroll
    for (int k = 0; k < kFewChannels; ++k) {
      const int c = c0 + lane + k * kWave;
      if (c < c1) y[static_cast<size_t>(first + j) * C + c] = head ? v[k] * r : v[k];
    }
  }
  if (count <= 0) return;
#pragma unroll
  for (int k = 0; k < kFewChannels; ++k) {
    const int c = c0 + lane + k * kWave;
    if (c >= c1) continue;
#pragma unroll
    for (int i = 0; i + 1 < kMaxTaps; ++i)
      if (i + 1 < n) tail[static_cast<size_t>(i) * C + c] = win[k][i + 1];
  }
}

// The recurrence.  A workgroup of 256 threads takes 256 / LPC columns of one head's state for one request: LPC lanes
// (4, 16 or a whole wave of 64) share a column, lane `part` of them holding rows part, part + LPC, ...
// of it in registers (DK / LPC of them).  The step's q, k and v of kRuleTokens tokens at a time go through LDS.
// Columns are independent of each other; a column's sums run within a lane over its rows in increasing order, in
// four partial sums that are added in a fixed order, then across the lanes by data-parallel primitives in a fixed
// order: nothing depends on how the tokens are cut into steps or on the batch.  The chain of dependent operations
// per token, and the instructions that one wave issues for it, are what bound a prompt's time (tokens follow one
// another, and a head's columns are all the waves there are): 16 lanes per column, or a wave, keep both short where
// a column has 64 rows or more.
constexpr int kRuleTokens = 16;
template <int DK, int LPC>
__global__ __launch_bounds__(256) void delta_rule_kernel(const float* __restrict__ qkv, int C, int G, int dk, int dv,
                                                         const float* __restrict__ gates, int H,
                                                         float* __restrict__ state, int64_t state_stride,
                                                         const int* __restrict__ seq_meta, float* __restrict__ out) {
  constexpr int R = DK / LPC, COLS = 256 / LPC;
  static_assert(R % 4 == 0 || R < 4, "rows per lane come in fours");
  constexpr int NACC = R < 4 ? 1 : 4;
  __shared__ float qs[kRuleTokens][DK], ks[kRuleTokens][DK], vs[kRuleTokens][COLS], bg[kRuleTokens][2];
  const int* meta = seq_meta + 4 * blockIdx.x;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int h = blockIdx.y, tid = threadIdx.x;
  const int col = blockIdx.z * COLS + tid / LPC, part = tid % LPC;
  const bool live = col < dv;
  const int qk_head = h / (H / G);
  // a head's state is kept column by column, [dv][dk]: the lanes that share a column read neighbouring words
  float* S = state + static_cast<size_t>(slot) * state_stride + static_cast<size_t>(h) * dk * dv;
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = r * LPC + part;
    s[r] = (live && i < dk) ? S[static_cast<size_t>(col) * dk + i] : 0.f;
  }
  const int v_at = 2 * G * dk + h * dv;
  // A tile's q, k, v and gates are asked for a tile ahead, into registers, and put into LDS when the tile's turn
  // comes: the loads are under way while the tile before is worked through.
  constexpr int PQ = kRuleTokens * DK / 256, PV = (kRuleTokens * COLS + 255) / 256;
  float pq[PQ], pk[PQ], pv[PV], pg = 0.f;
  auto fetch = [&](int t0) __attribute__((always_inline)) {
    const int tn = count - t0 < kRuleTokens ? count - t0 : kRuleTokens;
#pragma unroll
    for (int i = 0; i < PQ; ++i) {
      const int idx = tid + i * 256, j = idx / DK, d = idx % DK;
      const bool ok = j < tn && d < dk;
      const float* row = qkv + static_cast<size_t>(first + t0 + (ok ? j : 0)) * C;
      pq[i] = ok ? row[qk_head * dk + d] : 0.f;
      pk[i] = ok ? row[(G + qk_head) * dk + d] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256, j = idx / COLS, c = blockIdx.z * COLS + idx % COLS;
      const bool ok = idx < kRuleTokens * COLS && j < tn && c < dv;
      pv[i] = ok ? qkv[static_cast<size_t>(first + t0 + j) * C + v_at + c] : 0.f;
    }
    pg = tid < 2 * tn ? gates[static_cast<size_t>(first + t0 + tid / 2) * 2 * H + (tid % 2) * H + h] : 0.f;
  };
  if (count > 0) fetch(0);
  for (int t0 = 0; t0 < count; t0 += kRuleTokens) {
    const int tn = count - t0 < kRuleTokens ? count - t0 : kRuleTokens;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PQ; ++i) {
      const int idx = tid + i * 256;
      qs[idx / DK][idx % DK] = pq[i];
      ks[idx / DK][idx % DK] = pk[i];
    }
#pragma unroll
    for (int i = 0; i < PV; ++i) {
      const int idx = tid + i * 256;
      if (idx < kRuleTokens * COLS) vs[idx / COLS][idx % COLS] = pv[i];
    }
    if (tid < 2 * kRuleTokens) bg[tid / 2][tid % 2] = pg;
    __syncthreads();
    if (t0 + kRuleTokens < count) fetch(t0 + kRuleTokens);
    // the token's operands are read from LDS a token ahead, into one of two sets of registers in turn
    struct Operands {
      float k[R], q[R], v, beta, g;
    };
    auto read = [&](Operands& x, int j) __attribute__((always_inline)) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        x.k[r] = ks[j][r * LPC + part];
        x.q[r] = qs[j][r * LPC + part];
      }
      x.v = vs[j][tid / LPC];
      x.beta = bg[j][0];
      x.g = bg[j][1];
    };
    auto token = [&](const Operands& x, int j) __attribute__((always_inline)) {
      float d[NACC];
#pragma unroll
      for (int a = 0; a < NACC; ++a) d[a] = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        s[r] *= x.g;
        d[r % NACC] = fmaf(s[r], x.k[r], d[r % NACC]);
      }
      float dot = NACC == 4 ? (d[0] + d[1]) + (d[2] + d[3]) : d[0];
      dot = lanes_sum<LPC>(dot);
      const float u = x.beta * (x.v - dot);
#pragma unroll
      for (int a = 0; a < NACC; ++a) d[a] = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        s[r] = fmaf(x.k[r], u, s[r]);
        d[r % NACC] = fmaf(s[r], x.q[r], d[r % NACC]);
      }
      float o = NACC == 4 ? (d[0] + d[1]) + (d[2] + d[3]) : d[0];
      o = lanes_sum<LPC>(o);
      if (live && part == 0)
        out[static_cast<size_t>(first + t0 + j) * (static_cast<size_t>(H) * dv) + static_cast<size_t>(h) * dv + col] = o;
    };
    Operands A, B;
    read(A, 0);
    for (int j = 0; j < tn; j += 2) {
      if (j + 1 < tn) read(B, j + 1);
      token(A, j);
      if (j + 1 < tn) {
        if (j + 2 < tn) read(A, j + 2);
        token(B, j + 1);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = r * LPC + part;
    if (live && i < dk) S[static_cast<size_t>(col) * dk + i] = s[r];
  }
}

}  // namespace sa

using namespace sa;

extern "C" int sa_short_conv(const void* x, int x_dtype, int64_t x_stride, const void* in_bias, const void* taps,
                             int taps_dtype, int num_taps, const void* out_bias, int bias_dtype, int silu, float* tails,
                             int64_t tail_stride, const int* seq_meta, int num_seqs, int max_q_len, float* y, int C,
                             int update_tails, hipStream_t stream) {
  if (num_seqs == 0 || max_q_len == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && max_q_len > 0 && C > 0 && x != nullptr && taps != nullptr &&
                 (tails != nullptr || num_taps == 1) && seq_meta != nullptr && y != nullptr,
             "short_conv: bad sizes S=%d q=%d C=%d", num_seqs, max_q_len, C);
  SA_REQUIRE(num_taps >= 1 && num_taps <= kMaxTaps, "short_conv: 1 to %d taps, got %d", kMaxTaps, num_taps);
  SA_REQUIRE(x_stride >= C && tail_stride >= static_cast<int64_t>(num_taps - 1) * C,
             "short_conv: a stride is below what the %d channels need", C);
  SA_REQUIRE(num_seqs <= 65535 && (C + kWave - 1) / kWave <= 65535, "short_conv: too many requests or channels");
  const dim3 grid((max_q_len + kConvTokens - 1) / kConvTokens, num_seqs, (C + kWave - 1) / kWave);
  if (silu)
    short_conv_kernel<true><<<grid, kWave, 0, stream>>>(x, x_dtype, x_stride, taps, taps_dtype, num_taps, tails,
                                                        tail_stride, seq_meta, y, C, in_bias, out_bias, bias_dtype);
  else
    short_conv_kernel<false><<<grid, kWave, 0, stream>>>(x, x_dtype, x_stride, taps, taps_dtype, num_taps, tails,
                                                         tail_stride, seq_meta, y, C, in_bias, out_bias, bias_dtype);
  if (update_tails && num_taps > 1)
    conv_tail_update_kernel<<<dim3((C + kWave - 1) / kWave, num_seqs), kWave, 0, stream>>>(
        x, x_dtype, x_stride, num_taps, tails, tail_stride, seq_meta, C, in_bias, bias_dtype);
  return check_launch("short_conv");
}

extern "C" int sa_short_conv_silu(const void* x, int x_dtype, int64_t x_stride, const void* taps, int taps_dtype,
                                  int num_taps, float* tails, int64_t tail_stride, const int* seq_meta, int num_seqs,
                                  int max_q_len, float* y, int C, int update_tails, hipStream_t stream) {
  return sa_short_conv(x, x_dtype, x_stride, nullptr, taps, taps_dtype, num_taps, nullptr, 0, 1, tails, tail_stride,
                       seq_meta, num_seqs, max_q_len, y, C, update_tails, stream);
}

extern "C" int sa_delta_prepare(float* qkv, int T, int C, int G, int dk, const void* ab, int ab_dtype, int64_t ab_stride,
                                const void* a_log, const void* dt_bias, int vec_dtype, int H, float* gates,
                                hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && G > 0 && dk > 0 && H > 0 && C >= 2 * G * dk && H % G == 0 && ab_stride >= 2 * H,
             "delta_prepare: bad sizes T=%d C=%d G=%d dk=%d H=%d", T, C, G, dk, H);
  SA_REQUIRE(qkv != nullptr && ab != nullptr && a_log != nullptr && dt_bias != nullptr && gates != nullptr,
             "delta_prepare: a null pointer");
  SA_REQUIRE(2 * G + 1 <= 65535, "delta_prepare: too many heads");
  delta_prepare_kernel<<<dim3(T, 2 * G + 1), kWave, 0, stream>>>(qkv, C, G, dk, ab, ab_dtype, ab_stride, a_log, dt_bias,
                                                                 vec_dtype, H, gates);
  return check_launch("delta_prepare");
}

extern "C" int sa_delta_inputs_few_takes(int max_q_len, int dk) {
  return max_q_len >= 1 && max_q_len <= kFewTokens && dk <= kFewChannels * kWave;
}

extern "C" int sa_delta_inputs_few(const void* x, int x_dtype, int64_t x_stride, const void* taps, int taps_dtype,
                                   int num_taps, float* tails, int64_t tail_stride, const int* seq_meta, int num_seqs,
                                   int max_q_len, float* y, int C, int G, int dk, const void* ab, int ab_dtype,
                                   int64_t ab_stride, const void* a_log, const void* dt_bias, int vec_dtype, int H,
                                   float* gates, hipStream_t stream) {
  if (num_seqs == 0 || max_q_len == 0) return 0;
  SA_REQUIRE(sa_delta_inputs_few_takes(max_q_len, dk), "delta_inputs_few: at most %d tokens a request and key sizes up to %d",
             kFewTokens, kFewChannels * kWave);
  SA_REQUIRE(num_seqs > 0 && num_seqs <= 65535 && C > 0 && G > 0 && dk > 0 && H > 0 && H % G == 0 && C >= 2 * G * dk,
             "delta_inputs_few: bad sizes S=%d C=%d G=%d dk=%d H=%d", num_seqs, C, G, dk, H);
  SA_REQUIRE(num_taps >= 1 && num_taps <= kMaxTaps, "delta_inputs_few: 1 to %d taps, got %d", kMaxTaps, num_taps);
  SA_REQUIRE(x != nullptr && taps != nullptr && (tails != nullptr || num_taps == 1) && seq_meta != nullptr &&
                 y != nullptr && ab != nullptr && a_log != nullptr && dt_bias != nullptr && gates != nullptr,
             "delta_inputs_few: a null pointer");
  SA_REQUIRE(x_stride >= C && ab_stride >= 2 * H && tail_stride >= static_cast<int64_t>(num_taps - 1) * C,
             "delta_inputs_few: a stride is below what the sizes need");
  const int value_units = (C - 2 * G * dk + kFewChannels * kWave - 1) / (kFewChannels * kWave);
  SA_REQUIRE(2 * G + value_units + 1 <= 65535, "delta_inputs_few: too many heads or channels");
  SA_REQUIRE(x_dtype == taps_dtype && (x_dtype == kF32 || x_dtype == kBF16),
             "delta_inputs_few: inputs and taps of one element type, float32 or bfloat16");
  const dim3 grid(num_seqs, 2 * G + value_units + 1);
  if (x_dtype == kBF16)
    delta_inputs_few_kernel<bf16><<<grid, kWave, 0, stream>>>(
        static_cast<const bf16*>(x), x_stride, static_cast<const bf16*>(taps), num_taps, tails, tail_stride, seq_meta, y,
        C, G, dk, ab, ab_dtype, ab_stride, a_log, dt_bias, vec_dtype, H, gates);
  else
    delta_inputs_few_kernel<float><<<grid, kWave, 0, stream>>>(
        static_cast<const float*>(x), x_stride, static_cast<const float*>(taps), num_taps, tails, tail_stride, seq_meta,
        y, C, G, dk, ab, ab_dtype, ab_stride, a_log, dt_bias, vec_dtype, H, gates);
  return check_launch("delta_inputs_few");
}

extern "C" int sa_delta_rule(const float* qkv, int C, int G, int dk, int dv, const float* gates, int H, float* state,
                             int64_t state_stride, const int* seq_meta, int num_seqs, float* out, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && G > 0 && H > 0 && H % G == 0 && dk > 0 && dv > 0 && C >= 2 * G * dk + H * dv,
             "delta_rule: bad sizes S=%d C=%d G=%d H=%d dk=%d dv=%d", num_seqs, C, G, H, dk, dv);
  SA_REQUIRE(dk <= 256, "delta_rule: key size %d is above 256", dk);
  SA_REQUIRE(state_stride >= static_cast<int64_t>(H) * dk * dv, "delta_rule: the state rows are too short");
  SA_REQUIRE(qkv != nullptr && gates != nullptr && state != nullptr && seq_meta != nullptr && out != nullptr,
             "delta_rule: a null pointer");
  SA_REQUIRE(H <= 65535 && dv <= 65535 * 16, "delta_rule: too many heads or columns");
#define SA_DELTA_RULE(DK, LPC)                                                                                      \
  delta_rule_kernel<DK, LPC><<<dim3(num_seqs, H, (dv + 256 / LPC - 1) / (256 / LPC)), 256, 0, stream>>>(             \
      qkv, C, G, dk, dv, gates, H, state, state_stride, seq_meta, out)
  if (dk <= 16) SA_DELTA_RULE(16, 4);
  else if (dk <= 32) SA_DELTA_RULE(32, 4);
  else if (dk <= 64) SA_DELTA_RULE(64, 16);
  else if (dk <= 128) SA_DELTA_RULE(128, 64);
  else SA_DELTA_RULE(256, 64);
#undef SA_DELTA_RULE
  return check_launch("delta_rule");
}
