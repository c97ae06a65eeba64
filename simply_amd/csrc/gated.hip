// Row-wise kernels of blocks that norm a part's output instead of its input, and of mixers with gates:
//   residual += mult * norm(y)  and the residual handed on in the activation type (no norm in front of the next part);
//   heads normed one by one and multiplied by a gate, sigmoid(g) or silu(g);
//   an activation applied to a product in place;
//   queries and keys rotated on their first dimensions only, then divided by their root mean square, values mixed
//   with those of an earlier layer, keys and values written into pages whose value size differs from the key size.
// Statistics, angles and sums are 32-bit whatever the activation type is; square roots and divisions are the
// correctly rounded ones (no reciprocal-square-root instruction).
#include "api.h"
#include "common.h"

namespace sa {

// ------------------------------------------------------------------ residual += mult * norm(y); out = residual
// y null: nothing is added (the residual is only handed on in out's type).  out null: nothing is handed on.
__global__ __launch_bounds__(256) void residual_add_norm_kernel(
    const void* __restrict__ y, int y_dtype, int64_t y_stride, const void* __restrict__ w, int w_dtype, float eps,
    float plus_one, float mult, float* __restrict__ residual, void* __restrict__ out, int out_dtype, int D) {
  __shared__ float scratch[16];
  const size_t yb = static_cast<size_t>(blockIdx.x) * y_stride, rb = static_cast<size_t>(blockIdx.x) * D;
  if (y == nullptr) {
    for (int d = threadIdx.x; d < D; d += blockDim.x) store_f(out, out_dtype, rb + d, residual[rb + d]);
    return;
  }
  float r = 1.f;
  if (w != nullptr) {
    float ss = 0.f;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      const float v = load_f(y, y_dtype, yb + d);
      ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    r = 1.f / sqrtf(ss / static_cast<float>(D) + eps);
  }
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float v = load_f(y, y_dtype, yb + d);
    if (w != nullptr) v = v * r * (load_f(w, w_dtype, d) + plus_one);
    const float h = residual[rb + d] + mult * v;
    residual[rb + d] = h;
    if (out != nullptr) store_f(out, out_dtype, rb + d, h);
  }
}

// The same with the element types known at compile time and a row held in registers (NP elements a thread): every
// load of a row is asked for before the first use, so the kernel waits for memory once.  It runs a dozen times per
// layer and decode step on a handful of rows, where the kernel above, whose loads sit behind tests of the element
// type, took 10 us; the sums run in the same order, the results are the same bits.
template <typename YT, typename WT, typename OT, int NP>
__global__ __launch_bounds__(256) void residual_add_norm_typed_kernel(
    const YT* __restrict__ y, int64_t y_stride, const WT* __restrict__ w, float eps, float plus_one, float mult,
    float* __restrict__ residual, OT* __restrict__ out, int D) {
  __shared__ float scratch[16];
  const size_t yb = static_cast<size_t>(blockIdx.x) * y_stride, rb = static_cast<size_t>(blockIdx.x) * D;
  float yv[NP], hv[NP], wv[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int d = threadIdx.x + p * 256;
    const bool ok = d < D;
    yv[p] = ok ? to_float(y[yb + d]) : 0.f;
    hv[p] = ok ? residual[rb + d] : 0.f;
    wv[p] = (ok && w != nullptr) ? to_float(w[d]) + plus_one : 1.f;
  }
  float r = 1.f;
  if (w != nullptr) {
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < NP; ++p) ss = fmaf(yv[p], yv[p], ss);
    ss = block_sum(ss, scratch);
    r = 1.f / sqrtf(ss / static_cast<float>(D) + eps);
  }
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int d = threadIdx.x + p * 256;
    if (d >= D) continue;
    const float v = w != nullptr ? yv[p] * r * wv[p] : yv[p];
    const float h = hv[p] + mult * v;
    residual[rb + d] = h;
    if (out != nullptr) out[rb + d] = from_float<OT>(h);
  }
}

template <typename YT, typename WT, typename OT>
static bool launch_residual_add_norm_typed(const void* y, int64_t y_stride, const void* w, float eps, float plus_one,
                                           float mult, float* residual, void* out, int T, int D, hipStream_t stream) {
  const YT* yp = static_cast<const YT*>(y);
  const WT* wp = static_cast<const WT*>(w);
  OT* op = static_cast<OT*>(out);
  if (D <= 1024)
    residual_add_norm_typed_kernel<YT, WT, OT, 4><<<T, 256, 0, stream>>>(yp, y_stride, wp, eps, plus_one, mult, residual, op, D);
  else if (D <= 2048)
    residual_add_norm_typed_kernel<YT, WT, OT, 8><<<T, 256, 0, stream>>>(yp, y_stride, wp, eps, plus_one, mult, residual, op, D);
  else if (D <= 4096)
    residual_add_norm_typed_kernel<YT, WT, OT, 16><<<T, 256, 0, stream>>>(yp, y_stride, wp, eps, plus_one, mult, residual, op, D);
  else
    return false;
  return true;
}

// ------------------------------------------------------------------ residual += mult * y; out = norm(residual)
// The sum of a block that norms what its parts read (their results are added as they are, times a constant), fused
// with the norm in front of the next part: out = h / sqrt(mean(h^2) + eps) * (w + plus_one) over the updated row h,
// which is held in registers between the two.  y null: nothing is added.
template <typename YT, typename OT, int NP>
__global__ __launch_bounds__(256) void residual_add_next_norm_kernel(
    const YT* __restrict__ y, int64_t y_stride, float mult, float* __restrict__ residual, const void* __restrict__ w,
    int w_dtype, float eps, float plus_one, OT* __restrict__ out, int D) {
  __shared__ float scratch[16];
  const size_t yb = static_cast<size_t>(blockIdx.x) * y_stride, rb = static_cast<size_t>(blockIdx.x) * D;
  float hv[NP], wv[NP];
  float ss = 0.f;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int d = threadIdx.x + p * 256;
    const bool ok = d < D;
    const float yv = (ok && y != nullptr) ? to_float(y[yb + d]) : 0.f;
    const float h = ok ? residual[rb + d] : 0.f;
    wv[p] = ok ? load_f(w, w_dtype, d) + plus_one : 0.f;
    hv[p] = y != nullptr ? h + mult * yv : h;
    if (ok && y != nullptr) residual[rb + d] = hv[p];
    ss = fmaf(hv[p], hv[p], ss);
  }
  ss = block_sum(ss, scratch);
  const float r = 1.f / sqrtf(ss / static_cast<float>(D) + eps);
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int d = threadIdx.x + p * 256;
    if (d < D) out[rb + d] = from_float<OT>(hv[p] * r * wv[p]);
  }
}

template <typename YT, typename OT>
static void launch_residual_add_next_norm(const void* y, int64_t y_stride, float mult, float* residual, const void* w,
                                          int w_dtype, float eps, float plus_one, void* out, int T, int D,
                                          hipStream_t stream) {
  const YT* yp = static_cast<const YT*>(y);
  OT* op = static_cast<OT*>(out);
  if (D <= 1024)
    residual_add_next_norm_kernel<YT, OT, 4><<<T, 256, 0, stream>>>(yp, y_stride, mult, residual, w, w_dtype, eps, plus_one, op, D);
  else if (D <= 2048)
    residual_add_next_norm_kernel<YT, OT, 8><<<T, 256, 0, stream>>>(yp, y_stride, mult, residual, w, w_dtype, eps, plus_one, op, D);
  else if (D <= 4096)
    residual_add_next_norm_kernel<YT, OT, 16><<<T, 256, 0, stream>>>(yp, y_stride, mult, residual, w, w_dtype, eps, plus_one, op, D);
  else
    residual_add_next_norm_kernel<YT, OT, 32><<<T, 256, 0, stream>>>(yp, y_stride, mult, residual, w, w_dtype, eps, plus_one, op, D);
}

// ------------------------------------------------------------------ heads normed and gated
// out[t, h, :] = (w ? x[t, h, :] / sqrt(mean(x[t, h, :]^2) + eps) * w : x[t, h, :]) * gate(g[t, h, :]),
// gate 0: sigmoid, 1: silu.  One wave per (token, head); w [size] is shared by the heads.
__device__ inline float gate_value(int kind, float g) {
  const float s = 1.f / (1.f + expf(-g));
  return kind == 1 ? g * s : s;
}

__global__ __launch_bounds__(kWave) void gated_heads_kernel(
    const void* __restrict__ x, int x_dtype, int64_t x_stride, const void* __restrict__ g, int g_dtype,
    int64_t g_stride, const void* __restrict__ w, int w_dtype, float eps, int gate, void* __restrict__ out,
    int out_dtype, int64_t out_stride, int size, int gate_per_head) {
  // gate_per_head: a gate row holds one number per head, which all of the head's entries share
  const int t = blockIdx.x, h = blockIdx.y;
  const size_t xb = static_cast<size_t>(t) * x_stride + static_cast<size_t>(h) * size;
  const size_t gb = static_cast<size_t>(t) * g_stride + (gate_per_head ? h : static_cast<size_t>(h) * size);
  const size_t ob = static_cast<size_t>(t) * out_stride + static_cast<size_t>(h) * size;
  float r = 1.f;
  if (w != nullptr) {
    float ss = 0.f;
    for (int d = threadIdx.x; d < size; d += kWave) {
      const float v = load_f(x, x_dtype, xb + d);
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    r = 1.f / sqrtf(ss / static_cast<float>(size) + eps);
  }
  for (int d = threadIdx.x; d < size; d += kWave) {
    float v = load_f(x, x_dtype, xb + d);
    if (w != nullptr) v = v * r * load_f(w, w_dtype, d);
    store_f(out, out_dtype, ob + d, v * gate_value(gate, load_f(g, g_dtype, gate_per_head ? gb : gb + d)));
  }
}

// ------------------------------------------------------------------ an activation in place
__global__ void activation_kernel(void* __restrict__ x, int dtype, int64_t stride, int N, int act) {
  const size_t rb = static_cast<size_t>(blockIdx.y) * stride;
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n < N) store_f(x, dtype, rb + n, gated_activation_exact(act, load_f(x, dtype, rb + n)));
}

// ------------------------------------------------------------------ queries and keys: partial rotation, unit RMS
// One wave per (token, head) of a fused projection row [H * dk queries | K * dk keys | K * dv values | ...].
//   q, k: the first rot_dims dimensions are rotated in pairs (i, i + rot_dims / 2) by position * inv_freq[i], the
//         others pass; then the head is divided by sqrt(mean(x^2) + eps) (eps < 0: left as it is).  Queries, times
//         q_mult (the scores' factor, for attention kernels that have none), go back in place, keys into the key pages.
//   v:    v <- (1 - lambda) v + lambda v_first (v_first null: v as it is), into the value pages (transposed).
constexpr int kQkPerLane = 8;  // key sizes up to 512
template <typename T>
__global__ __launch_bounds__(kWave) void qk_norm_rope_cache_write_kernel(
    T* __restrict__ proj, int64_t row_stride, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    int rot_dims, float eps, float q_mult, const T* __restrict__ v_first, int64_t v_first_stride,
    const void* __restrict__ lambda,
    int lambda_dtype, const int64_t* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int H, int K, int dk, int dv, int page_size) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  T* row = proj + static_cast<size_t>(t) * row_stride;
  if (head < H + K) {
    const bool is_q = head < H;
    T* src = row + static_cast<size_t>(head) * dk;
    const int half = rot_dims / 2;
    const float pos = static_cast<float>(positions[t]);
    float o[kQkPerLane];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kQkPerLane; ++j) {
      const int i = lane + j * kWave;
      o[j] = 0.f;
      if (i < dk) {
        float v = to_float(src[i]);
        if (i < rot_dims) {
          const int pair = i < half ? i : i - half;
          float s, c;
          sincosf(pos * inv_freq[pair], &s, &c);
          const float other = to_float(src[i < half ? i + half : i - half]);
          v = i < half ? v * c - other * s : v * c + other * s;
        }
        o[j] = v;
        ss = fmaf(v, v, ss);
      }
    }
    ss = wave_sum(ss);
    const float r = eps >= 0.f ? 1.f / sqrtf(ss / static_cast<float>(dk) + eps) : 1.f;
    // (every lane has read what it needs of the head before any lane writes: the wave runs in lockstep, and the
    // reduction above lies between the reads and the writes)
    if (is_q) {
#pragma unroll
      for (int j = 0; j < kQkPerLane; ++j) {
        const int i = lane + j * kWave;
        if (i < dk) src[i] = from_float<T>(o[j] * r * q_mult);
      }
      return;
    }
    if (k_pages == nullptr) return;
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    const int koff = static_cast<int>(slot % page_size);
    T* dst = k_pages + ((slot / page_size) * K + (head - H)) * page_size * dk;
    const bool tiled = keys_tiled(page_size, dk);
#pragma unroll
    for (int j = 0; j < kQkPerLane; ++j) {
      const int i = lane + j * kWave;
      if (i < dk) dst[key_index(tiled, page_size, dk, koff, i)] = from_float<T>(o[j] * r);
    }
    return;
  }
  if (v_pages == nullptr) return;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int vh = head - H - K;
  const T* src = row + static_cast<size_t>(H + K) * dk + static_cast<size_t>(vh) * dv;
  const T* first = v_first == nullptr ? nullptr : v_first + static_cast<size_t>(t) * v_first_stride + static_cast<size_t>(vh) * dv;
  const float lam = first != nullptr ? load_f(lambda, lambda_dtype, 0) : 0.f;
  // value pages are [page, head, dv, page_size]: the keys of a page are contiguous for each dimension
  T* dst = v_pages + ((slot / page_size) * K + vh) * page_size * dv + slot % page_size;
  for (int i = lane; i < dv; i += kWave) {
    float v = to_float(src[i]);
    if (first != nullptr) v = (1.f - lam) * v + lam * to_float(first[i]);
    dst[static_cast<size_t>(i) * page_size] = from_float<T>(v);
  }
}

// ------------------------------------------------------------------ queries and keys: weighted norm, then rotation
// One wave per (token, head) of a fused projection row [H * dk queries | K * dk keys | K * dv values | ...].  A query
// or key vector of dk entries is cut into `sub` equal parts (the score maps of a head); in every part
//   the first norm_dims entries are divided by sqrt(mean of their squares + eps) and multiplied by w[i] (w null: not),
//   then the entries [rot_at, rot_at + rot_dims) turn in neighbouring pairs: (u, v) at the pair p becomes
//   rot_mult * (u cos a - v sin a, v cos a + u sin a) with a = position * freq[p].
// Queries go back in place, keys into the key pages (rows of dk entries), values as they are into the value pages
// (transposed); dv == 0: there are no values.  norm_dims, rot_at and w are given for queries and for keys.
struct HeadNormRope {
  const void* w;
  int norm_dims, rot_at;
};
constexpr int kPartPerLane = 16;  // parts of up to 1024 entries
// NP: pieces of 64 entries that a lane holds of a part (registers for no more than the part needs)
template <typename T, int NP>
__global__ __launch_bounds__(kWave) void norm_rope_cache_write_kernel(
    T* __restrict__ proj, int64_t row_stride, const int* __restrict__ positions, const float* __restrict__ freq,
    int rot_dims, float rot_mult, HeadNormRope qn, HeadNormRope kn, int w_dtype, float eps, int sub,
    const int64_t* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages, int H, int K, int dk,
    int dv, int page_size, int key_values) {
  // key_values > 0: a key row's first key_values entries, as they are stored, are the token's values as well (a latent
  // that is scored and read): they also go into value pages [num_pages, K, key_values, page_size]
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  T* row = proj + static_cast<size_t>(t) * row_stride;
  if (head < H + K) {
    const bool is_q = head < H;
    const HeadNormRope hn = is_q ? qn : kn;
    const int ds = dk / sub;
    const float pos = static_cast<float>(positions[t]);
    int64_t slot = -1;
    T* dst = nullptr;
    bool tiled = false;
    int koff = 0;
    if (!is_q) {
      if (k_pages == nullptr) return;
      slot = slot_mapping[t];
      if (slot < 0) return;
      koff = static_cast<int>(slot % page_size);
      dst = k_pages + ((slot / page_size) * K + (head - H)) * page_size * dk;
      tiled = keys_tiled(page_size, dk);
    }
    for (int part = 0; part < sub; ++part) {
      T* src = row + static_cast<size_t>(head) * dk + static_cast<size_t>(part) * ds;
      float raw[NP], other[NP];
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        const int i = lane + j * kWave;
        raw[j] = other[j] = 0.f;
        if (j * kWave < ds && i < ds) {   // (the first test is uniform: pieces beyond the part cost a branch)
          const int e = i - hn.rot_at;
          const bool turns = e >= 0 && e < rot_dims;
          // a query entry that is neither normed nor rotated stays where it is: it is not even read
          if (!is_q || turns || (hn.w != nullptr && i < hn.norm_dims)) raw[j] = to_float(src[i]);
          if (turns) other[j] = to_float(src[hn.rot_at + (e ^ 1)]);
          if (i < hn.norm_dims) ss = fmaf(raw[j], raw[j], ss);
        }
      }
      float r = 1.f;
      if (hn.w != nullptr && hn.norm_dims > 0) {
        ss = wave_sum(ss);
        r = 1.f / sqrtf(ss / static_cast<float>(hn.norm_dims) + eps);
      }
      // (every lane has read what it needs of the part before any lane writes: the wave runs in lockstep)
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        const int i = lane + j * kWave;
        if (j * kWave >= ds || i >= ds) continue;
        if (is_q && (i - hn.rot_at < 0 || i - hn.rot_at >= rot_dims) && !(hn.w != nullptr && i < hn.norm_dims)) continue;
        float v = raw[j];
        if (hn.w != nullptr && i < hn.norm_dims) v = v * r * load_f(hn.w, w_dtype, i);
        const int e = i - hn.rot_at;
        if (e >= 0 && e < rot_dims) {
          const int pi = hn.rot_at + (e ^ 1);
          float o = other[j];
          if (hn.w != nullptr && pi < hn.norm_dims) o = o * r * load_f(hn.w, w_dtype, pi);
          float sn, cs;
          sincosf(pos * freq[e >> 1], &sn, &cs);
          sn *= rot_mult;
          cs *= rot_mult;
          v = (e & 1) == 0 ? v * cs - o * sn : v * cs + o * sn;
        }
        if (is_q) {
          src[i] = from_float<T>(v);
        } else {
          dst[key_index(tiled, page_size, dk, koff, part * ds + i)] = from_float<T>(v);
          if (part * ds + i < key_values)
            v_pages[(((slot / page_size) * K + (head - H)) * key_values + part * ds + i) * page_size + koff] =
                from_float<T>(v);
        }
      }
    }
    return;
  }
  if (v_pages == nullptr) return;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int vh = head - H - K;
  const T* src = row + static_cast<size_t>(H + K) * dk + static_cast<size_t>(vh) * dv;
  T* dst = v_pages + ((slot / page_size) * K + vh) * page_size * dv + slot % page_size;
  for (int i = lane; i < dv; i += kWave) dst[static_cast<size_t>(i) * page_size] = src[i];
}

}  // namespace sa

using namespace sa;

extern "C" int sa_residual_add_norm(const void* y, int y_dtype, int64_t y_stride, const void* w, int w_dtype, float eps,
                                    int plus_one, float mult, float* residual, void* out, int out_dtype, int T, int D,
                                    hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && D > 0 && residual != nullptr, "residual_add_norm: bad sizes T=%d D=%d", T, D);
  SA_REQUIRE(y != nullptr || out != nullptr, "residual_add_norm: nothing to add and nowhere to hand the residual on");
  SA_REQUIRE(y == nullptr || y_stride >= D, "residual_add_norm: row stride %lld is below the width %d",
             (long long)y_stride, D);
  SA_REQUIRE(eps >= 0.f, "residual_add_norm: eps must not be negative");
  // the usual combinations of element types have kernels of their own (a bfloat16 run, a 32-bit run)
  const float plus = plus_one ? 1.f : 0.f;
  bool done = false;
  if (y != nullptr && y_dtype == kBF16 && (w == nullptr || w_dtype == kBF16) && (out == nullptr || out_dtype == kBF16))
    done = launch_residual_add_norm_typed<bf16, bf16, bf16>(y, y_stride, w, eps, plus, mult, residual, out, T, D, stream);
  else if (y != nullptr && y_dtype == kF32 && (w == nullptr || w_dtype == kF32) && (out == nullptr || out_dtype == kF32))
    done = launch_residual_add_norm_typed<float, float, float>(y, y_stride, w, eps, plus, mult, residual, out, T, D, stream);
  if (!done)
    residual_add_norm_kernel<<<T, 256, 0, stream>>>(y, y_dtype, y_stride, w, w_dtype, eps, plus, mult, residual, out,
                                                    out_dtype, D);
  return check_launch("residual_add_norm");
}

extern "C" int sa_residual_add_next_norm(const void* y, int y_dtype, int64_t y_stride, float mult, float* residual,
                                         const void* w, int w_dtype, float eps, int plus_one, void* out, int out_dtype,
                                         int T, int D, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && D > 0 && D <= 8192 && residual != nullptr && w != nullptr && out != nullptr,
             "residual_add_next_norm: bad sizes T=%d D=%d (rows of at most 8192), or a null pointer", T, D);
  SA_REQUIRE(y == nullptr || y_stride >= D, "residual_add_next_norm: row stride %lld is below the width %d",
             (long long)y_stride, D);
  SA_REQUIRE(eps >= 0.f, "residual_add_next_norm: eps must not be negative");
  const float plus = plus_one ? 1.f : 0.f;
  const bool yb = y == nullptr ? out_dtype == kBF16 : y_dtype == kBF16;
  SA_REQUIRE((y == nullptr || y_dtype == kBF16 || y_dtype == kF32) && (out_dtype == kBF16 || out_dtype == kF32),
             "residual_add_next_norm: rows are bfloat16 or float32");
  if (yb && out_dtype == kBF16)
    launch_residual_add_next_norm<bf16, bf16>(y, y_stride, mult, residual, w, w_dtype, eps, plus, out, T, D, stream);
  else if (yb)
    launch_residual_add_next_norm<bf16, float>(y, y_stride, mult, residual, w, w_dtype, eps, plus, out, T, D, stream);
  else if (out_dtype == kBF16)
    launch_residual_add_next_norm<float, bf16>(y, y_stride, mult, residual, w, w_dtype, eps, plus, out, T, D, stream);
  else
    launch_residual_add_next_norm<float, float>(y, y_stride, mult, residual, w, w_dtype, eps, plus, out, T, D, stream);
  return check_launch("residual_add_next_norm");
}

extern "C" int sa_gated_heads(const void* x, int x_dtype, int64_t x_stride, const void* g, int g_dtype, int64_t g_stride,
                              const void* w, int w_dtype, float eps, int gate, void* out, int out_dtype,
                              int64_t out_stride, int T, int H, int size, int gate_per_head, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && H > 0 && size > 0 && x != nullptr && g != nullptr && out != nullptr,
             "gated_heads: bad sizes T=%d H=%d size=%d", T, H, size);
  const int64_t width = static_cast<int64_t>(H) * size;
  SA_REQUIRE(x_stride >= width && g_stride >= (gate_per_head ? H : width) && out_stride >= width,
             "gated_heads: a row stride is below %lld", (long long)width);
  SA_REQUIRE(gate == 0 || gate == 1, "gated_heads: unknown gate %d (0: sigmoid, 1: silu)", gate);
  SA_REQUIRE(H <= 65535, "gated_heads: at most 65535 heads");
  gated_heads_kernel<<<dim3(T, H), kWave, 0, stream>>>(x, x_dtype, x_stride, g, g_dtype, g_stride, w, w_dtype, eps, gate,
                                                       out, out_dtype, out_stride, size, gate_per_head);
  return check_launch("gated_heads");
}

namespace sa {
int apply_activation(void* x, int dtype, int64_t stride, int M, int N, int act, hipStream_t stream) {
  return sa_activation(x, dtype, stride, M, N, act, stream);
}
}  // namespace sa

extern "C" int sa_activation(void* x, int dtype, int64_t stride, int T, int N, int act, hipStream_t stream) {
  if (T == 0 || N == 0) return 0;
  SA_REQUIRE(T > 0 && N > 0 && stride >= N && T <= 65535 * 1024, "activation: bad sizes T=%d N=%d", T, N);
  SA_REQUIRE(act >= 0 && act < kNumActivations, "activation: unknown activation %d", act);
  SA_REQUIRE(dtype == kF32 || dtype == kBF16, "activation: unknown dtype %d", dtype);
  // rows beyond 65535 go in further launches (the grid's second dimension)
  for (int t0 = 0; t0 < T; t0 += 65535) {
    const int rows = T - t0 < 65535 ? T - t0 : 65535;
    char* base = static_cast<char*>(x) + static_cast<size_t>(t0) * stride * (dtype == kF32 ? 4 : 2);
    activation_kernel<<<dim3((N + 255) / 256, rows), 256, 0, stream>>>(base, dtype, stride, N, act);
  }
  return check_launch("activation");
}

extern "C" int sa_qk_norm_rope_cache_write(void* proj, int dtype, int64_t row_stride, const int* positions,
                                           const float* inv_freq, int rot_dims, float eps, float q_mult,
                                           const void* v_first, int64_t v_first_stride, const void* lambda, int lambda_dtype,
                                           const int64_t* slot_mapping, void* k_pages, void* v_pages, int T, int H,
                                           int K, int dk, int dv, int page_size, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && H >= 0 && K >= 0 && H + 2 * K > 0 && dk > 0 && dv > 0 && page_size > 0,
             "qk_norm_rope_cache_write: bad sizes T=%d H=%d K=%d dk=%d dv=%d P=%d", T, H, K, dk, dv, page_size);
  SA_REQUIRE(dk <= kQkPerLane * kWave, "qk_norm_rope_cache_write: key size %d is above %d", dk, kQkPerLane * kWave);
  SA_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk && (rot_dims == 0 || inv_freq != nullptr),
             "qk_norm_rope_cache_write: %d rotated dimensions of %d (an even number, with their frequencies)", rot_dims, dk);
  SA_REQUIRE(row_stride >= static_cast<int64_t>(H + K) * dk + static_cast<int64_t>(K) * dv,
             "qk_norm_rope_cache_write: row stride %lld is too small", (long long)row_stride);
  SA_REQUIRE((k_pages == nullptr) == (v_pages == nullptr) && (k_pages == nullptr || slot_mapping != nullptr),
             "qk_norm_rope_cache_write: key pages, value pages and slots come together");
  SA_REQUIRE(v_first == nullptr || (lambda != nullptr && v_first_stride >= static_cast<int64_t>(K) * dv),
             "qk_norm_rope_cache_write: mixed values need the factor and rows of K * dv values");
  SA_REQUIRE(H + 2 * K <= 65535, "qk_norm_rope_cache_write: too many heads");
  const dim3 grid(T, H + 2 * K);
  if (dtype == kF32)
    qk_norm_rope_cache_write_kernel<float><<<grid, kWave, 0, stream>>>(
        static_cast<float*>(proj), row_stride, positions, inv_freq, rot_dims, eps, q_mult, static_cast<const float*>(v_first),
        v_first_stride, lambda, lambda_dtype, slot_mapping, static_cast<float*>(k_pages), static_cast<float*>(v_pages),
        H, K, dk, dv, page_size);
  else if (dtype == kBF16)
    qk_norm_rope_cache_write_kernel<bf16><<<grid, kWave, 0, stream>>>(
        static_cast<bf16*>(proj), row_stride, positions, inv_freq, rot_dims, eps, q_mult, static_cast<const bf16*>(v_first),
        v_first_stride, lambda, lambda_dtype, slot_mapping, static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), H,
        K, dk, dv, page_size);
  else
    SA_REQUIRE(false, "qk_norm_rope_cache_write: unknown dtype %d", dtype);
  return check_launch("qk_norm_rope_cache_write");
}

extern "C" int sa_norm_rope_cache_write(void* proj, int dtype, int64_t row_stride, const int* positions,
                                        const float* freq, int rot_dims, float rot_mult, const void* q_weight,
                                        int q_norm_dims, int q_rot_at, const void* k_weight, int k_norm_dims,
                                        int k_rot_at, int w_dtype, float eps, int sub, const int64_t* slot_mapping,
                                        void* k_pages, void* v_pages, int T, int H, int K, int dk, int dv,
                                        int page_size, int key_values, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(key_values >= 0 && key_values <= dk && (key_values == 0 || (dv == 0 && v_pages != nullptr)),
             "norm_rope_cache_write: %d of a key row's %d entries as values (then there are value pages and no values "
             "of their own)", key_values, dk);
  SA_REQUIRE(T > 0 && H >= 0 && K >= 0 && H + K > 0 && dk > 0 && dv >= 0 && page_size > 0 && sub > 0,
             "norm_rope_cache_write: bad sizes T=%d H=%d K=%d dk=%d dv=%d P=%d sub=%d", T, H, K, dk, dv, page_size, sub);
  SA_REQUIRE(dk % sub == 0 && dk / sub <= kPartPerLane * kWave,
             "norm_rope_cache_write: vectors of %d entries in %d parts (equal parts of at most %d)", dk, sub,
             kPartPerLane * kWave);
  const int ds = dk / sub;
  SA_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && (rot_dims == 0 || freq != nullptr) && q_rot_at >= 0 && k_rot_at >= 0 &&
                 q_rot_at + rot_dims <= ds && k_rot_at + rot_dims <= ds,
             "norm_rope_cache_write: %d rotated entries do not fit into parts of %d", rot_dims, ds);
  SA_REQUIRE(q_norm_dims >= 0 && q_norm_dims <= ds && k_norm_dims >= 0 && k_norm_dims <= ds && eps >= 0.f,
             "norm_rope_cache_write: normed entries beyond a part, or a negative eps");
  SA_REQUIRE(row_stride >= static_cast<int64_t>(H + K) * dk + static_cast<int64_t>(K) * dv,
             "norm_rope_cache_write: row stride %lld is too small", (long long)row_stride);
  SA_REQUIRE(k_pages == nullptr || (slot_mapping != nullptr && (dv == 0 || v_pages != nullptr)),
             "norm_rope_cache_write: key pages come with slots (and value pages, if there are values)");
  SA_REQUIRE(H + 2 * K <= 65535, "norm_rope_cache_write: too many heads");
  const dim3 grid(T, H + K + (dv > 0 ? K : 0));
  const HeadNormRope qn{q_weight, q_norm_dims, q_rot_at}, kn{k_weight, k_norm_dims, k_rot_at};
  SA_REQUIRE(dtype == kF32 || dtype == kBF16, "norm_rope_cache_write: unknown dtype %d", dtype);
#define SA_LAUNCH(NP)                                                                                                 \
  do {                                                                                                                \
    if (dtype == kF32)                                                                                                \
      norm_rope_cache_write_kernel<float, NP><<<grid, kWave, 0, stream>>>(                                            \
          static_cast<float*>(proj), row_stride, positions, freq, rot_dims, rot_mult, qn, kn, w_dtype, eps, sub,      \
          slot_mapping, static_cast<float*>(k_pages), static_cast<float*>(v_pages), H, K, dk, dv, page_size,          \
          key_values);                                                                                                \
    else                                                                                                              \
      norm_rope_cache_write_kernel<bf16, NP><<<grid, kWave, 0, stream>>>(                                             \
          static_cast<bf16*>(proj), row_stride, positions, freq, rot_dims, rot_mult, qn, kn, w_dtype, eps, sub,       \
          slot_mapping, static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), H, K, dk, dv, page_size,            \
          key_values);                                                                                                \
  } while (0)
  const int pieces = (ds + kWave - 1) / kWave;
  if (pieces <= 1) SA_LAUNCH(1);
  else if (pieces <= 2) SA_LAUNCH(2);
  else if (pieces <= 4) SA_LAUNCH(4);
  else if (pieces <= 9) SA_LAUNCH(9);
  else SA_LAUNCH(16);
#undef SA_LAUNCH
  return check_launch("norm_rope_cache_write");
}
