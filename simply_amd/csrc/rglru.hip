// A recurrent mixer with one number of state per channel (the real-gated linear recurrent unit), and the product per
// head that its block-diagonal gates (and the per-head factors of a latent attention) are:
//
//   out[t, h, :] = w[h] x[t, h, :]                                         head_product_kernel
//   a = exp(-c sigmoid(.) softplus(lam));  S <- a S + sqrt(1 - a^2) i u    rglru_scan_kernel
//
// Everything is summed in 32-bit in an order that the sizes alone fix, so a token's result is the same however the
// tokens are cut into steps and whatever else is in the batch.
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kHpTokens = 16;   // tokens of a tile
constexpr int kHpOutputs = 64;  // outputs of a tile
constexpr int kHpChunk = 64;    // inputs staged at a time

// A workgroup of 256 threads takes 16 tokens x 64 outputs of one head: thread (ty, tx) sums output tx for the tokens
// 4 ty .. 4 ty + 3 over the inputs in their order, with the weights' and the rows' chunk of 64 inputs in LDS.
__global__ __launch_bounds__(256) void head_product_kernel(
    const void* __restrict__ x, int x_dtype, int64_t x_stride, int64_t x_head_stride, const void* __restrict__ w,
    int w_dtype, void* __restrict__ out, int out_dtype, int64_t out_stride, int64_t out_head_stride, int T, int I, int O,
    int tail, const void* __restrict__ gate, int gate_dtype, int64_t gate_stride) {
  __shared__ float ws[kHpChunk][kHpOutputs + 1];
  __shared__ float xs[kHpTokens][kHpChunk];
  const int t0 = blockIdx.x * kHpTokens, h = blockIdx.y, o0 = blockIdx.z * kHpOutputs;
  const int tid = threadIdx.x, tx = tid % kHpOutputs, ty = tid / kHpOutputs;
  const size_t wb = static_cast<size_t>(h) * O * I;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int i0 = 0; i0 < I; i0 += kHpChunk) {
    __syncthreads();
    for (int e = tid; e < kHpOutputs * kHpChunk; e += 256) {
      const int o = e / kHpChunk, i = e % kHpChunk;
      ws[i][o] = (o0 + o < O && i0 + i < I) ? load_f(w, w_dtype, wb + static_cast<size_t>(o0 + o) * I + i0 + i) : 0.f;
    }
    for (int e = tid; e < kHpTokens * kHpChunk; e += 256) {
      const int k = e / kHpChunk, i = e % kHpChunk;
      xs[k][i] = (t0 + k < T && i0 + i < I)
                     ? load_f(x, x_dtype, static_cast<size_t>(t0 + k) * x_stride + static_cast<size_t>(h) * x_head_stride + i0 + i)
                     : 0.f;
    }
    __syncthreads();
    const int in = I - i0 < kHpChunk ? I - i0 : kHpChunk;
    for (int i = 0; i < in; ++i) {
      const float wv = ws[i][tx];
#pragma unroll
      for (int k = 0; k < 4; ++k) acc[k] = fmaf(xs[4 * ty + k][i], wv, acc[k]);
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int t = t0 + 4 * ty + k;
    if (t >= T) continue;
    const size_t ob = static_cast<size_t>(t) * out_stride + static_cast<size_t>(h) * out_head_stride;
    if (o0 + tx < O) {
      float v = acc[k];
      if (gate != nullptr) v *= 1.f / (1.f + expf(-load_f(gate, gate_dtype, static_cast<size_t>(t) * gate_stride + h)));
      store_f(out, out_dtype, ob + o0 + tx, v);
    }
    if (blockIdx.z == 0 && tx < tail) {   // (tails of up to 64 entries per pass)
      const size_t xb = static_cast<size_t>(t) * x_stride + static_cast<size_t>(h) * x_head_stride + I;
      for (int e = tx; e < tail; e += kHpOutputs) store_f(out, out_dtype, ob + O + e, load_f(x, x_dtype, xb + e));
    }
  }
}

// A thread per (request, channel) walks the request's tokens in order; the loads of eight tokens are asked for
// together, the recurrence itself is one multiply-add a token.
constexpr int kScanAhead = 8;
__global__ __launch_bounds__(kWave) void rglru_scan_kernel(
    const float* __restrict__ u, const float* __restrict__ gates, int block, const void* __restrict__ r_bias,
    const void* __restrict__ i_bias, const void* __restrict__ lam, int vec_dtype, float c_mult,
    const void* __restrict__ y, int y_dtype, int64_t y_stride, const void* __restrict__ y_bias,
    float* __restrict__ state, int64_t state_stride, const int* __restrict__ seq_meta, void* __restrict__ out,
    int out_dtype, int C) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int c = blockIdx.x * kWave + threadIdx.x;
  if (c >= C || count <= 0) return;
  const int gcol = (c / block) * 2 * block + c % block;   // the channel's r input; its i input lies `block` further
  const float br = load_f(r_bias, vec_dtype, c), bi = load_f(i_bias, vec_dtype, c);
  const float by = y_bias != nullptr ? load_f(y_bias, vec_dtype, c) : 0.f;
  const float lm = load_f(lam, vec_dtype, c);
  const float sp = lm > 30.f ? lm : log1pf(expf(lm));
  float S = state[static_cast<size_t>(slot) * state_stride + c];
  for (int j0 = 0; j0 < count; j0 += kScanAhead) {
    float uv[kScanAhead], gr[kScanAhead], gi[kScanAhead], yv[kScanAhead];
#pragma unroll
    for (int k = 0; k < kScanAhead; ++k) {
      const int j = j0 + k < count ? j0 + k : count - 1;
      const size_t t = static_cast<size_t>(first + j);
      uv[k] = u[t * C + c];
      gr[k] = gates[t * 2 * C + gcol];
      gi[k] = gates[t * 2 * C + gcol + block];
      yv[k] = load_f(y, y_dtype, t * y_stride + c);
    }
#pragma unroll
    for (int k = 0; k < kScanAhead; ++k) {
      if (j0 + k >= count) break;
      const float r = 1.f / (1.f + expf(-(gr[k] + br)));
      const float i = 1.f / (1.f + expf(-(gi[k] + bi)));
      const float la = -c_mult * r * sp;                 // log a
      const float a = expf(la);
      const float m = sqrtf(-expm1f(2.f * la));           // sqrt(1 - a^2), without the cancellation near a = 1
      S = fmaf(a, S, m * (i * uv[k]));
      const float z = yv[k] + by;
      const float g = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
      store_f(out, out_dtype, static_cast<size_t>(first + j0 + k) * C + c, S * g);
    }
  }
  state[static_cast<size_t>(slot) * state_stride + c] = S;
}

}  // namespace sa

using namespace sa;

extern "C" int sa_head_product(const void* x, int x_dtype, int64_t x_stride, int64_t x_head_stride, const void* w,
                               int w_dtype, void* out, int out_dtype, int64_t out_stride, int64_t out_head_stride, int T,
                               int H, int I, int O, int tail, const void* gate, int gate_dtype, int64_t gate_stride,
                               hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && H > 0 && I > 0 && O > 0 && tail >= 0 && x != nullptr && w != nullptr && out != nullptr,
             "head_product: bad sizes T=%d H=%d I=%d O=%d tail=%d", T, H, I, O, tail);
  SA_REQUIRE(x_head_stride >= I + tail && out_head_stride >= O + tail &&
                 x_stride >= static_cast<int64_t>(H - 1) * x_head_stride + I + tail &&
                 out_stride >= static_cast<int64_t>(H - 1) * out_head_stride + O + tail,
             "head_product: a stride is below what %d heads of %d inputs and %d outputs need", H, I + tail, O + tail);
  SA_REQUIRE(gate == nullptr || gate_stride >= H, "head_product: the gates' row stride is below the heads");
  const int tiles = (T + kHpTokens - 1) / kHpTokens, cols = (O + kHpOutputs - 1) / kHpOutputs;
  SA_REQUIRE(H <= 65535 && cols <= 65535, "head_product: too many heads or outputs");
  head_product_kernel<<<dim3(tiles, H, cols), 256, 0, stream>>>(x, x_dtype, x_stride, x_head_stride, w, w_dtype, out,
                                                                out_dtype, out_stride, out_head_stride, T, I, O, tail,
                                                                gate, gate_dtype, gate_stride);
  return check_launch("head_product");
}

extern "C" int sa_rglru_scan(const float* u, const float* gates, int block, const void* r_bias, const void* i_bias,
                             const void* lam, int vec_dtype, float c, const void* y, int y_dtype, int64_t y_stride,
                             const void* y_bias, float* state, int64_t state_stride, const int* seq_meta, int num_seqs,
                             void* out, int out_dtype, int C, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && C > 0 && block > 0 && C % block == 0, "rglru_scan: bad sizes S=%d C=%d block=%d", num_seqs, C,
             block);
  SA_REQUIRE(u != nullptr && gates != nullptr && r_bias != nullptr && i_bias != nullptr && lam != nullptr &&
                 y != nullptr && state != nullptr && seq_meta != nullptr && out != nullptr,
             "rglru_scan: a null pointer");
  SA_REQUIRE(y_stride >= C && state_stride >= C, "rglru_scan: a stride is below the %d channels", C);
  SA_REQUIRE(num_seqs <= 65535, "rglru_scan: too many requests");
  rglru_scan_kernel<<<dim3((C + kWave - 1) / kWave, num_seqs), kWave, 0, stream>>>(
      u, gates, block, r_bias, i_bias, lam, vec_dtype, c, y, y_dtype, y_stride, y_bias, state, state_stride, seq_meta,
      out, out_dtype, C);
  return check_launch("rglru_scan");
}
