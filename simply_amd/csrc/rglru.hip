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

constexpr int kHpTokens = 64;   // tokens of a tile
constexpr int kHpOutputs = 64;  // outputs of a tile
constexpr int kHpChunk = 32;    // inputs staged at a time

// A workgroup of 256 threads takes 64 tokens x 64 outputs of one head: thread (ty, tx) sums the outputs 4 tx .. 4 tx + 3
// for the tokens 4 ty .. 4 ty + 3 over the inputs in their order, with the weights' and the rows' chunk of 32 inputs
// in LDS, both with the inputs as the slow index, so that a thread reads four outputs' weights and four tokens'
// inputs as one 16-byte piece each for sixteen multiply-adds.
__global__ __launch_bounds__(256) void head_product_kernel(
    const void* __restrict__ x, int x_dtype, int64_t x_stride, int64_t x_head_stride, const void* __restrict__ w,
    int w_dtype, void* __restrict__ out, int out_dtype, int64_t out_stride, int64_t out_head_stride, int T, int I, int O,
    int tail, const void* __restrict__ gate, int gate_dtype, int64_t gate_stride) {
  // (rows four words longer: a staging write's 32 inputs of one output then fall into 16 banks, and rows stay 16-byte aligned)
  __shared__ __align__(16) float ws[kHpChunk][kHpOutputs + 4];
  __shared__ __align__(16) float xs[kHpChunk][kHpTokens + 4];
  const int t0 = blockIdx.x * kHpTokens, h = blockIdx.y, o0 = blockIdx.z * kHpOutputs;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const size_t wb = static_cast<size_t>(h) * O * I;
  float acc[4][4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[k][j] = 0.f;
  for (int i0 = 0; i0 < I; i0 += kHpChunk) {
    __syncthreads();
    for (int e = tid; e < kHpOutputs * kHpChunk; e += 256) {
      const int o = e / kHpChunk, i = e % kHpChunk;
      ws[i][o] = (o0 + o < O && i0 + i < I) ? load_f(w, w_dtype, wb + static_cast<size_t>(o0 + o) * I + i0 + i) : 0.f;
    }
    for (int e = tid; e < kHpTokens * kHpChunk; e += 256) {
      const int k = e / kHpChunk, i = e % kHpChunk;
      xs[i][k] = (t0 + k < T && i0 + i < I)
                     ? load_f(x, x_dtype, static_cast<size_t>(t0 + k) * x_stride + static_cast<size_t>(h) * x_head_stride + i0 + i)
                     : 0.f;
    }
    __syncthreads();
    const int in = I - i0 < kHpChunk ? I - i0 : kHpChunk;
    for (int i = 0; i < in; ++i) {
      const float4 wv = *reinterpret_cast<const float4*>(&ws[i][4 * tx]);
      const float4 xv = *reinterpret_cast<const float4*>(&xs[i][4 * ty]);
      const float wa[4] = {wv.x, wv.y, wv.z, wv.w}, xa[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
      for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[k][j] = fmaf(xa[k], wa[j], acc[k][j]);
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int t = t0 + 4 * ty + k;
    if (t >= T) continue;
    const size_t ob = static_cast<size_t>(t) * out_stride + static_cast<size_t>(h) * out_head_stride;
    const float gv = gate != nullptr
                         ? 1.f / (1.f + expf(-load_f(gate, gate_dtype, static_cast<size_t>(t) * gate_stride + h)))
                         : 1.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (o0 + 4 * tx + j < O) store_f(out, out_dtype, ob + o0 + 4 * tx + j, acc[k][j] * gv);
    if (blockIdx.z == 0) {
      const size_t xb = static_cast<size_t>(t) * x_stride + static_cast<size_t>(h) * x_head_stride + I;
      for (int e = tx; e < tail; e += 16) store_f(out, out_dtype, ob + O + e, load_f(x, x_dtype, xb + e));
    }
  }
}

// The same product for a handful of tokens (decoding): a wave per (head, output) holds up to kHpFewTokens tokens'
// sums in its lanes, every lane over the inputs lane, lane + 64, ..., and adds the lanes up at the end, so the
// weights are streamed once in contiguous pieces by as many waves as there are outputs.
constexpr int kHpFewTokens = 8;
__global__ __launch_bounds__(256) void head_product_few_kernel(
    const void* __restrict__ x, int x_dtype, int64_t x_stride, int64_t x_head_stride, const void* __restrict__ w,
    int w_dtype, void* __restrict__ out, int out_dtype, int64_t out_stride, int64_t out_head_stride, int T, int I, int O,
    int tail, const void* __restrict__ gate, int gate_dtype, int64_t gate_stride) {
  const int lane = threadIdx.x % kWave, o = blockIdx.x * 4 + threadIdx.x / kWave, h = blockIdx.y;
  const int t0 = blockIdx.z * kHpFewTokens;
  if (o >= O) return;   // (a whole wave)
  const size_t wb = (static_cast<size_t>(h) * O + o) * I;
  float acc[kHpFewTokens];
#pragma unroll
  for (int k = 0; k < kHpFewTokens; ++k) acc[k] = 0.f;
  for (int i = lane; i < I; i += kWave) {
    const float wv = load_f(w, w_dtype, wb + i);
#pragma unroll
    for (int k = 0; k < kHpFewTokens; ++k) {
      const int t = t0 + k < T ? t0 + k : T - 1;
      acc[k] = fmaf(load_f(x, x_dtype, static_cast<size_t>(t) * x_stride + static_cast<size_t>(h) * x_head_stride + i), wv,
                    acc[k]);
    }
  }
#pragma unroll
  for (int k = 0; k < kHpFewTokens; ++k) {
    const float v = wave_sum(acc[k]);
    const int t = t0 + k;
    if (t >= T) continue;
    const size_t ob = static_cast<size_t>(t) * out_stride + static_cast<size_t>(h) * out_head_stride;
    if (lane == 0) {
      const float gv = gate != nullptr
                           ? 1.f / (1.f + expf(-load_f(gate, gate_dtype, static_cast<size_t>(t) * gate_stride + h)))
                           : 1.f;
      store_f(out, out_dtype, ob + o, v * gv);
    }
    if (o == 0) {
      const size_t xb = static_cast<size_t>(t) * x_stride + static_cast<size_t>(h) * x_head_stride + I;
      for (int e = lane; e < tail; e += kWave) store_f(out, out_dtype, ob + O + e, load_f(x, x_dtype, xb + e));
    }
  }
}

// The recurrence of one channel over the tokens [j0, j1) of a request from the state S: the loads of eight tokens are
// asked for together, the recurrence itself is one multiply-add a token.  kOut: results are written; else only the
// state and the product of the decays come back (a segment's summary).
struct ScanArgs {
  const float* u;
  const float* gates;
  int block;
  const void* r_bias;
  const void* i_bias;
  const void* lam;
  int vec_dtype;
  float c_mult;
  const void* y;
  int y_dtype;
  int64_t y_stride;
  const void* y_bias;
  void* out;
  int out_dtype;
  int C;
};
constexpr int kScanAhead = 8;
template <bool kOut>
__device__ __forceinline__ void scan_tokens(const ScanArgs& p, int c, int first, int j0, int j1, float& S, float& A) {
  const int gcol = (c / p.block) * 2 * p.block + c % p.block;   // the channel's r input; its i input lies `block` further
  const float br = load_f(p.r_bias, p.vec_dtype, c), bi = load_f(p.i_bias, p.vec_dtype, c);
  const float by = (kOut && p.y_bias != nullptr) ? load_f(p.y_bias, p.vec_dtype, c) : 0.f;
  const float lm = load_f(p.lam, p.vec_dtype, c);
  const float sp = lm > 30.f ? lm : log1pf(expf(lm));
  const int C = p.C;
  for (int jb = j0; jb < j1; jb += kScanAhead) {
    float uv[kScanAhead], gr[kScanAhead], gi[kScanAhead], yv[kScanAhead];
#pragma unroll
    for (int k = 0; k < kScanAhead; ++k) {
      const int j = jb + k < j1 ? jb + k : j1 - 1;
      const size_t t = static_cast<size_t>(first + j);
      uv[k] = p.u[t * C + c];
      gr[k] = p.gates[t * 2 * C + gcol];
      gi[k] = p.gates[t * 2 * C + gcol + p.block];
      yv[k] = kOut ? load_f(p.y, p.y_dtype, t * p.y_stride + c) : 0.f;
    }
    // decays and inputs of the eight tokens side by side, then the chain of multiply-adds
    float a[kScanAhead], b[kScanAhead];
#pragma unroll
    for (int k = 0; k < kScanAhead; ++k) {
      const float r = 1.f / (1.f + expf(-(gr[k] + br)));
      const float i = 1.f / (1.f + expf(-(gi[k] + bi)));
      const float la = -p.c_mult * r * sp;                  // log a
      a[k] = expf(la);
      b[k] = sqrtf(-expm1f(2.f * la)) * (i * uv[k]);        // sqrt(1 - a^2), without the cancellation near a = 1
    }
#pragma unroll
    for (int k = 0; k < kScanAhead; ++k) {
      if (jb + k >= j1) break;
      S = fmaf(a[k], S, b[k]);
      if (kOut) {
        const float z = yv[k] + by;
        const float g = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
        store_f(p.out, p.out_dtype, static_cast<size_t>(first + jb + k) * C + c, S * g);
      } else {
        A *= a[k];
      }
    }
  }
}

// A thread per (request, channel) walks the request's tokens in order: steps of few tokens (decoding).
__global__ __launch_bounds__(kWave) void rglru_scan_kernel(ScanArgs p, float* __restrict__ state, int64_t state_stride,
                                                           const int* __restrict__ seq_meta) {
  const int* meta = seq_meta + 4 * blockIdx.y;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int c = blockIdx.x * kWave + threadIdx.x;
  if (c >= p.C || count <= 0) return;
  float S = state[static_cast<size_t>(slot) * state_stride + c], A = 1.f;
  scan_tokens<true>(p, c, first, 0, count, S, A);
  state[static_cast<size_t>(slot) * state_stride + c] = S;
}

// Long portions: a request's tokens are cut into segments of `seg` tokens (from the step's first token) that run side
// by side.  First every segment but the last is summarised from a state of zero: S' = A S + B with A the product of its
// decays (rglru_segments_kernel; segment 0's thread also saves the request's state, which the second kernel overwrites
// while others still want it).  Then every segment starts from the state that the summaries before it give, applied
// in their order, and writes its results; the last one leaves the state (rglru_scan_segments_kernel).
// summaries: [request][segment][A | B][C]; start: [request][C].
__global__ __launch_bounds__(kWave) void rglru_segments_kernel(ScanArgs p, const float* __restrict__ state,
                                                               int64_t state_stride, const int* __restrict__ seq_meta,
                                                               int seg, int max_segs, float* __restrict__ summaries,
                                                               float* __restrict__ start) {
  const int* meta = seq_meta + 4 * blockIdx.z;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int c = blockIdx.x * kWave + threadIdx.x, j = blockIdx.y;
  if (c >= p.C || count <= 0) return;
  if (j == 0) start[static_cast<size_t>(blockIdx.z) * p.C + c] = state[static_cast<size_t>(slot) * state_stride + c];
  if ((j + 1) * seg >= count) return;   // the last segment (and what lies beyond): nobody starts behind it
  float S = 0.f, A = 1.f;
  scan_tokens<false>(p, c, first, j * seg, (j + 1) * seg, S, A);
  float* sum = summaries + (static_cast<size_t>(blockIdx.z) * max_segs + j) * 2 * p.C;
  sum[c] = A;
  sum[p.C + c] = S;
}

__global__ __launch_bounds__(kWave) void rglru_scan_segments_kernel(ScanArgs p, float* __restrict__ state,
                                                                    int64_t state_stride,
                                                                    const int* __restrict__ seq_meta, int seg,
                                                                    int max_segs, const float* __restrict__ summaries,
                                                                    const float* __restrict__ start) {
  const int* meta = seq_meta + 4 * blockIdx.z;
  const int slot = meta[0], first = meta[1], count = meta[2];
  const int c = blockIdx.x * kWave + threadIdx.x, j = blockIdx.y;
  if (c >= p.C || j * seg >= count) return;
  float S = start[static_cast<size_t>(blockIdx.z) * p.C + c], A = 1.f;
  const float* sum = summaries + static_cast<size_t>(blockIdx.z) * max_segs * 2 * p.C;
  for (int jj = 0; jj < j; ++jj) S = fmaf(sum[static_cast<size_t>(jj) * 2 * p.C + c], S, sum[static_cast<size_t>(jj) * 2 * p.C + p.C + c]);
  const int j1 = (j + 1) * seg < count ? (j + 1) * seg : count;
  scan_tokens<true>(p, c, first, j * seg, j1, S, A);
  if (j1 == count) state[static_cast<size_t>(slot) * state_stride + c] = S;
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
  if (T <= 2 * kHpFewTokens && (O + 3) / 4 <= 65535) {
    head_product_few_kernel<<<dim3((O + 3) / 4, H, (T + kHpFewTokens - 1) / kHpFewTokens), 256, 0, stream>>>(
        x, x_dtype, x_stride, x_head_stride, w, w_dtype, out, out_dtype, out_stride, out_head_stride, T, I, O, tail, gate,
        gate_dtype, gate_stride);
    return check_launch("head_product_few");
  }
  head_product_kernel<<<dim3(tiles, H, cols), 256, 0, stream>>>(x, x_dtype, x_stride, x_head_stride, w, w_dtype, out,
                                                                out_dtype, out_stride, out_head_stride, T, I, O, tail,
                                                                gate, gate_dtype, gate_stride);
  return check_launch("head_product");
}

extern "C" int sa_rglru_scan(const float* u, const float* gates, int block, const void* r_bias, const void* i_bias,
                             const void* lam, int vec_dtype, float c, const void* y, int y_dtype, int64_t y_stride,
                             const void* y_bias, float* state, int64_t state_stride, const int* seq_meta, int num_seqs,
                             int max_q_len, float* scratch, size_t scratch_floats, void* out, int out_dtype, int C,
                             hipStream_t stream) {
  if (num_seqs == 0) return 0;
  SA_REQUIRE(num_seqs > 0 && C > 0 && block > 0 && C % block == 0 && max_q_len > 0,
             "rglru_scan: bad sizes S=%d C=%d block=%d q=%d", num_seqs, C, block, max_q_len);
  SA_REQUIRE(u != nullptr && gates != nullptr && r_bias != nullptr && i_bias != nullptr && lam != nullptr &&
                 y != nullptr && state != nullptr && seq_meta != nullptr && out != nullptr,
             "rglru_scan: a null pointer");
  SA_REQUIRE(y_stride >= C && state_stride >= C, "rglru_scan: a stride is below the %d channels", C);
  SA_REQUIRE(num_seqs <= 65535, "rglru_scan: too many requests");
  const ScanArgs p{u, gates, block, r_bias, i_bias, lam, vec_dtype, c, y, y_dtype, y_stride, y_bias, out, out_dtype, C};
  const int cb = (C + kWave - 1) / kWave;
  // segments of 64 tokens (longer ones for very long portions); steps of up to two segments run as one
  int seg = 64;
  while ((max_q_len + seg - 1) / seg > 1024) seg *= 2;
  const int segs = (max_q_len + seg - 1) / seg;
  const size_t need = static_cast<size_t>(num_seqs) * (static_cast<size_t>(segs) * 2 + 1) * C;
  if (segs <= 2 || scratch == nullptr || scratch_floats < need) {
    rglru_scan_kernel<<<dim3(cb, num_seqs), kWave, 0, stream>>>(p, state, state_stride, seq_meta);
    return check_launch("rglru_scan");
  }
  float* start = scratch;
  float* summaries = scratch + static_cast<size_t>(num_seqs) * C;
  rglru_segments_kernel<<<dim3(cb, segs, num_seqs), kWave, 0, stream>>>(p, state, state_stride, seq_meta, seg, segs,
                                                                        summaries, start);
  if (check_launch("rglru_segments")) return 1;
  rglru_scan_segments_kernel<<<dim3(cb, segs, num_seqs), kWave, 0, stream>>>(p, state, state_stride, seq_meta, seg, segs,
                                                                             summaries, start);
  return check_launch("rglru_scan_segments");
}
