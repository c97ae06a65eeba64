// A feed-forward of routed experts over a ragged batch of tokens.
//
//   route_kernel          softmax of the router's logits, the `top` largest scores and their experts
//   sort_kernel           the (token, choice) pairs in the order of their experts, cut into tiles of rows of one expert
//   expert_product_kernel h = act(Wg[e] x) * (Wu[e] x) for every pair, rows in the sorted order; then
//                         y = Wd[e] h, one row per pair (in the pairs' own order)
//   combine_kernel        out[t] = sum_k weight[t, k] y[t, k] + sigmoid(s[t]) * shared[t]
//
// Nothing comes back to the host between them: the tiles are found on the device, and the grid of the expert
// kernels is sized for the most tiles that the pairs can make.  Every pair's row is computed by itself, with sums
// in an order that depends on the sizes alone, so a token's result does not depend on the batch.  Scores are
// 32-bit; the products are bfloat16 on the matrix cores (32-bit accumulation) or 32-bit on the vector unit.
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kRouteSlots = 8;    // experts per lane: up to 512 experts
constexpr int kTileRowsMax = 64;  // rows of a tile: 16 (one MFMA operand) or 64 (four, which share the weights' operands)

// A wave per token.  scores = softmax(logits); `top` times the largest score that is left (of equal ones the lowest
// index); weight = score * scale.
__global__ __launch_bounds__(kWave) void route_kernel(const float* __restrict__ logits, int64_t stride, int E, int top,
                                                      float scale, int* __restrict__ experts,
                                                      float* __restrict__ weights) {
  const int t = blockIdx.x, lane = threadIdx.x;
  float z[kRouteSlots];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < kRouteSlots; ++i) {
    const int e = lane + i * kWave;
    z[i] = e < E ? logits[static_cast<size_t>(t) * stride + e] : -INFINITY;
    mx = fmaxf(mx, z[i]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kRouteSlots; ++i) {
    z[i] = (lane + i * kWave) < E ? expf(z[i] - mx) : -1.f;   // (a score is never negative: -1 marks what is taken or absent)
    sum += z[i] > 0.f ? z[i] : 0.f;
  }
  sum = wave_sum(sum);
  for (int r = 0; r < top; ++r) {
    float best = -1.f;
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i) best = fmaxf(best, z[i]);
    best = wave_max(best);
    float mine = 1e9f;
#pragma unroll
    for (int i = kRouteSlots - 1; i >= 0; --i)
      if (z[i] == best) mine = static_cast<float>(lane + i * kWave);
    const float first = -wave_max(-mine);
    const int e = static_cast<int>(first);
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i)
      if (lane + i * kWave == e) z[i] = -1.f;
    if (lane == 0) {
      experts[static_cast<size_t>(t) * top + r] = e;
      weights[static_cast<size_t>(t) * top + r] = best / sum * scale;
    }
  }
}

// A wave per token, for routers whose scores are sigmoids of the logits.  The choice is made by score + correction[e]
// (correction null: by the score); the experts form `groups` equal groups of neighbours, a group's score is the sum of
// its two largest choice scores (of its only one, in groups of one), and only experts of the `keep` groups with the
// largest scores can be chosen (of equal ones the lowest index, for groups and for experts).  weight = score * scale,
// without the correction and not renormalized.  Choice scores can be negative: what is taken or shut out is -inf.
__global__ __launch_bounds__(kWave) void route_choice_kernel(const float* __restrict__ logits, int64_t stride, int E,
                                                             int top, float scale, const void* __restrict__ correction,
                                                             int corr_dtype, int groups, int keep,
                                                             int* __restrict__ experts, float* __restrict__ weights) {
  __shared__ float choice_s[kRouteSlots * kWave];
  __shared__ float group_s[kRouteSlots * kWave];
  const int t = blockIdx.x, lane = threadIdx.x;
  float s[kRouteSlots], c[kRouteSlots];
#pragma unroll
  for (int i = 0; i < kRouteSlots; ++i) {
    const int e = lane + i * kWave;
    s[i] = 0.f;
    c[i] = -INFINITY;
    if (e < E) {
      s[i] = 1.f / (1.f + expf(-logits[static_cast<size_t>(t) * stride + e]));
      c[i] = correction != nullptr ? s[i] + load_f(correction, corr_dtype, e) : s[i];
      choice_s[e] = c[i];
    }
  }
  if (groups > 1) {
    __syncthreads();
    const int per = E / groups;
    for (int g = lane; g < groups; g += kWave) {
      float a = -INFINITY, b = -INFINITY;   // the two largest of the group
      for (int k = 0; k < per; ++k) {
        const float v = choice_s[g * per + k];
        if (v > a) {
          b = a;
          a = v;
        } else if (v > b) {
          b = v;
        }
      }
      group_s[g] = per > 1 ? a + b : a;
    }
    __syncthreads();
    // the `keep` best groups, one after the other; lane 0 marks them by sign in LDS
    for (int r = 0; r < keep; ++r) {
      float best = -INFINITY;
      for (int g = lane; g < groups; g += kWave) best = fmaxf(best, group_s[g]);
      best = wave_max(best);
      float mine = 1e9f;
      for (int g = lane; g < groups; g += kWave)
        if (group_s[g] == best && static_cast<float>(g) < mine) mine = static_cast<float>(g);
      const int g_best = static_cast<int>(-wave_max(-mine));
      __syncthreads();
      if (lane == 0) group_s[g_best] = -INFINITY;   // taken: -inf marks a group that stays
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i) {
      const int e = lane + i * kWave;
      if (e < E && group_s[e / per] != -INFINITY) c[i] = -INFINITY;
    }
  }
  for (int r = 0; r < top; ++r) {
    float best = -INFINITY;
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i) best = fmaxf(best, c[i]);
    best = wave_max(best);
    float mine = 1e9f;
#pragma unroll
    for (int i = kRouteSlots - 1; i >= 0; --i)
      if (c[i] == best && lane + i * kWave < E) mine = static_cast<float>(lane + i * kWave);
    const int e = static_cast<int>(-wave_max(-mine));
    float w = 0.f;
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i)
      if (lane + i * kWave == e) {
        c[i] = -INFINITY;
        w = s[i];
      }
    w = wave_sum(w);   // (one lane holds it, the others 0)
    if (lane == 0) {
      experts[static_cast<size_t>(t) * top + r] = e;
      weights[static_cast<size_t>(t) * top + r] = w * scale;
    }
  }
}

// One workgroup.  plan: [0] number of tiles; [1 .. 1 + 2 * max_tiles): per tile its expert and its first row in the
// sorted order with the number of its rows packed as first * 128 + rows.  sorted [P]: pair indices by expert.
__global__ __launch_bounds__(1024) void sort_kernel(const int* __restrict__ experts, int P, int E,
                                                    int* __restrict__ sorted, int* __restrict__ plan, int max_tiles,
                                                    int kTileRows) {
  extern __shared__ int lds[];   // counts [E], offsets [E + 1], tile offsets [E + 1], cursors [E]
  int* counts = lds;
  int* offsets = lds + E;
  int* tiles = offsets + E + 1;
  int* cursor = tiles + E + 1;
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&counts[experts[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = at;
      tiles[e] = nt;
      at += counts[e];
      nt += (counts[e] + kTileRows - 1) / kTileRows;
    }
    offsets[E] = at;
    tiles[E] = nt;
    plan[0] = nt < max_tiles ? nt : max_tiles;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    cursor[e] = 0;
    for (int i = 0; tiles[e] + i < tiles[e + 1]; ++i) {
      const int n = tiles[e] + i;
      if (n >= max_tiles) break;
      const int rows = counts[e] - i * kTileRows < kTileRows ? counts[e] - i * kTileRows : kTileRows;
      plan[1 + 2 * n] = e;
      plan[2 + 2 * n] = (offsets[e] + i * kTileRows) * 128 + rows;
    }
  }
  __syncthreads();
  // (the order of an expert's rows among themselves is whatever the atomics give: every row is computed by itself)
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = experts[p];
    sorted[offsets[e] + atomicAdd(&cursor[e], 1)] = p;
  }
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }

// h[row, f] = act(x[token] . Wg[e, f]) * (x[token] . Wu[e, f]); GATED false: y[pair, n] = h[row] . Wd[e, n].
// A workgroup of four waves takes one tile of rows and 64 columns (a wave 16 of them, for all RT sub-tiles of 16 rows).
// bfloat16: the weights are tiled ([E][N / 16][K / 32][64][8], see the product kernels), a wave's operands are one
// 16-byte load a lane (rows that are not 16-byte aligned are read element by element); 32-bit: row-major weights
// [E][N][K], a lane per (row, column) of the tile in turn.
template <typename T, bool GATED, int RT>
__global__ __launch_bounds__(256) void expert_product_kernel(
    const T* __restrict__ a, int64_t a_stride, int a_by_token, int top, const T* __restrict__ w1, const T* __restrict__ w2,
    int N, int K, const int* __restrict__ sorted, const int* __restrict__ plan, int act, void* __restrict__ out,
    int64_t out_stride, int out_by_pair, int activate) {
  // activate (without a second weight): out[row] = act(a . w1[e]^T) in a's type instead of the 32-bit product
  const int tile = blockIdx.x;
  if (tile >= plan[0]) return;
  const int e = plan[1 + 2 * tile], packed = plan[2 + 2 * tile];
  const int row0 = packed / 128, rows = packed % 128;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int n0 = (blockIdx.y * 4 + wave) * 16;
  if (n0 >= N) return;
  if constexpr (sizeof(T) == 2) {
    const int Nt = (N + 15) / 16, Kt = (K + 31) / 32;
    const int r = lane % 16, kq = lane / 16;
    const bool aligned = a_stride % 8 == 0;
    const T* arow[RT];
    int pairs[RT];
#pragma unroll
    for (int s = 0; s < RT; ++s) {
      const int rr = s * 16 + r < rows ? s * 16 + r : rows - 1;
      pairs[s] = sorted[row0 + rr];
      arow[s] = a + static_cast<size_t>(a_by_token ? pairs[s] / top : row0 + rr) * a_stride;
    }
    const size_t wbase = (static_cast<size_t>(e) * Nt + n0 / 16) * Kt;
    const bf16* g = reinterpret_cast<const bf16*>(w1) + wbase * 512 + lane * 8;
    const bf16* u = GATED ? reinterpret_cast<const bf16*>(w2) + wbase * 512 + lane * 8 : nullptr;
    floatx4 accg[RT], accu[RT];
#pragma unroll
    for (int s = 0; s < RT; ++s) accg[s] = accu[s] = floatx4{0.f, 0.f, 0.f, 0.f};
    // Whole k tiles of aligned rows, four at a time: their loads are all asked for before the first product (few
    // waves run on a SIMD here, so a wave covers its own waits), the products in the order of k.
    int kt = 0;
    if (aligned && RT == 1) {
      const bf16* src = reinterpret_cast<const bf16*>(arow[0]) + kq * 8;
      constexpr int kAhead = 4;
      for (; kt + kAhead <= K / 32; kt += kAhead) {
        bf16x8 gv[kAhead], uv[kAhead], av[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
          gv[i] = load8(g + static_cast<size_t>(kt + i) * 512);
          if constexpr (GATED) uv[i] = load8(u + static_cast<size_t>(kt + i) * 512);
          av[i] = load8(src + (kt + i) * 32);
        }
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
          accg[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gv[i], av[i], accg[0], 0, 0, 0);
          if constexpr (GATED) accu[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uv[i], av[i], accu[0], 0, 0, 0);
        }
      }
    }
    for (; kt < Kt; ++kt) {
      const int k = kt * 32 + kq * 8;
      const bf16x8 gv = load8(g + static_cast<size_t>(kt) * 512);
      bf16x8 uv = gv;
      if constexpr (GATED) uv = load8(u + static_cast<size_t>(kt) * 512);
#pragma unroll
      for (int s = 0; s < RT; ++s) {
        if (s * 16 >= rows) break;   // (uniform: the tile's rows are)
        const bf16* src = reinterpret_cast<const bf16*>(arow[s]);
        bf16x8 av;
        if (aligned && k + 8 <= K) {
          av = load8(src + k);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            av[i] = k + i < K ? __builtin_bit_cast(__bf16, src[k + i]) : static_cast<__bf16>(0.f);
        }
        // the weights' rows are the product's columns: C^T = W . A^T, a lane holds four columns of the output of
        // one token
        accg[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gv, av, accg[s], 0, 0, 0);
        if constexpr (GATED) accu[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uv, av, accu[s], 0, 0, 0);
      }
    }
    // lane: token s * 16 + lane % 16, output columns n0 + kq * 4 + i
#pragma unroll
    for (int s = 0; s < RT; ++s) {
      if (s * 16 + r >= rows) continue;
      const size_t orow = static_cast<size_t>(out_by_pair ? pairs[s] : row0 + s * 16 + r) * out_stride;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + kq * 4 + i;
        if (n >= N) continue;
        if constexpr (GATED) {
          const float v = gated_activation(act, to_float(float_to_bf16(accg[s][i]))) * to_float(float_to_bf16(accu[s][i]));
          static_cast<bf16*>(out)[orow + n] = float_to_bf16(v);
        } else if (activate) {
          static_cast<bf16*>(out)[orow + n] = float_to_bf16(gated_activation(act, to_float(float_to_bf16(accg[s][i]))));
        } else {
          static_cast<float*>(out)[orow + n] = accg[s][i];
        }
      }
    }
  } else {
    // 32-bit: 16 columns x the rows of the tile over the wave's 64 lanes, four rows at a time
    const int c = lane % 16, n = n0 + c;
    for (int r = lane / 16; r < rows; r += 4) {
      const int pair = sorted[row0 + r];
      const T* arow = a + static_cast<size_t>(a_by_token ? pair / top : row0 + r) * a_stride;
      if (n >= N) continue;
      const T* g = w1 + (static_cast<size_t>(e) * N + n) * K;
      float sg = 0.f, su = 0.f;
      for (int k = 0; k < K; ++k) sg = fmaf(to_float(arow[k]), to_float(g[k]), sg);
      const size_t orow = static_cast<size_t>(out_by_pair ? pair : row0 + r) * out_stride;
      if constexpr (GATED) {
        const T* u = w2 + (static_cast<size_t>(e) * N + n) * K;
        for (int k = 0; k < K; ++k) su = fmaf(to_float(arow[k]), to_float(u[k]), su);
        static_cast<float*>(out)[orow + n] = gated_activation_exact(act, sg) * su;
      } else {
        static_cast<float*>(out)[orow + n] = activate ? gated_activation_exact(act, sg) : sg;
      }
    }
  }
}

// The same products for tiles of 64 rows (steps that bring an expert many rows), bfloat16: a workgroup takes the tile's
// rows and 128 columns, a wave 32 of them (two column tiles) for all four sub-tiles of 16 rows.  The rows' operands of
// 64 columns of K at a time go through LDS in operand order (every wave needs all of them: read from memory once
// instead of four times), asked for a chunk ahead into registers; the weights' operands come straight from their
// tiles.  A row's sums are those of the kernel above, in its order.
constexpr int kChunkK = 64;
template <bool GATED>
__global__ __launch_bounds__(256) void expert_product_rows64_kernel(
    const bf16* __restrict__ a, int64_t a_stride, int a_by_token, int top, const bf16* __restrict__ w1,
    const bf16* __restrict__ w2, int N, int K, const int* __restrict__ sorted, const int* __restrict__ plan, int act,
    void* __restrict__ out, int64_t out_stride, int out_by_pair, int activate) {
  __shared__ bf16x8 rows_lds[4][kChunkK / 32][kWave];   // [sub-tile of 16 rows][k tile of the chunk][lane]
  __shared__ int pair_of[kTileRowsMax];
  const int tile = blockIdx.x;
  if (tile >= plan[0]) return;
  const int e = plan[1 + 2 * tile], packed = plan[2 + 2 * tile];
  const int row0 = packed / 128, rows = packed % 128;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int r = lane % 16, kq = lane / 16;
  const int n0 = (blockIdx.y * 4 + wave) * 32;
  const bool mine = n0 < N;   // (a wave without columns still stages rows and meets the barriers)
  if (tid < kTileRowsMax) pair_of[tid] = sorted[row0 + (tid < rows ? tid : rows - 1)];
  __syncthreads();
  const bool aligned = a_stride % 8 == 0;
  // staging: this thread's two pieces of 8 elements of a chunk, and where they go
  const bf16* src[2];
  int koff[2];
  bf16x8* dst[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int combo = wave + 4 * i, sub = combo / 2, kt = combo % 2;
    const int row = sub * 16 + r, rr = row < rows ? row : rows - 1;
    src[i] = a + static_cast<size_t>(a_by_token ? pair_of[rr] / top : row0 + rr) * a_stride;
    koff[i] = kt * 32 + kq * 8;
    dst[i] = &rows_lds[sub][kt][lane];
  }
  bf16x8 staged[2];
  auto fetch = [&](int c) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int k = c * kChunkK + koff[i];
      if (aligned && k + 8 <= K) {
        staged[i] = load8(src[i] + k);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          staged[i][j] = k + j < K ? __builtin_bit_cast(__bf16, src[i][k + j]) : static_cast<__bf16>(0.f);
      }
    }
  };
  const int Nt = (N + 15) / 16, Kt = (K + 31) / 32;
  const int nsub = (rows + 15) / 16;
  floatx4 accg[4][2], accu[4][2];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int j = 0; j < 2; ++j) accg[s][j] = accu[s][j] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int chunks = (K + kChunkK - 1) / kChunkK;
  fetch(0);
  for (int c = 0; c < chunks; ++c) {
    __syncthreads();   // the chunk before has been read
    *dst[0] = staged[0];
    *dst[1] = staged[1];
    __syncthreads();
    if (c + 1 < chunks) fetch(c + 1);
    if (!mine) continue;
#pragma unroll
    for (int kt = 0; kt < kChunkK / 32; ++kt) {
      const int ktg = c * (kChunkK / 32) + kt;
      if (ktg >= Kt) break;
      bf16x8 gv[2], uv[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int nt = n0 / 16 + j < Nt ? n0 / 16 + j : Nt - 1;
        const size_t at = ((static_cast<size_t>(e) * Nt + nt) * Kt + ktg) * 512 + lane * 8;
        gv[j] = load8(w1 + at);
        if constexpr (GATED) uv[j] = load8(w2 + at);
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (s >= nsub) break;
        const bf16x8 av = rows_lds[s][kt][lane];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          accg[s][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(gv[j], av, accg[s][j], 0, 0, 0);
          if constexpr (GATED) accu[s][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uv[j], av, accu[s][j], 0, 0, 0);
        }
      }
    }
  }
  if (!mine) return;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int row = s * 16 + r;
    if (row >= rows) continue;
    const size_t orow = static_cast<size_t>(out_by_pair ? pair_of[row] : row0 + row) * out_stride;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + j * 16 + kq * 4 + i;
        if (n >= N) continue;
        if constexpr (GATED) {
          const float v = gated_activation(act, to_float(float_to_bf16(accg[s][j][i]))) * to_float(float_to_bf16(accu[s][j][i]));
          static_cast<bf16*>(out)[orow + n] = float_to_bf16(v);
        } else if (activate) {
          static_cast<bf16*>(out)[orow + n] =
              float_to_bf16(gated_activation(act, to_float(float_to_bf16(accg[s][j][i]))));
        } else {
          static_cast<float*>(out)[orow + n] = accg[s][j][i];
        }
      }
  }
}

// out[t, d] = sum_k weights[t, k] * y[t * top + k, d] (in the order of k) + sigmoid(gate[t]) * shared[t, d].
__global__ void combine_kernel(const float* __restrict__ y, const float* __restrict__ weights, int top,
                               const void* __restrict__ shared, int shared_dtype, int64_t shared_stride,
                               const float* __restrict__ gate, int64_t gate_stride, void* __restrict__ out, int out_dtype,
                               int64_t out_stride, int D) {
  const int t = blockIdx.y, d = blockIdx.x * blockDim.x + threadIdx.x;
  if (d >= D) return;
  float v = 0.f;
  for (int k = 0; k < top; ++k)
    v = fmaf(weights[static_cast<size_t>(t) * top + k], y[(static_cast<size_t>(t) * top + k) * D + d], v);
  if (shared != nullptr) {
    const float s = load_f(shared, shared_dtype, static_cast<size_t>(t) * shared_stride + d);
    v += gate != nullptr ? s / (1.f + expf(-gate[static_cast<size_t>(t) * gate_stride])) : s;
  }
  store_f(out, out_dtype, static_cast<size_t>(t) * out_stride + d, v);
}

}  // namespace sa

using namespace sa;

extern "C" int sa_route(const float* logits, int64_t stride, int T, int E, int top, float scale, int* experts,
                        float* weights, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && E > 0 && E <= kRouteSlots * kWave && top > 0 && top <= E && stride >= E,
             "route: bad sizes T=%d E=%d top=%d (at most %d experts)", T, E, top, kRouteSlots * kWave);
  SA_REQUIRE(logits != nullptr && experts != nullptr && weights != nullptr, "route: a null pointer");
  route_kernel<<<T, kWave, 0, stream>>>(logits, stride, E, top, scale, experts, weights);
  return check_launch("route");
}

extern "C" int sa_route_choice(const float* logits, int64_t stride, int T, int E, int top, float scale,
                               const void* correction, int corr_dtype, int groups, int keep, int* experts,
                               float* weights, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && E > 0 && E <= kRouteSlots * kWave && top > 0 && stride >= E,
             "route_choice: bad sizes T=%d E=%d top=%d (at most %d experts)", T, E, top, kRouteSlots * kWave);
  SA_REQUIRE(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups,
             "route_choice: %d experts in %d groups of which %d stay", E, groups, keep);
  SA_REQUIRE(top <= keep * (E / groups), "route_choice: %d experts cannot be chosen from %d groups of %d", top, keep,
             E / groups);
  SA_REQUIRE(correction == nullptr || corr_dtype == kF32 || corr_dtype == kBF16, "route_choice: unknown dtype %d",
             corr_dtype);
  route_choice_kernel<<<T, kWave, 0, stream>>>(logits, stride, E, top, scale, correction, corr_dtype, groups, keep,
                                               experts, weights);
  return check_launch("route_choice");
}

extern "C" int sa_expert_tiles_max(int P, int E, int tile_rows) {
  return (P + tile_rows - 1) / tile_rows + (E < P ? E : P);
}

extern "C" int sa_expert_sort(const int* experts, int P, int E, int tile_rows, int* sorted, int* plan, int plan_words,
                              hipStream_t stream) {
  if (P == 0) return 0;
  SA_REQUIRE(tile_rows == 16 || tile_rows == kTileRowsMax, "expert_sort: tiles of 16 or %d rows", kTileRowsMax);
  const int max_tiles = sa_expert_tiles_max(P, E, tile_rows);
  SA_REQUIRE(P > 0 && E > 0 && E <= 4096 && P < (1 << 26), "expert_sort: bad sizes P=%d E=%d", P, E);
  SA_REQUIRE(plan_words >= 1 + 2 * max_tiles, "expert_sort: the plan needs %d words", 1 + 2 * max_tiles);
  SA_REQUIRE(experts != nullptr && sorted != nullptr && plan != nullptr, "expert_sort: a null pointer");
  const int threads = P >= 1024 ? 1024 : ((P + kWave - 1) / kWave) * kWave;
  sort_kernel<<<1, threads, (4 * E + 2) * sizeof(int), stream>>>(experts, P, E, sorted, plan, max_tiles, tile_rows);
  return check_launch("expert_sort");
}

extern "C" int sa_expert_product(const void* a, int dtype, int64_t a_stride, int a_by_token, int top, const void* w1,
                                 const void* w2, int N, int K, const int* sorted, const int* plan, int P, int E,
                                 int tile_rows, int act, void* out, int64_t out_stride, int out_by_pair, int activate,
                                 hipStream_t stream) {
  if (P == 0) return 0;
  SA_REQUIRE(!activate || w2 == nullptr, "expert_product: a gated product has its activation already");
  SA_REQUIRE(P > 0 && E > 0 && N > 0 && K > 0 && top > 0 && a_stride >= K && out_stride >= N,
             "expert_product: bad sizes P=%d E=%d N=%d K=%d", P, E, N, K);
  SA_REQUIRE(a != nullptr && w1 != nullptr && sorted != nullptr && plan != nullptr && out != nullptr,
             "expert_product: a null pointer");
  SA_REQUIRE(act >= 0 && act < kNumActivations, "expert_product: unknown activation %d", act);
  SA_REQUIRE(dtype == kF32 || dtype == kBF16, "expert_product: unknown dtype %d", dtype);
  SA_REQUIRE(tile_rows == 16 || tile_rows == kTileRowsMax, "expert_product: tiles of 16 or %d rows", kTileRowsMax);
  const dim3 grid(sa_expert_tiles_max(P, E, tile_rows), (N + 63) / 64);
  SA_REQUIRE(grid.y <= 65535, "expert_product: too many columns");
  const bool gated = w2 != nullptr;
#define SA_EXPERT(T, G, RT)                                                                                            \
  expert_product_kernel<T, G, RT><<<grid, 256, 0, stream>>>(static_cast<const T*>(a), a_stride, a_by_token, top,        \
                                                             static_cast<const T*>(w1), static_cast<const T*>(w2), N,  \
                                                             K, sorted, plan, act, out, out_stride, out_by_pair,       \
                                                             activate)
  if (dtype == kBF16) {
    if (tile_rows == 16) {
      if (gated) SA_EXPERT(bf16, true, 1);
      else SA_EXPERT(bf16, false, 1);
    } else {
      const dim3 wide(grid.x, (N + 127) / 128);
      if (gated)
        expert_product_rows64_kernel<true><<<wide, 256, 0, stream>>>(
            static_cast<const bf16*>(a), a_stride, a_by_token, top, static_cast<const bf16*>(w1),
            static_cast<const bf16*>(w2), N, K, sorted, plan, act, out, out_stride, out_by_pair, 0);
      else
        expert_product_rows64_kernel<false><<<wide, 256, 0, stream>>>(
            static_cast<const bf16*>(a), a_stride, a_by_token, top, static_cast<const bf16*>(w1), nullptr, N, K, sorted,
            plan, act, out, out_stride, out_by_pair, activate);
    }
  } else {
    if (gated) SA_EXPERT(float, true, 1);
    else SA_EXPERT(float, false, 1);
  }
#undef SA_EXPERT
  return check_launch("expert_product");
}

extern "C" int sa_expert_combine(const float* y, const float* weights, int top, const void* shared, int shared_dtype,
                                 int64_t shared_stride, const float* gate, int64_t gate_stride, void* out, int out_dtype,
                                 int64_t out_stride, int T, int D, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && T <= 65535 && D > 0 && top > 0 && out_stride >= D, "expert_combine: bad sizes T=%d D=%d top=%d", T, D,
             top);
  SA_REQUIRE(y != nullptr && weights != nullptr && out != nullptr, "expert_combine: a null pointer");
  SA_REQUIRE(shared == nullptr || shared_stride >= D, "expert_combine: the shared rows are too short");
  combine_kernel<<<dim3((D + 255) / 256, T), 256, 0, stream>>>(y, weights, top, shared, shared_dtype, shared_stride, gate,
                                                               gate_stride, out, out_dtype, out_stride, D);
  return check_launch("expert_combine");
}
