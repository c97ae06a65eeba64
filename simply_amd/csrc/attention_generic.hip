// Paged attention for every size and both element types: one workgroup per
// (query token, key/value head), all arithmetic in 32-bit on the vector ALU.
//
// A query at absolute position p of its request sees the keys [lo, p] with
// lo = max(0, p - window + 1) for a windowed layer and 0 otherwise; the keys of
// this step have been written to the pages before the launch.  Keys are taken
// in chunks of 64 aligned to absolute positions, in increasing order, with a
// running maximum, sum and output (online softmax).  The order of every sum is
// fixed by p alone, so the result for a token does not depend on how the tokens
// were cut into steps, on what else is in the batch, or on which pages hold the
// keys.
//
// Scores -> cap -> mask -> softmax -> values as in simply/model_lib.py:611-638
// and simply/kernels/ragged_paged_attention.py:222-249; query head h reads
// key/value head h / G (simply/kernels/ragged_paged_attention.py:214-215).
//
// Options for mixers that are not plain softmax attention:
//   slopes           a bias by distance: slopes[h] * (query position - key position) is taken off head h's scaled scores
//                    (with sinks, below the entry points: one more term exp(sinks[h]) in the sum, without a value).
//   maps (M > 1)     every query head has M score maps over the same values: its query row is M vectors of hd
//                    entries, a key row M * hd entries (one key vector per map); each map is a softmax of its own.
//                    To the kernel a map is one more query head ("virtual head" g = head * M + map).
//   differential     (M == 2) a head's result is (a_1 - lambda a_2) / sqrt(mean(.^2) + eps) * mult over its values,
//                    with a_m the maps' results; otherwise every map's result is written, map by map.
//   values_in_keys   there are no value pages: a key's value is the first hd_v entries of its key row (a latent that
//                    is scored as it is and read as it is).
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kChunk = 64;     // keys per chunk
constexpr int kThreads = 256;  // 4 waves
constexpr int kMaxDimsPerThread = 2;  // head sizes up to 512

struct AttentionOptions {
  int values_in_keys = 0;
  int differential = 0;
  float lambda = 0.f, eps = 0.f, mult = 1.f;
};

// G: query vectors per key/value head (heads times maps); hd: entries of one of them.
template <typename T, int M>
__global__ __launch_bounds__(kThreads) void paged_attention_generic_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_seq,
    const int* __restrict__ positions, T* __restrict__ out, int64_t out_stride, int Kh, int G, int hd, int hd_v,
    int page_size, int window, float soft_cap, float scale, const void* __restrict__ sinks, int sinks_dtype,
    AttentionOptions opt, int G_all, const float* __restrict__ slopes) {
  // G_all query vectors per key/value head, of which this workgroup takes G (the last one of a head what is left):
  // many heads over one key head need not fit into one workgroup's LDS
  const int gz = blockIdx.z * G;          // the workgroup's first vector among its key head's
  if (G > G_all - gz) G = G_all - gz;
  extern __shared__ float smem[];
  __shared__ float red_s[16];
  float* q_s = smem;                      // [G][hd]
  float* s_s = q_s + G * hd;              // [G][kChunk] scores, then probabilities
  float* m_s = s_s + G * kChunk;          // [G] running maximum
  float* l_s = m_s + G;                   // [G] running sum
  float* a_s = l_s + G;                   // [G] rescale factor of this chunk
  int* page_s = reinterpret_cast<int*>(a_s + G);  // [kChunk] page of each key of the chunk

  const int t = blockIdx.x, kh = blockIdx.y, tid = threadIdx.x;
  const int hd_k = M * hd;   // entries of a key row
  const bool tiled = keys_tiled(page_size, hd_k);
  const int seq = token_seq[t];
  const int pos = positions[t];
  const int hi = pos + 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + static_cast<size_t>(seq) * table_stride;

  for (int i = tid; i < G * hd; i += kThreads) {
    const int g = i / hd, d = i % hd;
    q_s[i] = to_float(q[static_cast<size_t>(t) * q_stride + static_cast<size_t>(kh * G_all + gz + g) * hd + d]);
  }
  for (int g = tid; g < G; g += kThreads) {
    m_s[g] = -INFINITY;
    l_s[g] = 0.f;
  }
  float acc[kMaxDimsPerThread][8];  // [dim slot][g within a tile of 8 heads]; G > 8 loops over head tiles
  // Heads are processed in tiles of 8 so that the accumulators stay in registers.
  for (int g0 = 0; g0 < G; g0 += 8) {
    const int gn = G - g0 < 8 ? G - g0 : 8;
#pragma unroll
    for (int s = 0; s < kMaxDimsPerThread; ++s)
#pragma unroll
      for (int g = 0; g < 8; ++g) acc[s][g] = 0.f;
    __syncthreads();

    for (int c0 = (lo / kChunk) * kChunk; c0 < hi; c0 += kChunk) {
      const int jlo = lo > c0 ? lo - c0 : 0;
      const int jhi = hi - c0 < kChunk ? hi - c0 : kChunk;
      if (tid < kChunk) {
        const int key = c0 + tid;
        page_s[tid] = (tid >= jlo && tid < jhi) ? table[key / page_size] : -1;
      }
      __syncthreads();
      // ---- scores: 4 threads per key, each over a quarter of the head size (interleaved)
      {
        const int j = tid / 4, part = tid % 4;
        const bool valid = j >= jlo && j < jhi;
        float dot[8];
#pragma unroll
        for (int g = 0; g < 8; ++g) dot[g] = 0.f;
        if (valid) {
          const int key = c0 + j;
          const T* kp = k_pages + (static_cast<size_t>(page_s[j]) * Kh + kh) * page_size * hd_k;
          const int kin = key % page_size;
          for (int d = part; d < hd; d += 4) {
            float kv[M];   // the key vector of every map (g0 is a multiple of M: head g's map is g % M)
#pragma unroll
            for (int m = 0; m < M; ++m) kv[m] = to_float(kp[key_index(tiled, page_size, hd_k, kin, m * hd + d)]);
#pragma unroll
            for (int g = 0; g < 8; ++g)
              if (g < gn) dot[g] = fmaf(q_s[(g0 + g) * hd + d], kv[g % M], dot[g]);
          }
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
          if (g < gn) {
            float s = dot[g];
            s += __shfl_xor(s, 1, kWave);
            s += __shfl_xor(s, 2, kWave);
            if (part == 0) {
              s *= scale;
              if (soft_cap > 0.f) s = soft_cap * tanhf(s / soft_cap);
              // a bias by distance: the head's slope times how far back the key lies is taken off
              if (slopes != nullptr) s -= slopes[(kh * G_all + gz + g0 + g) / M] * static_cast<float>(pos - (c0 + j));
              s_s[(g0 + g) * kChunk + j] = valid ? s : -INFINITY;
            }
          }
        }
      }
      __syncthreads();
      // ---- softmax update: wave w takes heads w, w + 4, ...
      {
        const int wave = tid / kWave, lane = tid % kWave;
        for (int g = wave; g < gn; g += kThreads / kWave) {
          const float s = s_s[(g0 + g) * kChunk + lane];
          const float m_old = m_s[g0 + g];
          const float m_new = fmaxf(m_old, wave_max(s));
          const float p = (lane >= jlo && lane < jhi) ? expf(s - m_new) : 0.f;
          const float sum = wave_sum(p);
          s_s[(g0 + g) * kChunk + lane] = p;
          if (lane == 0) {
            const float alpha = expf(m_old - m_new);  // 0 for the first chunk (m_old = -inf)
            a_s[g0 + g] = alpha;
            l_s[g0 + g] = l_s[g0 + g] * alpha + sum;
            m_s[g0 + g] = m_new;
          }
        }
      }
      __syncthreads();
      // ---- values: thread d accumulates output dimension d for every head of the tile
#pragma unroll
      for (int s = 0; s < kMaxDimsPerThread; ++s) {
        const int d = tid + s * kThreads;
        if (d < hd_v) {
#pragma unroll
          for (int g = 0; g < 8; ++g)
            if (g < gn) acc[s][g] *= a_s[g0 + g];
          for (int j = jlo; j < jhi; ++j) {
            const int key = c0 + j;
            const float v = to_float(
                opt.values_in_keys
                    ? k_pages[(static_cast<size_t>(page_s[j]) * Kh + kh) * page_size * hd_k +
                              key_index(tiled, page_size, hd_k, key % page_size, d)]
                    : v_pages[((static_cast<size_t>(page_s[j]) * Kh + kh) * hd_v + d) * page_size + key % page_size]);
#pragma unroll
            for (int g = 0; g < 8; ++g)
              if (g < gn) acc[s][g] = fmaf(s_s[(g0 + g) * kChunk + j], v, acc[s][g]);
          }
        }
      }
      __syncthreads();
    }
    if (M == 2 && opt.differential) {
      // heads g0 / 2 .. : o = a_1 - lambda a_2, divided by its root mean square over the head's values, times mult
      float o[kMaxDimsPerThread][4], ss[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) ss[p] = 0.f;
#pragma unroll
      for (int s = 0; s < kMaxDimsPerThread; ++s) {
        const int d = tid + s * kThreads;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          o[s][p] = 0.f;
          if (d < hd_v && 2 * p + 1 < gn) {
            o[s][p] = acc[s][2 * p] / l_s[g0 + 2 * p] - opt.lambda * (acc[s][2 * p + 1] / l_s[g0 + 2 * p + 1]);
            ss[p] = fmaf(o[s][p], o[s][p], ss[p]);
          }
        }
      }
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        if (2 * p + 1 >= gn) break;   // (uniform over the workgroup)
        const float r = opt.mult / sqrtf(block_sum(ss[p], red_s) / static_cast<float>(hd_v) + opt.eps);
#pragma unroll
        for (int s = 0; s < kMaxDimsPerThread; ++s) {
          const int d = tid + s * kThreads;
          if (d < hd_v)
            out[static_cast<size_t>(t) * out_stride + static_cast<size_t>((kh * G_all + gz + g0) / 2 + p) * hd_v + d] =
                from_float<T>(o[s][p] * r);
        }
      }
      continue;
    }
#pragma unroll
    for (int s = 0; s < kMaxDimsPerThread; ++s) {
      const int d = tid + s * kThreads;
      if (d < hd_v) {
#pragma unroll
        for (int g = 0; g < 8; ++g)
          if (g < gn) {
            // a sink is one more term of the softmax's sum, exp(sink - maximum), without a value
            float l = l_s[g0 + g];
            if (sinks != nullptr) l += expf(load_f(sinks, sinks_dtype, kh * G_all + gz + g0 + g) - m_s[g0 + g]);
            out[static_cast<size_t>(t) * out_stride + static_cast<size_t>(kh * G_all + gz + g0 + g) * hd_v + d] =
                from_float<T>(acc[s][g] / l);
          }
      }
    }
  }
}

template <int M>
static void launch_generic(const void* q, int dtype, int64_t q_stride, const void* k_pages, const void* v_pages,
                           const int* block_table, int table_stride, const int* token_seq, const int* positions,
                           void* out, int64_t out_stride, int T, int Kh, int G, int hd, int hd_v, int page_size,
                           int window, float soft_cap, float scale, const void* sinks, int sinks_dtype,
                           AttentionOptions opt, size_t smem, int G_all, const float* slopes, hipStream_t stream) {
  const dim3 grid(T, Kh, (G_all + G - 1) / G);
  if (dtype == kF32)
    paged_attention_generic_kernel<float, M><<<grid, kThreads, smem, stream>>>(
        static_cast<const float*>(q), q_stride, static_cast<const float*>(k_pages),
        static_cast<const float*>(v_pages), block_table, table_stride, token_seq, positions, static_cast<float*>(out),
        out_stride, Kh, G, hd, hd_v, page_size, window, soft_cap, scale, sinks, sinks_dtype, opt, G_all, slopes);
  else
    paged_attention_generic_kernel<bf16, M><<<grid, kThreads, smem, stream>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<const bf16*>(k_pages), static_cast<const bf16*>(v_pages),
        block_table, table_stride, token_seq, positions, static_cast<bf16*>(out), out_stride, Kh, G, hd, hd_v, page_size,
        window, soft_cap, scale, sinks, sinks_dtype, opt, G_all, slopes);
}

int paged_attention_generic(const void* q, int dtype, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* token_seq, const int* positions,
                            void* out, int64_t out_stride, int T, int H, int Kh, int hd, int page_size, int window,
                            float soft_cap, hipStream_t stream, int hd_v, float scale, const void* sinks,
                            int sinks_dtype, int maps, int values_in_keys, int differential, float lambda, float eps,
                            float mult, const float* slopes) {
  int G = H / Kh * maps;   // query vectors per key/value head (below: per workgroup)
  if (hd_v <= 0) hd_v = hd;
  if (maps != 1 && maps != 2) {
    set_error("paged_attention: %d score maps per head (1 or 2)", maps);
    return 1;
  }
  if (differential && maps != 2) {
    set_error("paged_attention: the differential combination needs two score maps per head");
    return 1;
  }
  if (maps > 1 && sinks != nullptr) {
    set_error("paged_attention: sinks and several score maps do not combine");
    return 1;
  }
  if (values_in_keys && hd_v > maps * hd) {
    set_error("paged_attention: %d values cannot be read from key rows of %d entries", hd_v, maps * hd);
    return 1;
  }
  if (hd_v > kThreads * kMaxDimsPerThread) {
    set_error("paged_attention: value size %d is above the largest supported (%d)", hd_v, kThreads * kMaxDimsPerThread);
    return 1;
  }
  // the query vectors of a key head are cut over workgroups (in multiples of 8, the heads that run side by side) until
  // a workgroup's share fits into LDS
  const int G_all = G;
  auto lds = [&](int g) {
    return sizeof(float) * (static_cast<size_t>(g) * hd + static_cast<size_t>(g) * kChunk + 3 * g) + sizeof(int) * kChunk;
  };
  while (lds(G) > 64 * 1024 && G > 8) G = ((G + 1) / 2 + 7) / 8 * 8;
  const size_t smem = lds(G);
  if (smem > 64 * 1024) {
    set_error("paged_attention: %d query vectors of size %d need %zu bytes of LDS (limit 65536)", G, hd, smem);
    return 1;
  }
  AttentionOptions opt;
  opt.values_in_keys = values_in_keys;
  opt.differential = differential;
  opt.lambda = lambda;
  opt.eps = eps;
  opt.mult = mult;
  if (maps == 2)
    launch_generic<2>(q, dtype, q_stride, k_pages, v_pages, block_table, table_stride, token_seq, positions, out,
                      out_stride, T, Kh, G, hd, hd_v, page_size, window, soft_cap, scale, sinks, sinks_dtype, opt, smem,
                      G_all, slopes, stream);
  else
    launch_generic<1>(q, dtype, q_stride, k_pages, v_pages, block_table, table_stride, token_seq, positions, out,
                      out_stride, T, Kh, G, hd, hd_v, page_size, window, soft_cap, scale, sinks, sinks_dtype, opt, smem,
                      G_all, slopes, stream);
  return check_launch("paged_attention_generic");
}

}  // namespace sa
