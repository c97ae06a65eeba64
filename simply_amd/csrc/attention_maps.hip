// Paged attention in bfloat16 on the matrix cores for mixers whose keys and values have sizes of their own, whose
// heads have several score maps, or whose many heads share one key head (latents): the few-rows kernel of
// attention_decode.hip with the sizes as launch arguments.
//
// A unit of work is up to 16 query rows of one request: 16 / Gc consecutive tokens times Gc query vectors that read
// the same key vectors (the heads of a key head, one map of each; more than 16 heads over one key head are cut into
// `chunks` of Gc).  One workgroup of four waves takes (unit, key head x map x chunk, range of keys).  Per tile of
// 32 keys every wave computes
//     S^T[key, row] = K[key, :] . Q[row, :]        v_mfma_f32_16x16x32_bf16, the key blocks straight from the page
//                                                  (16 keys x 32 entries are stored as one operand), Q from LDS
//     scale, mask, running maximum and sum per row (float32)
// and then its own quarter of the value entries,
//     O^T[d, row] += V^T[d, key] . P^T[key, row]   value pages are stored transposed, so V^T is a plain load.
// The waves therefore need no exchange at the end (each has the same maxima and sums); the scores are computed four
// times, which costs MFMA cycles that a kernel bound by reading keys and values has to spare.  Ranges of keys are
// merged by a second kernel from the workspace in their order; the same kernel forms the differential combination
// (a_1 - lambda a_2, divided by its root mean square) of two maps in 32-bit.
#include "api.h"
#include "attention_common.h"

namespace sa {

int paged_attention_decode_ranges(int seq_count, int Kh, int window, int max_kv_len, int num_splits);

constexpr int kMapsSubTiles = 2048;   // sub-tiles of 16 keys whose page a workgroup looks up at a time
constexpr int kWaveUnitsFrom = 2048;  // (units x heads) from which a wave takes a unit of its own

struct MapsShape {
  int Kh, maps, chunks, Gc, G_all;   // key heads; maps per head; chunks of Gc query heads per key head (G_all in all)
  int ndc, row_blocks, hdv;          // 32-entry blocks of one map's key vector, of a whole key row; value entries
  int page_size, window;
  float scale;
};

// NDBW: blocks of 16 value entries that a wave owns (its quarter of them, rounded up).  KB: key blocks of 32 entries
// whose loads are asked for together (0: block by block, for launches with many workgroups on a CU, whose waits cover
// one another; with a few workgroups on the GPU a wave waits for memory once a batch instead of once a block).
template <int NDBW, int KB>
__global__ __launch_bounds__(256) void paged_attention_maps_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const SeqMeta* __restrict__ units, int unit_begin,
    bf16* __restrict__ out, int64_t out_stride, MapsShape sh, float* __restrict__ workspace, int always_partial) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16x8* q_s = reinterpret_cast<bf16x8*>(smem_raw);   // [ndc][64]: the B operands of the unit's rows
  __shared__ int2 where_s[kMapsSubTiles];

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r = lane % 16, grp = lane / 16;
  const int split = blockIdx.x, num_splits = gridDim.x, vy = blockIdx.y, KhV = gridDim.y;
  const int chunk = vy % sh.chunks, map = (vy / sh.chunks) % sh.maps, kh = vy / (sh.chunks * sh.maps);
  const SeqMeta sm = units[unit_begin + blockIdx.z];
  const int Gc = sh.Gc, NDC = sh.ndc, HDV = sh.hdv, page_size = sh.page_size, window = sh.window;
  const int NDB = HDV / 16;
  const int rows = Gc * sm.q_len;   // <= 16
  if (rows == 0) return;            // (an empty unit that fills a group: uniform over the workgroup)
  const int* table = block_table + static_cast<size_t>(sm.slot) * table_stride;
  const int qi = r / Gc, g = r % Gc;
  const bool row_ok = r < rows;
  const int pos_r = sm.pos0 + qi;
  const int hi = sm.pos0 + sm.q_len;
  const int lo = (window > 0 && sm.pos0 - window + 1 > 0) ? sm.pos0 - window + 1 : 0;
  const int lo_r = (window > 0 && pos_r - window + 1 > 0) ? pos_r - window + 1 : 0;

  const int tile0 = lo / kTile, tile1 = (hi + kTile - 1) / kTile;
  const int ntiles = tile1 - tile0;
  const int tb = tile0 + static_cast<int>(static_cast<int64_t>(ntiles) * split / num_splits);
  const int te = tile0 + static_cast<int>(static_cast<int64_t>(ntiles) * (split + 1) / num_splits);

  // the rows' query vectors as B operands: lane (row r, grp) of block dc holds Q[row r][dc * 32 + grp * 8 .. + 8]
  {
    const int head = kh * sh.G_all + chunk * Gc + (row_ok ? g : 0);
    const bf16* qp = q + static_cast<size_t>(sm.q_start + (row_ok ? qi : 0)) * q_stride +
                     (static_cast<size_t>(head) * sh.maps + map) * (NDC * 32) + grp * 8;
    for (int dc = wave; dc < NDC; dc += 4)
      q_s[dc * kWave + lane] = row_ok ? *reinterpret_cast<const bf16x8*>(qp + dc * 32) : bf16x8{};
  }
  constexpr int kPassTiles = kMapsSubTiles / 2;
  int pass_b = tb;
  int pass_e = te - tb > kPassTiles ? tb + kPassTiles : te;
  int sub0 = 2 * pass_b;
  auto look_up = [&]() {
    const int nsub = pass_e > pass_b ? 2 * (pass_e - pass_b) : 1;
    for (int i = tid; i < nsub; i += 256) {
      const int key = (sub0 + i) * 16;
      int2 w = {0, 0};
      if (key < hi && key + 16 > lo) {
        const int block = key / page_size;
        w.x = table[block];
        w.y = (key - block * page_size) / 16;
      }
      where_s[i] = w;
    }
    __syncthreads();
  };
  look_up();

  floatx4 acc[NDBW];
#pragma unroll
  for (int j = 0; j < NDBW; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const int db0 = wave * NDBW;   // this wave's first block of value entries
  const size_t row_elems = static_cast<size_t>(sh.row_blocks) * 32;

  for (;;) {
    for (int tile = pass_b; tile < pass_e; ++tile) {
      const int key0 = tile * kTile;
      bool sub_ok[2];
      const bf16* kp[2];
      const bf16* vp[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int sk0 = key0 + t * 16;
        sub_ok[t] = sk0 < hi && sk0 + 16 > lo;   // wave-uniform
        // (a sub-tile outside the range is loaded all the same, from where the pass's first sub-tile lies, and masked)
        const int2 w = where_s[sub_ok[t] ? 2 * tile + t - sub0 : 0];
        const size_t head = static_cast<size_t>(w.x) * sh.Kh + kh;
        kp[t] = k_pages + head * page_size * row_elems + static_cast<size_t>(w.y) * (sh.row_blocks * 512) +
                static_cast<size_t>(map * NDC) * 512 + lane * 8;
        vp[t] = v_pages + (head * HDV + r) * page_size + w.y * 16 + grp * 4;
      }
      // this wave's values of the tile are asked for first: they are under way during the scores
      bf16x4 vf[2][NDBW];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < NDBW; ++j)
          vf[t][j] = db0 + j < NDB ? *reinterpret_cast<const bf16x4*>(vp[t] + static_cast<size_t>(db0 + j) * 16 * page_size)
                                   : bf16x4{};
      floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
      if constexpr (KB == 0) {
        for (int dc = 0; dc < NDC; ++dc) {
          const bf16x8 k0 = *reinterpret_cast<const bf16x8*>(kp[0] + dc * 512);
          const bf16x8 k1 = *reinterpret_cast<const bf16x8*>(kp[1] + dc * 512);
          const bf16x8 qf = q_s[dc * kWave + lane];
          s[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qf, s[0], 0, 0, 0);
          s[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qf, s[1], 0, 0, 0);
        }
      } else {
        // (a block beyond the vector's last is the last one again, loaded and not used: every load of a batch is
        // unconditional)
        for (int dc0 = 0; dc0 < NDC; dc0 += KB) {
          bf16x8 kf[2][KB > 0 ? KB : 1];
#pragma unroll
          for (int j = 0; j < KB; ++j) {
            const int dc = dc0 + j < NDC ? dc0 + j : NDC - 1;
            kf[0][j] = *reinterpret_cast<const bf16x8*>(kp[0] + dc * 512);
            kf[1][j] = *reinterpret_cast<const bf16x8*>(kp[1] + dc * 512);
          }
#pragma unroll
          for (int j = 0; j < KB; ++j) {
            if (dc0 + j < NDC) {
              const bf16x8 qf = q_s[(dc0 + j) * kWave + lane];
              s[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][j], qf, s[0], 0, 0, 0);
              s[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][j], qf, s[1], 0, 0, 0);
            }
          }
        }
      }
      // ---- scale, mask, online softmax.  Lane (row r, grp) holds keys sk0 + 4 * grp + v of each sub-tile.
      float p[2][4];
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int key = key0 + t * 16 + grp * 4 + v;
          const bool vis = sub_ok[t] && row_ok && key <= pos_r && key >= lo_r;
          const float x = vis ? s[t][v] * sh.scale : -INFINITY;
          p[t][v] = x;
          mx = fmaxf(mx, x);
        }
      mx = max_over_row_lanes(mx);
      const float m_new = fmaxf(m_run, mx);
      const float alpha = m_new == -INFINITY ? 1.f : __expf(m_run - m_new);
      float psum = 0.f;
      bf16x8 pf;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float e = p[t][v] == -INFINITY ? 0.f : __expf(p[t][v] - m_new);
          psum += e;
          pf[t * 4 + v] = to_bf16_raw(e);
        }
      l_run = l_run * alpha + psum;
      m_run = m_new;
      // ---- O^T[d][row] = alpha O^T + V^T[d][keys] . P^T[keys][row]
      const bool tail = key0 + kTile > hi || !sub_ok[0] || !sub_ok[1];   // keys that may be unwritten count as 0
#pragma unroll
      for (int j = 0; j < NDBW; ++j) {
        bf16x8 a;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) a[t * 4 + v] = vf[t][j][v];
        if (tail) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int key = key0 + (e / 4) * 16 + grp * 4 + (e % 4);
            if (key >= hi || !sub_ok[e / 4]) a[e] = to_bf16_raw(0.f);
          }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[j][v] *= alpha;
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf, acc[j], 0, 0, 0);
      }
    }
    if (pass_e >= te) break;
    __syncthreads();
    pass_b = pass_e;
    pass_e = te - pass_b > kPassTiles ? pass_b + kPassTiles : te;
    sub0 = 2 * pass_b;
    look_up();
  }

  // acc[j][v] is O^T[d = (db0 + j) * 16 + 4 * grp + v][row r]; every wave holds the same maxima and sums
  l_run = sum_over_row_lanes(l_run);
  if (!row_ok) return;
  const int KS = num_splits;
  if (KS == 1 && !always_partial) {
    bf16* op = out + static_cast<size_t>(sm.q_start + qi) * out_stride + static_cast<size_t>(vy * Gc + g) * HDV;
    const float inv = 1.f / l_run;
#pragma unroll
    for (int j = 0; j < NDBW; ++j)
      if (db0 + j < NDB)
#pragma unroll
        for (int v = 0; v < 4; ++v) op[(db0 + j) * 16 + 4 * grp + v] = float_to_bf16(acc[j][v] * inv);
    return;
  }
  const size_t row_words = HDV + kRowExtra;
  const size_t unit = static_cast<size_t>(blockIdx.z) * KhV + vy;
  float* wp = workspace + ((unit * KS + split) * 16 + r) * row_words;
#pragma unroll
  for (int j = 0; j < NDBW; ++j)
    if (db0 + j < NDB) *reinterpret_cast<floatx4*>(wp + (db0 + j) * 16 + 4 * grp) = acc[j];
  if (wave == 0 && grp == 0) {
    wp[HDV] = m_run;
    wp[HDV + 1] = l_run;
  }
}

// The same attention for launches with many units (portions of prompts): every wave of a workgroup takes a unit of
// its own, four consecutive units a workgroup (fewer where the waves' queries would not fit into LDS), and owns all of its value entries, so the scores are computed once.  The
// four waves walk nearly the same keys at nearly the same time (consecutive tokens of a request), so the key blocks that
// one of them brings come from the CU's cache for the others.  No ranges of keys, no barrier: a wave looks its pages up
// itself, sub-tile by sub-tile, and waves of other workgroups cover that wait.
// NDBT: blocks of 16 value entries (rounded up to a power of two; those beyond the values' are skipped).
constexpr int kValueBatch = 8;   // value blocks whose loads are asked for together
template <int NDBT>
__global__ __launch_bounds__(256) void paged_attention_maps_waves_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const SeqMeta* __restrict__ units, int unit_begin,
    int unit_count, bf16* __restrict__ out, int64_t out_stride, MapsShape sh, float* __restrict__ workspace,
    int always_partial) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int u = blockIdx.z * (blockDim.x / kWave) + wave, vy = blockIdx.y, KhV = gridDim.y;   // (four waves, or as many as LDS holds)
  if (u >= unit_count) return;   // (a whole wave; nothing below waits for another wave)
  const int r = lane % 16, grp = lane / 16;
  const int chunk = vy % sh.chunks, map = (vy / sh.chunks) % sh.maps, kh = vy / (sh.chunks * sh.maps);
  const SeqMeta sm = units[unit_begin + u];
  const int Gc = sh.Gc, NDC = sh.ndc, HDV = sh.hdv, page_size = sh.page_size, window = sh.window;
  const int NDB = HDV / 16;
  const int rows = Gc * sm.q_len;
  if (rows == 0) return;
  bf16x8* q_s = reinterpret_cast<bf16x8*>(smem_raw) + static_cast<size_t>(wave) * NDC * kWave;   // this wave's own
  const int* table = block_table + static_cast<size_t>(sm.slot) * table_stride;
  const int qi = r / Gc, g = r % Gc;
  const bool row_ok = r < rows;
  const int pos_r = sm.pos0 + qi;
  const int hi = sm.pos0 + sm.q_len;
  const int lo = (window > 0 && sm.pos0 - window + 1 > 0) ? sm.pos0 - window + 1 : 0;
  const int lo_r = (window > 0 && pos_r - window + 1 > 0) ? pos_r - window + 1 : 0;
  {
    const int head = kh * sh.G_all + chunk * Gc + (row_ok ? g : 0);
    const bf16* qp = q + static_cast<size_t>(sm.q_start + (row_ok ? qi : 0)) * q_stride +
                     (static_cast<size_t>(head) * sh.maps + map) * (NDC * 32) + grp * 8;
    for (int dc = 0; dc < NDC; ++dc)
      q_s[dc * kWave + lane] = row_ok ? *reinterpret_cast<const bf16x8*>(qp + dc * 32) : bf16x8{};
  }
  const int safe_page = table[(hi - 1) / page_size];   // the unit's last token has a page: loads that are not needed go there
  floatx4 acc[NDBT];
#pragma unroll
  for (int j = 0; j < NDBT; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const size_t row_elems = static_cast<size_t>(sh.row_blocks) * 32;

  for (int tile = lo / kTile; tile * kTile < hi; ++tile) {
    const int key0 = tile * kTile;
    bool sub_ok[2];
    const bf16* kp[2];
    const bf16* vp[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int sk0 = key0 + t * 16;
      sub_ok[t] = sk0 < hi && sk0 + 16 > lo;   // wave-uniform
      const int block = sk0 / page_size;
      const int page = sub_ok[t] ? table[block] : safe_page;
      const int blk = sub_ok[t] ? (sk0 - block * page_size) / 16 : 0;
      const size_t head = static_cast<size_t>(page) * sh.Kh + kh;
      kp[t] = k_pages + head * page_size * row_elems + static_cast<size_t>(blk) * (sh.row_blocks * 512) +
              static_cast<size_t>(map * NDC) * 512 + lane * 8;
      vp[t] = v_pages + (head * HDV + r) * page_size + blk * 16 + grp * 4;
    }
    floatx4 s[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    for (int dc = 0; dc < NDC; ++dc) {
      const bf16x8 k0 = *reinterpret_cast<const bf16x8*>(kp[0] + dc * 512);
      const bf16x8 k1 = *reinterpret_cast<const bf16x8*>(kp[1] + dc * 512);
      const bf16x8 qf = q_s[dc * kWave + lane];
      s[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qf, s[0], 0, 0, 0);
      s[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qf, s[1], 0, 0, 0);
    }
    float p[2][4];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int key = key0 + t * 16 + grp * 4 + v;
        const bool vis = sub_ok[t] && row_ok && key <= pos_r && key >= lo_r;
        const float x = vis ? s[t][v] * sh.scale : -INFINITY;
        p[t][v] = x;
        mx = fmaxf(mx, x);
      }
    mx = max_over_row_lanes(mx);
    const float m_new = fmaxf(m_run, mx);
    const float alpha = m_new == -INFINITY ? 1.f : __expf(m_run - m_new);
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float e = p[t][v] == -INFINITY ? 0.f : __expf(p[t][v] - m_new);
        psum += e;
        pf[t * 4 + v] = to_bf16_raw(e);
      }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    const bool tail = key0 + kTile > hi || !sub_ok[0] || !sub_ok[1];
#pragma unroll
    for (int j0 = 0; j0 < NDBT; j0 += kValueBatch) {
      constexpr int kB = NDBT < kValueBatch ? NDBT : kValueBatch;
      bf16x4 vf[2][kB];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < kB; ++j)
          vf[t][j] = j0 + j < NDB ? *reinterpret_cast<const bf16x4*>(vp[t] + static_cast<size_t>(j0 + j) * 16 * page_size)
                                  : bf16x4{};
#pragma unroll
      for (int j = 0; j < kB; ++j) {
        bf16x8 a;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) a[t * 4 + v] = vf[t][j][v];
        if (tail) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int key = key0 + (e / 4) * 16 + grp * 4 + (e % 4);
            if (key >= hi || !sub_ok[e / 4]) a[e] = to_bf16_raw(0.f);
          }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[j0 + j][v] *= alpha;
        acc[j0 + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf, acc[j0 + j], 0, 0, 0);
      }
    }
  }
  l_run = sum_over_row_lanes(l_run);
  if (!row_ok) return;
  if (!always_partial) {
    bf16* op = out + static_cast<size_t>(sm.q_start + qi) * out_stride + static_cast<size_t>(vy * Gc + g) * HDV;
    const float inv = 1.f / l_run;
#pragma unroll
    for (int j = 0; j < NDBT; ++j)
      if (j < NDB)
#pragma unroll
        for (int v = 0; v < 4; ++v) op[j * 16 + 4 * grp + v] = float_to_bf16(acc[j][v] * inv);
    return;
  }
  const size_t row_words = HDV + kRowExtra;
  float* wp = workspace + ((static_cast<size_t>(u) * KhV + vy) * 16 + r) * row_words;   // (one range of keys)
#pragma unroll
  for (int j = 0; j < NDBT; ++j)
    if (j < NDB) *reinterpret_cast<floatx4*>(wp + j * 16 + 4 * grp) = acc[j];
  if (grp == 0) {
    wp[HDV] = m_run;
    wp[HDV + 1] = l_run;
  }
}

// The differential combination from the partial results of two maps: per (unit, key head, chunk, row) both maps'
// ranges are added up in their order, o = a_1 - lambda a_2 is divided by its root mean square over the head's values
// and multiplied by mult.  One workgroup per row and (key head, chunk); a thread takes the value entries tid,
// tid + 256, ...
constexpr int kCombinePerThread = 4;   // value sizes up to 1024
__global__ __launch_bounds__(256) void attention_maps_combine_kernel(
    const float* __restrict__ workspace, int KS, const SeqMeta* __restrict__ units, int unit_begin,
    bf16* __restrict__ out, int64_t out_stride, int KhV, int chunks, int Gc, int G_all, int HDV, float lambda, float eps,
    float mult) {
  __shared__ float scratch[16];
  const int tid = threadIdx.x, pair = blockIdx.x, z = blockIdx.y, orow = blockIdx.z;   // pair: (key head, chunk)
  const SeqMeta sm = units[unit_begin + z];
  if (orow >= Gc * sm.q_len) return;
  const int kh = pair / chunks, chunk = pair % chunks;
  const size_t row_words = HDV + kRowExtra, stride = 16 * row_words;
  float o[kCombinePerThread];
#pragma unroll
  for (int e = 0; e < kCombinePerThread; ++e) o[e] = 0.f;
  for (int m = 0; m < 2; ++m) {
    const int vy = (kh * 2 + m) * chunks + chunk;
    const float* base = workspace + ((static_cast<size_t>(z) * KhV + vy) * KS * 16 + orow) * row_words;
    float M = -INFINITY;
    for (int y = 0; y < KS; ++y) M = fmaxf(M, base[y * stride + HDV]);
    float L = 0.f;
    for (int y = 0; y < KS; ++y) {
      const float my = base[y * stride + HDV];
      L += my == -INFINITY ? 0.f : base[y * stride + HDV + 1] * __expf(my - M);
    }
    const float f = (m == 0 ? 1.f : -lambda) / L;
    for (int y = 0; y < KS; ++y) {
      const float my = base[y * stride + HDV];
      const float wy = my == -INFINITY ? 0.f : __expf(my - M) * f;
#pragma unroll
      for (int e = 0; e < kCombinePerThread; ++e) {
        const int d = tid + e * 256;
        if (d < HDV) o[e] = fmaf(base[y * stride + d], wy, o[e]);
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < kCombinePerThread; ++e) ss = fmaf(o[e], o[e], ss);   // (entries beyond HDV are 0)
  ss = block_sum(ss, scratch);
  const float rr = mult / sqrtf(ss / static_cast<float>(HDV) + eps);
  const int oq = orow / Gc, og = orow % Gc;
  bf16* op = out + static_cast<size_t>(sm.q_start + oq) * out_stride +
             static_cast<size_t>(kh * G_all + chunk * Gc + og) * HDV;
#pragma unroll
  for (int e = 0; e < kCombinePerThread; ++e) {
    const int d = tid + e * 256;
    if (d < HDV) op[d] = float_to_bf16(o[e] * rr);
  }
}

// The most query heads of a key head that share a unit: the largest divisor of G that is at most 16.
static int heads_per_unit(int G) {
  for (int c = G < 16 ? G : 16; c > 1; --c)
    if (G % c == 0) return c;
  return 1;
}

}  // namespace sa

using namespace sa;

extern "C" int sa_attention_maps_heads_per_unit(int H, int Kh) {
  return (H > 0 && Kh > 0 && H % Kh == 0) ? heads_per_unit(H / Kh) : 0;
}

// Whether sa_paged_attention_maps_units takes these sizes: pages of a multiple of 16 keys, key vectors of a multiple
// of 32 entries (up to 1024), values of a multiple of 16 entries (up to 1024), 16-byte aligned query rows.
extern "C" int sa_paged_attention_maps_units_takes(int H, int Kh, int maps, int hd, int hd_v, int page_size,
                                                   int64_t q_stride, const void* q) {
  return H > 0 && Kh > 0 && H % Kh == 0 && (maps == 1 || maps == 2) && hd > 0 && hd % 32 == 0 && hd <= 1024 && hd_v > 0 &&
         hd_v % 16 == 0 && hd_v <= 1024 && page_size > 0 && page_size % 16 == 0 && q_stride % 8 == 0 &&
         (reinterpret_cast<uintptr_t>(q) & 15u) == 0;
}

// Attention of the units [unit_begin, unit_begin + unit_count) of `units` (rows: slot, first row, tokens, first
// position; at most 16 / sa_attention_maps_heads_per_unit tokens each), as sa_paged_attention_maps computes it, in
// bfloat16 on the matrix cores.  Key pages [pages, Kh, page_size, maps * hd] in operand blocks, value pages
// [pages, Kh, hd_v, page_size].  differential: out [T, H * hd_v]; else out [T, H * hd_v] too (maps must be 1).
extern "C" int sa_paged_attention_maps_units(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                             const int* block_table, int table_stride, const int* units,
                                             int unit_begin, int unit_count, void* out, int64_t out_stride, int H, int Kh,
                                             int hd, int hd_v, int page_size, int window, float scale, int maps,
                                             int differential, float lambda, float eps, float mult, int max_kv_len,
                                             int max_q_len, void* workspace, size_t workspace_bytes,
                                             hipStream_t stream) {
  if (unit_count == 0) return 0;
  SA_REQUIRE(unit_count > 0 && unit_begin >= 0 && table_stride > 0 && window >= 0 && max_kv_len > 0 && max_q_len > 0,
             "paged_attention_maps_units: bad counts, window, table or lengths");
  SA_REQUIRE(sa_paged_attention_maps_units_takes(H, Kh, maps, hd, hd_v, page_size, q_stride, q),
             "paged_attention_maps_units takes key vectors of a multiple of 32 entries, values of a multiple of 16, "
             "pages of a multiple of 16 keys and aligned query rows; got hd=%d hd_v=%d P=%d maps=%d", hd, hd_v,
             page_size, maps);
  SA_REQUIRE((maps == 2) == (differential != 0), "paged_attention_maps_units: two maps come with their combination");
  SA_REQUIRE(q_stride >= static_cast<int64_t>(H) * maps * hd && out_stride >= static_cast<int64_t>(H) * hd_v,
             "paged_attention_maps_units: row strides are below what the heads need");
  const int G = H / Kh, Gc = heads_per_unit(G);
  SA_REQUIRE(Gc * max_q_len <= 16, "paged_attention_maps_units: units of %d tokens x %d heads exceed 16 rows",
             max_q_len, Gc);
  MapsShape sh;
  sh.Kh = Kh, sh.maps = maps, sh.chunks = G / Gc, sh.Gc = Gc, sh.G_all = G;
  sh.ndc = hd / 32, sh.row_blocks = maps * hd / 32, sh.hdv = hd_v;
  sh.page_size = page_size, sh.window = window, sh.scale = scale;
  const int KhV = Kh * maps * sh.chunks;
  SA_REQUIRE(KhV <= 65535 && unit_count <= 65535, "paged_attention_maps_units: too many heads or units");
  int KS = paged_attention_decode_ranges(unit_count, KhV, window, max_kv_len, 0);
  const size_t per_split = static_cast<size_t>(unit_count) * KhV * 16 * (hd_v + kRowExtra) * sizeof(float);
  while (KS > 1 && (workspace == nullptr || per_split * KS > workspace_bytes)) --KS;
  const bool partial = differential != 0;
  SA_REQUIRE(!(partial || KS > 1) || (workspace != nullptr && per_split * KS <= workspace_bytes),
             "paged_attention_maps_units: the partial results (%zu bytes) do not fit the workspace", per_split * KS);
  const bf16* qp = static_cast<const bf16*>(q);
  const bf16* kp = static_cast<const bf16*>(k_pages);
  const bf16* vp = static_cast<const bf16*>(v_pages);
  const SeqMeta* um = reinterpret_cast<const SeqMeta*>(units);
  bf16* op = static_cast<bf16*>(out);
  float* ws = static_cast<float*>(workspace);
  // many units (portions of prompts) and one range of keys: a wave per unit, if four waves' queries fit into LDS
  int waves = 4;
  while (waves > 1 && static_cast<size_t>(waves) * sh.ndc * kWave * sizeof(bf16x8) > 64 * 1024) --waves;
  const size_t smem_waves = static_cast<size_t>(waves) * sh.ndc * kWave * sizeof(bf16x8);
  // (values of up to 128 entries: with wider ones a wave's accumulators leave room for two waves on a SIMD, and 2,048
  // units of a latent attention's 512 entries took 832 us so against 595 us with four waves a unit)
  if (KS == 1 && static_cast<int64_t>(unit_count) * KhV >= kWaveUnitsFrom && smem_waves <= 64 * 1024 && hd_v <= 128) {
    const dim3 grid(1, KhV, (unit_count + waves - 1) / waves);
    const int ndb = hd_v / 16;
#define SA_LAUNCH_W(N)                                                                                             \
  paged_attention_maps_waves_kernel<N><<<grid, waves * kWave, smem_waves, stream>>>(qp, q_stride, kp, vp, block_table, \
                                                                         table_stride, um, unit_begin, unit_count, \
                                                                         op, out_stride, sh, ws, partial ? 1 : 0)
    if (ndb <= 1) SA_LAUNCH_W(1);
    else if (ndb <= 2) SA_LAUNCH_W(2);
    else if (ndb <= 4) SA_LAUNCH_W(4);
    else if (ndb <= 8) SA_LAUNCH_W(8);
    else if (ndb <= 16) SA_LAUNCH_W(16);
    else if (ndb <= 32) SA_LAUNCH_W(32);
    else SA_LAUNCH_W(64);
#undef SA_LAUNCH_W
  } else {
  const dim3 grid(KS, KhV, unit_count);
  const size_t smem = static_cast<size_t>(sh.ndc) * kWave * sizeof(bf16x8);
  const int per_wave = (hd_v / 16 + 3) / 4;
#define SA_LAUNCH_KB(N, B)                                                                                            \
  paged_attention_maps_kernel<N, B><<<grid, 256, smem, stream>>>(qp, q_stride, kp, vp, block_table, table_stride, um, \
                                                                 unit_begin, op, out_stride, sh, ws, partial ? 1 : 0)
  // few workgroups for the GPU's 256 CUs: the key blocks' loads in batches
  const int batch = static_cast<int64_t>(KS) * KhV * unit_count > 1024 ? 0 : sh.ndc <= 2 ? 2 : sh.ndc <= 12 ? 6 : 18;
#define SA_LAUNCH(N)                   \
  if (batch == 0) SA_LAUNCH_KB(N, 0);  \
  else if (batch == 2) SA_LAUNCH_KB(N, 2); \
  else if (batch == 6) SA_LAUNCH_KB(N, 6); \
  else SA_LAUNCH_KB(N, 18)
  if (per_wave <= 1) { SA_LAUNCH(1); }
  else if (per_wave <= 2) { SA_LAUNCH(2); }
  else if (per_wave <= 4) { SA_LAUNCH(4); }
  else if (per_wave <= 8) { SA_LAUNCH(8); }
  else { SA_LAUNCH(16); }
#undef SA_LAUNCH_KB
#undef SA_LAUNCH
  }
  if (check_launch("paged_attention_maps_units")) return 1;
  const int max_rows = Gc * max_q_len < 16 ? Gc * max_q_len : 16;
  if (partial) {
    attention_maps_combine_kernel<<<dim3(Kh * sh.chunks, unit_count, max_rows), 256, 0, stream>>>(
        ws, KS, um, unit_begin, op, out_stride, KhV, sh.chunks, Gc, G, hd_v, lambda, eps, mult);
    return check_launch("attention_maps_combine");
  }
  if (KS > 1)
    return attention_merge_ranges(ws, KS, hd_v, um, unit_begin, unit_count, max_q_len, op, out_stride, KhV, Gc, stream);
  return 0;
}
