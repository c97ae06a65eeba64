// C interface of the gfx950 kernel library.  Every entry point returns 0 on
// success; otherwise sa_last_error() describes the refusal (a size the kernels
// do not take, an unknown element type, a failed launch).  Pointers are device
// pointers unless a comment says otherwise; `stream` is the HIP stream to
// launch on.  Element type codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

const char* sa_last_error();
int sa_version();

// out[t, :] = table[tokens[t], :] * scale (32-bit output: the residual stream).
// packed: the table is tiled like a matrix-product weight (see sa_gemm).
int sa_embed(const void* table, int table_dtype, const int* tokens, float* out, int T, int D, int V, float scale,
             int packed, hipStream_t stream);

// out = x * rsqrt(mean(x^2) + eps) * (w + plus_one), row by row.
int sa_rmsnorm(const void* x, int x_dtype, int64_t x_stride, const void* w, int w_dtype, void* out, int out_dtype,
               int64_t out_stride, int T, int D, float eps, int plus_one, hipStream_t stream);

// residual += norm(y; w_post) (w_post null: residual += y); then, if w_next is not null,
// out = norm(residual; w_next).
int sa_add_rmsnorm(const void* y, int y_dtype, const void* w_post, int w_post_dtype, float eps_post,
                   int plus_one_post, float* residual, const void* w_next, int w_next_dtype, float eps_next,
                   int plus_one_next, void* out, int out_dtype, int T, int D, hipStream_t stream);

// For the rows index[0..R-1] only, and without storing the sum: out[r] = norm(residual[index[r]] + norm(y[index[r]];
// w_post); w_next) (w_post null: + y as it is).  What a model's end needs: the rows whose logits are wanted.
int sa_add_rmsnorm_rows(const void* y, int y_dtype, const void* w_post, int w_post_dtype, float eps_post,
                        int plus_one_post, const float* residual, const void* w_next, int w_next_dtype, float eps_next,
                        int plus_one_next, void* out, int out_dtype, const int* index, int R, int D,
                        hipStream_t stream);

// The same with y given as `planes` partial results [planes][T][D] float32 (sa_gemm_planes): y is their sum in the
// order of the planes, rounded to bfloat16, as the sum kernel of the product would have left it.  D % 4 == 0.
int sa_add_rmsnorm_planes(const float* y_planes, int planes, const void* w_post, int w_post_dtype, float eps_post,
                          int plus_one_post, float* residual, const void* w_next, int w_next_dtype, float eps_next,
                          int plus_one_next, void* out, int out_dtype, int T, int D, hipStream_t stream);

// Fused projection rows [T, (H + 2K) * hd]: rotate q and k (timescale null: no rotation), divide q by
// q_div, write k and v into the pages at slot_mapping[t] = page * page_size + offset (k_pages null: no write).
int sa_rope_cache_write(void* qkv, int dtype, int64_t row_stride, const int* positions, const float* timescale,
                        float scale_factor, float q_div, const int64_t* slot_mapping, void* k_pages, void* v_pages,
                        int T, int H, int K, int hd, int page_size, hipStream_t stream);

// The same for a projection whose cuts of K are not added up yet (sa_gemm_planes): its elements are the sums of
// `count` planes [T][(H + 2K) hd] float32, rounded to bfloat16; the rotated and scaled queries go to qkv (bfloat16
// rows of row_stride elements; its key and value columns are not written).  A block per (token, head): for up to a
// few hundred tokens.
int sa_rope_cache_write_planes(const float* planes, int count, void* qkv, int64_t row_stride, const int* positions,
                               const float* timescale, float scale_factor, float q_div, const int64_t* slot_mapping,
                               void* k_pages, void* v_pages, int T, int H, int K, int hd, int page_size,
                               hipStream_t stream);

// Rotation alone, in place, then division by div.
int sa_rope(void* x, int dtype, int64_t row_stride, const int* positions, const float* timescale, float scale_factor,
            float div, int T, int n_heads, int hd, hipStream_t stream);

int sa_gather_rows(const void* x, int x_dtype, const int* index, void* out, int out_dtype, int R, int D,
                   hipStream_t stream);

int sa_fill_u32(void* p, uint32_t value, int64_t n, hipStream_t stream);

// Between two decode steps that run without the host in between (every request brings one token): records the tokens
// and log-probabilities just drawn as row *step_counter of out_tokens / out_logprobs [max_steps, B], makes them the
// next step's input tokens, adds one to every token's position, to every request's first position (seq_meta
// [B, 4], column 3) and draw counter, and to *step_counter.  B <= 1024.
int sa_decode_advance(int B, int* step_counter, const int* sampled_tokens, const float* sampled_logprobs,
                      int* tokens_in, int* positions, int* seq_meta, int* draw_counters, int* out_tokens,
                      float* out_logprobs, int max_steps, hipStream_t stream);
// sa_decode_advance and, in the same launch, sa_decode_slots at the new positions for num_groups (at most 4) cache
// groups: block_tables, table_strides and slot_mappings are host arrays of num_groups entries.
int sa_decode_advance_slots(int B, int* step_counter, const int* sampled_tokens, const float* sampled_logprobs,
                            int* tokens_in, int* positions, int* seq_meta, int* draw_counters, int* out_tokens,
                            float* out_logprobs, int max_steps, const int* token_seq, int num_groups,
                            const int* const* block_tables, const int* table_strides, int64_t* const* slot_mappings,
                            int page_size, hipStream_t stream);
// slot_mapping[b] = block_table[token_seq[b], positions[b] / page_size] * page_size + positions[b] % page_size
int sa_decode_slots(int B, const int* positions, const int* token_seq, const int* block_table, int table_stride,
                    int page_size, int64_t* slot_mapping, hipStream_t stream);

// C[M, N] = epilogue(A[M, K] . W[N, K]^T).  epilogue 0: none; 1 + 16 * a: act(A.W^T) * (A.W2^T) with the activation
// a of activations.h (0: tanh-approximated gelu, 1: silu, 2: squared relu), both products rounded to the output
// type first; 2: cap * tanh(. / cap); 3 + 16 * a: act(A.W^T), the product rounded to the output type first (in
// the epilogue of the few-rows kernel and of the wide kernel where it runs without a cut of K, else by a kernel
// behind the product).  algo 0: the library chooses; 1: the generic 32-bit-ALU kernel; 2: the
// few-rows bfloat16 kernel; 3: the tiled bfloat16 MFMA kernel; 4: the wide-tile bfloat16 MFMA kernel for very
// many rows (2, 3 and 4 refuse what they do not take).
// packed: W (and W2) are tiled instead of row-major: [ceil(N / 16)][ceil(K / 32)][64][8] bfloat16, block (i, j)
// holding rows 16 i .. 16 i + 15 and columns 32 j .. 32 j + 31 as element [(k % 32) / 8 * 16 + n % 16][k % 8],
// zero beyond N and K (one MFMA operand per block, in register order).  With epilogue 1 a packed W holds both
// matrices, their row blocks in turn (block row 2 i: rows 16 i .. of the gate, 2 i + 1: of the other factor), and
// W2 is null.
// shape > 0 fixes how a kernel cuts its work: for the few-rows kernel rows of W per workgroup (4, 8 or 16) * 100 +
// waves, for the tiled kernel the number of cuts of K, for the wide kernel (algo 4 only) stages * 1000000 + rows *
// 1000 + weight rows of a workgroup's tile.  workspace (bytes): scratch memory for partial results
// when K is cut over workgroups.
int sa_gemm(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C, int c_dtype,
            int64_t ldc, int M, int N, int K, int epilogue, float cap, int algo, int packed, int shape,
            void* workspace, int64_t workspace_bytes, hipStream_t stream);

// The same product, but where it is computed in cuts of K its last kernel, the sum of the cuts, is left to the
// caller: *planes receives their number, and the workspace then holds [planes][M][N] float32 partial results whose
// sum in the order of the planes, rounded to C's type, is the product (sa_add_rmsnorm_planes takes them).  *planes
// == 1: C holds the product as after sa_gemm.
// C = the sum of `count` planes [M][N] float32 in their order, rounded to C's type: the kernel that sa_gemm_planes
// leaves out.
// Which kernel sa_gemm would run for bfloat16 operands of these sizes with tiled weights and 16-byte aligned
// operands (2: few-rows, 3: tiled, 4: wide), and, in us[0..2] if it is not null, the microseconds that the library
// expects of the three (negative: not eligible).  c_dtype is the output's element type (the wide kernel writes
// bfloat16 only).  A host function: nothing is launched.
int sa_gemm_plan(int M, int N, int K, int epilogue, int c_dtype, int64_t workspace_bytes, double* us);
int sa_sum_planes(const float* planes, int count, void* C, int c_dtype, int64_t ldc, int M, int N, hipStream_t stream);
int sa_gemm_planes(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C,
                   int c_dtype, int64_t ldc, int M, int N, int K, int epilogue, float cap, int algo, int packed,
                   int shape, void* workspace, int64_t workspace_bytes, int* planes, hipStream_t stream);

// For 1..16 rows of bfloat16: h_out = h_in + norm(y; w_post) (y null: h_out is h_in and is not written; w_post null:
// h_out = h_in + y), a = norm(h_out; w_next), C = epilogue(a . W^T) with W tiled (paired tiles for the gated
// epilogue; epilogue codes as for sa_gemm).
// h_in, h_out: float32 [M, K], different buffers; y: bfloat16 [M, K]; norm weights float32 or bfloat16 [K].
int sa_gemm_normed_takes(int M, int N, int K);
// The most rows that sa_gemm_normed takes, and whether it is expected to be faster than the separate norm and
// product kernels at these sizes (it takes more sizes than it pays for: rows wider than 2560 elements pay only where
// the kernel has a prologue for exactly that width, and a weight with very many rows is better served by sa_gemm).
int sa_gemm_normed_max_rows();
int sa_gemm_normed_pays(int M, int N, int K);

// The fused q/k/v projection with the norms of sa_gemm_normed in front and the rotation, query scale and cache write
// of sa_rope_cache_write behind: C receives the queries [M, H * hd] (rows of ldc elements), keys and values go into
// the pages.  W has (H + 2 Kh) * hd rows, hd a multiple of 32.  timescale null: no rotation; slot_mapping null: no
// cache write.
int sa_gemm_normed_rotary(const void* y, const float* h_in, float* h_out, const void* w_post, int w_post_dtype,
                          float eps_post, int plus_one_post, const void* w_next, int w_next_dtype, float eps_next,
                          int plus_one_next, const void* W, void* C, int c_dtype, int64_t ldc, int M, int K,
                          const int* positions, const float* timescale, float scale_factor, float q_div,
                          const int64_t* slot_mapping, void* k_pages, void* v_pages, int H, int Kh, int hd,
                          int page_size, hipStream_t stream);
int sa_gemm_normed(const void* y, const float* h_in, float* h_out, const void* w_post, int w_post_dtype, float eps_post,
                   int plus_one_post, const void* w_next, int w_next_dtype, float eps_next, int plus_one_next,
                   const void* W, void* C, int c_dtype, int64_t ldc, int M, int N, int K, int epilogue, float cap,
                   hipStream_t stream);

// Attention of T query tokens over paged keys and values.
//   q[t, h, :] at q + t * q_stride + h * hd; key pages are [num_pages, Kh, page_size, hd] (each page row-major, or
//   in blocks of operand order if page_size % 16 == 0 and hd % 32 == 0: see key_index in common.h), value pages
//   [num_pages, Kh, hd, page_size];
//   token_seq[t] is the row of block_table of the token's request, positions[t] its absolute position;
//   window 0: all earlier keys, else the last `window` keys including the token's own; soft_cap 0: none.
// algo 0: the library chooses; 1: the generic kernel.
int sa_paged_attention(const void* q, int dtype, int64_t q_stride, const void* k_pages, const void* v_pages,
                       const int* block_table, int table_stride, const int* token_seq, const int* positions, void* out,
                       int64_t out_stride, int T, int H, int Kh, int hd, int page_size, int window, float soft_cap,
                       int algo, hipStream_t stream);

// The same attention for requests seq_begin .. seq_begin + seq_count - 1 of seq_meta (int32 [S, 4]: block-table
// row, index of the request's first token in this step, number of its tokens, position of its first token), each
// with (query heads per key head) * tokens <= 16: bfloat16, head size 64, 128 or 256, page size a multiple of 16.
// max_kv_len bounds the keys of any of them: it is what the cut of the keys into ranges is planned for (num_splits > 0
// fixes the number of ranges).  A request with more keys than that is still computed in full, only slower (its
// ranges are longer than planned; a range of more than 32768 keys is worked through in several passes).
// workspace (bytes): scratch memory for the partial results of the key ranges.
int sa_paged_attention_decode(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                              const int* block_table, int table_stride, const int* seq_meta, int seq_begin,
                              int seq_count, void* out, int64_t out_stride, int H, int Kh, int hd, int page_size,
                              int window, float soft_cap, int max_kv_len, int max_q_len, int num_splits,
                              void* workspace, int64_t workspace_bytes, hipStream_t stream);

// sa_paged_attention_decode for callers that cannot allocate device memory (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc): the same kernels, the same result, but the partial results of
// the key ranges go into an array of sa_paged_attention_decode_static_bytes() bytes (16 MiB) that is part of the
// library's code object, so no workspace is passed and nothing is allocated, by this call or by anything it calls.
// It has no counterpart in the reference (whose attention kernel keeps its scratch inside a compiled program).
// Sizes whose partial results (requests x key heads x key ranges x 16 x (head size + 4) floats, for the number of
// ranges that sa_paged_attention_decode would choose or that num_splits asks for) exceed the array are refused with
// an error, never run with fewer ranges.  Each GPU has one such array, every call on that GPU uses it and leaves
// its partial results there: calls on one GPU that overlap in time (two streams, two threads) race and must be
// ordered by the caller.  Nothing in the array has to be zero beforehand: every word that the merge reads has been
// written by the same call.
int sa_paged_attention_decode_static_bytes();
int sa_paged_attention_decode_static(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                     const int* block_table, int table_stride, const int* seq_meta, int seq_begin,
                                     int seq_count, void* out, int64_t out_stride, int H, int Kh, int hd, int page_size,
                                     int window, float soft_cap, int max_kv_len, int max_q_len, int num_splits,
                                     hipStream_t stream);

// The same for portions of prompts: the units (rows of seq_meta, each with (query heads per key head) * tokens <= 16)
// unit_begin .. unit_begin + unit_count - 1 are taken a group at a time by one workgroup, which reads the keys once
// for all of them.  unit_count is a multiple of the group (sa_paged_attention_prefill_group units) and the units of a
// group belong to one request; units with no tokens fill up a request's last group.
int sa_paged_attention_prefill_group();
// Whether the bfloat16 MFMA attention kernels (sa_paged_attention_decode and _prefill) take these sizes.
int sa_paged_attention_decode_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride, const void* q);
int sa_paged_attention_prefill(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                               const int* block_table, int table_stride, const int* seq_meta, int unit_begin,
                               int unit_count, void* out, int64_t out_stride, int H, int Kh, int hd, int page_size,
                               int window, float soft_cap, int max_kv_len, int max_q_len, int num_splits,
                               void* workspace, int64_t workspace_bytes, hipStream_t stream);

// One token per row of 32-bit logits.  temperature 0 or top_k 1: argmax.  top_k <= 0 and top_p >= 1: off.
// modes: what some row may ask for, as a sum of 1 (a draw: a temperature other than 0), 2 (top-k) and 4 (top-p); 7
// when that is not known.  A row that asks for what modes leaves out gets it all the same, from one workgroup.
// workspace: scratch memory for the kernels that work on large vocabularies in parts (none: one workgroup per row).
int sa_sample(const float* logits, int64_t row_stride, int R, int V, const float* temperature, const int* top_k,
              const float* top_p, const uint64_t* seed, const int* counter, int* tokens, float* logprobs, int modes,
              void* workspace, int64_t workspace_bytes, hipStream_t stream);

// The log-probability of a given token per row under the row's temperature, top-k and top-p (what sa_sample reports
// for the token it draws): 0 or -0.5 * FLT_MAX for greedy rows (the token is the argmax or not), -0.5 * FLT_MAX for
// a token that the masks leave out.  One workgroup per row.
int sa_score(const float* logits, int64_t row_stride, int R, int V, const float* temperature, const int* top_k,
             const float* top_p, const int* tokens, float* scores, hipStream_t stream);

// Host function: one block of the Philox4x32-10 generator that sa_sample uses.
void sa_philox4x32_10(const uint32_t* counter4, const uint32_t* key2, uint32_t* out4);

// Measurements of the machine (the caller times them).  All CUs read `bytes` (a multiple of 8 KiB) of `buffer` once,
// in 8 KiB pieces in their natural order or in the order given (piece numbers, one per piece: the pages of a cache).
// `sink` (512 floats) is never written in practice.
int sa_probe_hbm_read(const void* buffer, int64_t bytes, const int* order, void* sink, hipStream_t stream);
// `workgroups` workgroups of eight waves retire 16 * iters v_mfma_f32_16x16x32_bf16 per wave on operands taken from
// the 16 KiB at `operands`: 2 * 16 * 16 * 32 * 16 * iters * 8 * workgroups floating-point operations.
int sa_probe_mfma(const void* operands, int iters, int workgroups, void* sink, hipStream_t stream);
}

namespace sa {
int gemm_generic(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C,
                 int c_dtype, int64_t ldc, int M, int N, int K, int epi, int act, float cap, int packed,
                 hipStream_t stream);
// x = act(x) in place, row by row (the separate kernel behind products whose kernels have no such epilogue)
int apply_activation(void* x, int dtype, int64_t stride, int M, int N, int act, hipStream_t stream);
bool gemm_skinny_takes(int M, int N, int K, int64_t lda, const void* A, const void* W, const void* W2);
// Expected microseconds of each bfloat16 product kernel for these sizes (epi: 0 none, 1 gated, 2 soft-cap); negative:
// the kernel is not made for them.  The dispatcher runs the kernel with the smallest figure among those that take
// the arguments.
double gemm_skinny_predict_us(int M, int N, int K, int epi);
double gemm_tiled_predict_us(int M, int N, int K, int epi);
double gemm_wide_predict_us(int M, int N, int K, int epi, bool have_workspace, size_t workspace_bytes);
int gemm_skinny(const void* A, int64_t lda, const void* W, const void* W2, void* C, int c_dtype, int64_t ldc, int M,
                int N, int K, int epi, int act, float cap, int packed, int shape, hipStream_t stream);
bool paged_attention_decode_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride, const void* q);
int paged_attention_decode(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                           const int* block_table, int table_stride, const int* seq_meta, int seq_begin, int seq_count,
                           void* out, int64_t out_stride, int H, int Kh, int hd, int page_size, int window,
                           float soft_cap, int max_kv_len, int max_q_len, int num_splits, void* workspace, size_t workspace_bytes,
                           hipStream_t stream, const float* sinks = nullptr, const float* slopes = nullptr);
int paged_attention_prefill_group();  // units that one workgroup takes
bool paged_attention_prefill_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride, const void* q,
                                   int64_t out_stride, const void* out);
int paged_attention_prefill(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* units, int unit_begin, int unit_count,
                            void* out, int64_t out_stride, int H, int Kh, int hd, int page_size, int window,
                            float soft_cap, int max_kv_len, int max_q_len, int num_splits, void* workspace, size_t workspace_bytes,
                            hipStream_t stream, const float* sinks = nullptr, const float* slopes = nullptr);
bool gemm_wide_takes(int M, int N, int K, int64_t lda, int64_t ldc, const void* A, const void* W, const void* W2,
                     const void* C, int c_dtype, int epi, int packed);
int gemm_wide(const void* A, int64_t lda, const void* W, void* C, int64_t ldc, int M, int N, int K, int epi, int act,
              int shape, int ks, void* workspace, size_t workspace_bytes, hipStream_t stream, int* planes_left = nullptr);
// C = epilogue(sum over z of partials[z][M][NW]): the second kernel of every product that cuts K over workgroups
int gemm_sum_partials(const float* partials, int ks, void* C, int c_dtype, int64_t ldc, int M, int N, int NW, int epi,
                      int act, float cap, hipStream_t stream);
bool gemm_streams_weights(int M, int NW, int K);
bool gemm_tiled_takes(int M, int N, int K, int64_t lda, const void* A, const void* W, const void* W2, int packed);
int gemm_tiled(const void* A, int64_t lda, const void* W, void* C, int c_dtype, int64_t ldc, int M, int N, int K,
               int epi, int act, float cap, int ksplit, void* workspace, size_t workspace_bytes, hipStream_t stream);
int paged_attention_generic(const void* q, int dtype, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* token_seq, const int* positions,
                            void* out, int64_t out_stride, int T, int H, int Kh, int hd, int page_size, int window,
                            float soft_cap, hipStream_t stream, int hd_v = 0, float scale = 1.f,
                            const void* sinks = nullptr, int sinks_dtype = 0, int maps = 1, int values_in_keys = 0,
                            int differential = 0, float lambda = 0.f, float eps = 0.f, float mult = 1.f,
                            const float* slopes = nullptr);
}  // namespace sa

extern "C" {
// Attention as sa_paged_attention, for mixers whose values have another size than their keys, whose scores are
// multiplied by `scale` (before the cap, if there is one) and whose softmax may hold one more term per query head,
// exp(sinks[h]), that has no key and no value (sinks null: none).  Value pages are [num_pages, Kh, hd_v, page_size];
// out rows hold H * hd_v elements.  slopes (float32 [H], or null): slopes[h] * (query position - key position) is taken
// off the scaled score.
int sa_paged_attention_sink(const void* q, int dtype, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* token_seq, const int* positions,
                            void* out, int64_t out_stride, int T, int H, int Kh, int hd, int hd_v, int page_size,
                            int window, float soft_cap, float scale, const void* sinks, int sinks_dtype,
                            const float* slopes, hipStream_t stream);

// Attention as sa_paged_attention_sink (no sinks, no cap) with `maps` (1 or 2) score maps per query head: a query row
// holds H * maps vectors of hd entries (head by head, map by map), a key row maps * hd entries (key pages
// [num_pages, Kh, page_size, maps * hd]); every map is a softmax of its own over the same values.
// differential (maps == 2): out [T, H * hd_v] = (a_1 - lambda a_2) / sqrt(mean(.^2) + eps) * mult per head, a_m the
// maps' results; else out [T, H * maps * hd_v] holds every map's result.
// values_in_keys: there are no value pages (v_pages is not read); a key's value is the first hd_v entries of its row.
int sa_paged_attention_maps(const void* q, int dtype, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* token_seq, const int* positions,
                            void* out, int64_t out_stride, int T, int H, int Kh, int hd, int hd_v, int page_size,
                            int window, float scale, int maps, int values_in_keys, int differential, float lambda,
                            float eps, float mult, hipStream_t stream);

// sa_paged_attention_maps in bfloat16 on the matrix cores, over units of few rows (csrc/attention_maps.hip).
int sa_attention_maps_heads_per_unit(int H, int Kh);
int sa_paged_attention_maps_units_takes(int H, int Kh, int maps, int hd, int hd_v, int page_size, int64_t q_stride,
                                        const void* q);
int sa_paged_attention_maps_units(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                  const int* block_table, int table_stride, const int* units, int unit_begin,
                                  int unit_count, void* out, int64_t out_stride, int H, int Kh, int hd, int hd_v,
                                  int page_size, int window, float scale, int maps, int differential, float lambda,
                                  float eps, float mult, int max_kv_len, int max_q_len, void* workspace,
                                  size_t workspace_bytes, hipStream_t stream);

// residual += mult * norm(y; w) (w null: + mult * y; y null: nothing is added), then, if out is not null, out = the
// residual in out's type: the sum of a block that norms what a part returns, and the hand-over to a next part that
// has no norm in front of it.  The norm is y / sqrt(mean(y^2) + eps) * (w + plus_one).
int sa_residual_add_norm(const void* y, int y_dtype, int64_t y_stride, const void* w, int w_dtype, float eps,
                         int plus_one, float mult, float* residual, void* out, int out_dtype, int T, int D,
                         hipStream_t stream);

// out[t, h, :] = (w null ? x[t, h, :] : x[t, h, :] / sqrt(mean(x[t, h, :]^2) + eps) * w) * gate(g[t, h, :]) for H
// heads of `size` elements; w [size] is shared by the heads; gate 0: sigmoid, 1: silu.  out may be x.  gate_per_head: a
// gate row holds H numbers, one for all entries of a head.
int sa_gated_heads(const void* x, int x_dtype, int64_t x_stride, const void* g, int g_dtype, int64_t g_stride,
                   const void* w, int w_dtype, float eps, int gate, void* out, int out_dtype, int64_t out_stride, int T,
                   int H, int size, int gate_per_head, hipStream_t stream);

// x[t, n] = act(x[t, n]) in place (activation codes of activations.h).
int sa_activation(void* x, int dtype, int64_t stride, int T, int N, int act, hipStream_t stream);

// Rows [H * dk queries | K * dk keys | K * dv values | ...] of a fused projection: queries and keys are rotated on
// their first rot_dims dimensions (pairs (i, i + rot_dims / 2), angle position * inv_freq[i]) and then divided by
// sqrt(mean(x^2) + eps) over the head (eps < 0: not); queries, times q_mult, go back in place, keys into the key pages; values
// become (1 - *lambda) v + *lambda v_first[t] (v_first null: stay) and go into the value pages
// [num_pages, K, dv, page_size].  k_pages null: nothing is written.
int sa_qk_norm_rope_cache_write(void* proj, int dtype, int64_t row_stride, const int* positions, const float* inv_freq,
                                int rot_dims, float eps, float q_mult, const void* v_first, int64_t v_first_stride,
                                const void* lambda, int lambda_dtype, const int64_t* slot_mapping, void* k_pages,
                                void* v_pages, int T, int H, int K, int dk, int dv, int page_size, hipStream_t stream);

// residual += mult * y (y null: nothing is added), then out = residual / sqrt(mean(residual^2) + eps) * (w + plus_one):
// the sum of a block whose parts read normed input, with the norm in front of the next part.  Rows of up to 8192.
int sa_residual_add_next_norm(const void* y, int y_dtype, int64_t y_stride, float mult, float* residual, const void* w,
                              int w_dtype, float eps, int plus_one, void* out, int out_dtype, int T, int D,
                              hipStream_t stream);

// On fused projection rows [H * dk queries | K * dk keys | K * dv values | ...]: every query and key vector is cut into
// `sub` equal parts; in each part the first *_norm_dims entries are divided by sqrt(mean of their squares + eps) and
// multiplied by *_weight [>= *_norm_dims] (null: no norm), then the entries [*_rot_at, *_rot_at + rot_dims) turn in
// neighbouring pairs (2p, 2p + 1) by position * freq[p], cos and sin times rot_mult.  Queries go back in place, keys
// into key pages [num_pages, K, page_size, dk], values (dv > 0) into value pages [num_pages, K, dv, page_size].
// k_pages null: nothing is written (then K is best 0).  key_values > 0 (with dv == 0): the first key_values entries of
// every key row, as stored, also go into value pages [num_pages, K, key_values, page_size].
int sa_norm_rope_cache_write(void* proj, int dtype, int64_t row_stride, const int* positions, const float* freq,
                             int rot_dims, float rot_mult, const void* q_weight, int q_norm_dims, int q_rot_at,
                             const void* k_weight, int k_norm_dims, int k_rot_at, int w_dtype, float eps, int sub,
                             const int64_t* slot_mapping, void* k_pages, void* v_pages, int T, int H, int K, int dk,
                             int dv, int page_size, int key_values, hipStream_t stream);

// y[t, c] = act(sum_j taps[c, j] (x[t - (n - 1 - j), c] + in_bias[c]) + out_bias[c]), act silu or none, as
// sa_short_conv_silu below; either bias may be null; the tails hold x + in_bias.  Biases are of bias_dtype.
int sa_short_conv(const void* x, int x_dtype, int64_t x_stride, const void* in_bias, const void* taps, int taps_dtype,
                  int num_taps, const void* out_bias, int bias_dtype, int silu, float* tails, int64_t tail_stride,
                  const int* seq_meta, int num_seqs, int max_q_len, float* y, int C, int update_tails,
                  hipStream_t stream);

// A product per head: out[t, h, o] = sum_i w[h][o][i] x[t, h, i] for o < O (w [H, O, I], row-major), summed in 32-bit
// in the order of i.  x rows hold the heads x_head_stride apart, out rows out_head_stride apart.  tail > 0: the `tail`
// entries behind a head's I inputs are copied behind its O outputs.  gate (null: none): one number per token and head,
// gate[t * gate_stride + h]; the head's outputs are multiplied by sigmoid(gate).
int sa_head_product(const void* x, int x_dtype, int64_t x_stride, int64_t x_head_stride, const void* w, int w_dtype,
                    void* out, int out_dtype, int64_t out_stride, int64_t out_head_stride, int T, int H, int I, int O,
                    int tail, const void* gate, int gate_dtype, int64_t gate_stride, hipStream_t stream);

// The real-gated linear recurrence over each request's tokens (seq_meta [S, 4]: state slot, first row, rows, first
// position), channel by channel, from and into state[slot] [C] float32:
//   r = sigmoid(gr + r_bias), i = sigmoid(gi + i_bias), a = exp(-c r softplus(lam)),
//   S <- a S + sqrt(1 - a^2) i u,   out = S * gelu_tanh(y + y_bias)
// u [T, C] float32; gates [T, C / block] x [gr (block) | gi (block)] float32 (what sa_head_product leaves for the two
// stacked gate matrices of every block); y rows of the activation type; biases and lam of vec_dtype.  max_q_len: the
// most tokens of a request.  Long portions run in segments of tokens side by side, through `scratch` (at least
// num_seqs * (2 * ceil(max_q_len / 64) + 1) * C floats; null or less: one thread walks a request's channel alone).
int sa_rglru_scan(const float* u, const float* gates, int block, const void* r_bias, const void* i_bias, const void* lam,
                  int vec_dtype, float c, const void* y, int y_dtype, int64_t y_stride, const void* y_bias,
                  float* state, int64_t state_stride, const int* seq_meta, int num_seqs, int max_q_len, float* scratch,
                  size_t scratch_floats, void* out, int out_dtype, int C, hipStream_t stream);

// y[t, c] = silu(sum_j taps[c, j] x[t - (n - 1 - j), c]) over each request's tokens (seq_meta [S, 4]: state slot,
// first row, rows, first position), with the inputs before the step's first row taken from tails[slot]
// [n - 1][C] float32, oldest first.  update_tails: afterwards the tails hold each request's last n - 1 inputs.
int sa_short_conv_silu(const void* x, int x_dtype, int64_t x_stride, const void* taps, int taps_dtype, int num_taps,
                       float* tails, int64_t tail_stride, const int* seq_meta, int num_seqs, int max_q_len, float* y,
                       int C, int update_tails, hipStream_t stream);

// In place on qkv [T, C] float32 = [G q heads | G k heads | values]: q and k heads to unit length
// (x / sqrt(sum(x^2) + 1e-6)), q also times dk^(-1/2).  gates [T, 2 H] receives beta = sigmoid(b) and
// g = exp(-exp(a_log) * softplus(a + dt_bias)) from ab [T, a (H) | b (H)].
int sa_delta_prepare(float* qkv, int T, int C, int G, int dk, const void* ab, int ab_dtype, int64_t ab_stride,
                     const void* a_log, const void* dt_bias, int vec_dtype, int H, float* gates, hipStream_t stream);

// sa_short_conv_silu (with the tails updated) and sa_delta_prepare in one launch, for steps in which no request brings
// more than a handful of tokens (sa_delta_inputs_few_takes: decoding): y [T, C] receives the convolved, activated and,
// for the q and k heads, unit-length channels, gates [T, 2 H] beta and g.
int sa_delta_inputs_few_takes(int max_q_len, int dk);
int sa_delta_inputs_few(const void* x, int x_dtype, int64_t x_stride, const void* taps, int taps_dtype, int num_taps,
                        float* tails, int64_t tail_stride, const int* seq_meta, int num_seqs, int max_q_len, float* y,
                        int C, int G, int dk, const void* ab, int ab_dtype, int64_t ab_stride, const void* a_log,
                        const void* dt_bias, int vec_dtype, int H, float* gates, hipStream_t stream);

// The gated delta rule over each request's tokens, from and into state[slot] float32, per head the matrix S [dk, dv]
// stored column by column ([H][dv][dk]): per head
// S <- g S; u = beta (v - S^T k); S <- S + k u^T; out = S^T q.  Value head h reads q/k head h / (H / G).
int sa_delta_rule(const float* qkv, int C, int G, int dk, int dv, const float* gates, int H, float* state,
                  int64_t state_stride, const int* seq_meta, int num_seqs, float* out, hipStream_t stream);

// sa_paged_attention_decode and sa_paged_attention_prefill for softmax sums that hold one more term per query head,
// exp(sinks[h]) (float32 [H]; null: none), without a value, and with slopes (float32 [H]; null: none): slopes[h] times
// the distance between query and key is taken off the score.
int sa_paged_attention_decode_sink(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                   const int* block_table, int table_stride, const int* seq_meta, int seq_begin,
                                   int seq_count, void* out, int64_t out_stride, int H, int Kh, int hd, int page_size,
                                   int window, float soft_cap, int max_kv_len, int max_q_len, int num_splits,
                                   void* workspace, int64_t workspace_bytes, const float* sinks, const float* slopes,
                                    hipStream_t stream);
int sa_paged_attention_prefill_sink(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                    const int* block_table, int table_stride, const int* seq_meta, int unit_begin,
                                    int unit_count, void* out, int64_t out_stride, int H, int Kh, int hd, int page_size,
                                    int window, float soft_cap, int max_kv_len, int max_q_len, int num_splits,
                                    void* workspace, int64_t workspace_bytes, const float* sinks, const float* slopes,
                                    hipStream_t stream);
// ---- token tables
// out[t, :] = table[token] + pair[(previous * mul_prev + token * mul_cur) mod buckets] + pos[position]; a request's
// first token takes the pair table's row `buckets`; the token before a step's first one is last[slot], which is then
// set to the step's last token of the request.  pair, pos: null to leave them out.
int sa_embed_sum(const int* tokens, const int* positions, const int* seq_meta, int num_seqs, int max_q_len,
                 const void* table, int table_dtype, int V, const void* pair, int pair_dtype, int64_t buckets,
                 int64_t mul_prev, int64_t mul_cur, int* last, int64_t last_stride, const void* pos, int pos_dtype,
                 int max_positions, float* out, int D, hipStream_t stream);
// z[t, j] = act(z[t, j]) * table[tokens[t], col0 + j], in place.
int sa_token_gate(void* z, int dtype, int64_t stride, const int* tokens, const void* table, int table_dtype,
                  int64_t table_stride, int col0, int T, int N, int act, hipStream_t stream);
// x[t, n] += b[n], in place.
int sa_bias_add(void* x, int dtype, int64_t stride, const void* b, int b_dtype, int T, int N, hipStream_t stream);
// out = a x + b y.
int sa_weighted_sum(const void* x, int64_t x_stride, float a, const void* y, int64_t y_stride, float b, int dtype,
                    void* out, int64_t out_stride, int T, int N, hipStream_t stream);

// ---- matrix states that decay (linear_state.hip)
// raw [T, 2 H] (input gates, forget gates), bias [2 H] or null -> gates [T, 3 H]: decay, input factor, exp(-m), with
// the running maximum m of every (slot, head) read from and left in m_state[slot * state_stride + h].
int sa_exp_gates(const float* raw, int64_t raw_stride, const void* bias, int bias_dtype, float cap, int H,
                 float* m_state, int64_t state_stride, const int* seq_meta, int num_seqs, float* gates,
                 hipStream_t stream);
// S <- diag(a) S + c k v^T, out = S^T (q * q_mult) along every request's tokens; q, k, v are columns q_at, k_at, v_at
// of proj's rows.  scalar: gates [T, >= 2 H] hold a and c per head; else gates [T, H dk] hold a per key channel and
// c = 1; with tau > 0 these gates are z and a = sigmoid(z + gate_bias)^(1 / tau) (gate_bias [H dk] or null).  ones: the
// state has a column dv whose value is always 1.  state [slot][H][dv + ones][dk]; out [T, H (dv + ones)].
int sa_linear_state(const void* proj, int dtype, int64_t proj_stride, int q_at, int k_at, int v_at, float q_mult,
                    const float* gates, int64_t gates_stride, const void* gate_bias, int bias_dtype, float tau, int scalar,
                    int H, int dk, int dv, int ones, float* state, int64_t state_stride, const int* seq_meta, int num_seqs,
                    float* out, hipStream_t stream);
// x [T, H, size + 1] -> out[t, h, :] = unit_rms(x[t, h, :size] / (max(|x[t, h, size]|, floor[t, h]) + 1e-6)) * w[h, :]
// * sigmoid(g[t, h, :]).
int sa_normalized_readout(const float* x, const float* floor, int64_t floor_stride, const void* g, int g_dtype,
                          int64_t g_stride, const void* w, int w_dtype, float eps, void* out, int out_dtype,
                          int64_t out_stride, int T, int H, int size, hipStream_t stream);

// ---- what an attention kernel reads, from a fused projection (attention_inputs.hip)
// A projection row holds [H * dk queries | K * dk keys | K * dv values | ...] (values_are_keys: no value columns, the
// keys' columns as projected are the values; k_pages null: queries only).  num_taps > 1: every channel passes a causal
// convolution (taps [channels, num_taps] oldest first; tails float32 [slots, (num_taps - 1) * channels], updated).  norm
// 0: none; 1: queries and keys head by head with weights [dk]; 2: over the whole row with weights [H * dk] and
// [K * dk].  Then the first rot_dims entries of every head turn in pairs (i, i + rot_dims / 2) by position *
// inv_freq[i], and queries are multiplied by 1 + temp_coef * ln(floor((position + 1) / temp_every) + 1) (temp_every 0:
// not) and by q_mult.  Queries go to q_out [T, H * dk], keys and values into their pages.  taps_by_tap (or null): the
// taps once more as [num_taps, channels] in their type, which the kernel for aligned bfloat16 rows reads in pieces.
// in_bias (or null; only with num_taps 0): a bias per channel that the projection has not had added yet.
int sa_attention_inputs(const void* proj, int dtype, int64_t row_stride, int H, int K, int dk, int dv, int k_at, int v_at,
                        int values_are_keys, const void* taps, int taps_dtype, int num_taps, float* tails,
                        int64_t tail_stride, int norm, const void* q_w, const void* k_w, int w_dtype, float eps,
                        const float* inv_freq, int rot_dims, float temp_coef, int temp_every, float q_mult,
                        const int* seq_meta, int num_seqs, int max_q_len, const int64_t* slot_mapping, void* q_out, int64_t q_stride,
                        void* k_pages, void* v_pages, int page_size, const void* taps_by_tap, const void* in_bias,
                        int bias_dtype, hipStream_t stream);

// ---- routed experts (routed.hip)
// softmax over E logits, the top largest: experts [T, top], weights [T, top] = score * scale.
int sa_route(const float* logits, int64_t stride, int T, int E, int top, float scale, int* experts, float* weights,
             hipStream_t stream);
// Scores are sigmoids of the logits.  The choice goes by score + correction[e] (null: by the score); the experts form
// `groups` equal groups of neighbours, a group's score is the sum of its two largest choice scores, and only experts of
// the `keep` best groups can be chosen.  weights = score * scale (without the correction, not renormalized).
int sa_route_choice(const float* logits, int64_t stride, int T, int E, int top, float scale, const void* correction,
                    int corr_dtype, int groups, int keep, int* experts, float* weights, hipStream_t stream);
// The most tiles of tile_rows (16 or 64) rows of one expert that P pairs over E experts make.
int sa_expert_tiles_max(int P, int E, int tile_rows);
// sorted [P]: the pairs by expert; plan [1 + 2 * sa_expert_tiles_max(P, E, tile_rows)]: the tiles.
int sa_expert_sort(const int* experts, int P, int E, int tile_rows, int* sorted, int* plan, int plan_words,
                   hipStream_t stream);
// w2 given: out[row] = act(a . w1[e]^T) * (a . w2[e]^T) in a's type; else out[row] = a . w1[e]^T in 32-bit, or, with
// `activate`, act(a . w1[e]^T) in a's type (experts without a gate).  a's row is
// the pair's token (a_by_token) or its place in the sorted order; out's row the pair (out_by_pair) or that place.
// bfloat16 weights are tiled [E][ceil(N / 16)][ceil(K / 32)][64][8], 32-bit ones row-major [E][N][K].
int sa_expert_product(const void* a, int dtype, int64_t a_stride, int a_by_token, int top, const void* w1, const void* w2,
                      int N, int K, const int* sorted, const int* plan, int P, int E, int tile_rows, int act, void* out,
                      int64_t out_stride, int out_by_pair, int activate, hipStream_t stream);
// out[t] = sum_k weights[t, k] y[t * top + k] + sigmoid(gate[t]) * shared[t]  (shared null: none; gate null: 1).
int sa_expert_combine(const float* y, const float* weights, int top, const void* shared, int shared_dtype,
                      int64_t shared_stride, const float* gate, int64_t gate_stride, void* out, int out_dtype,
                      int64_t out_stride, int T, int D, hipStream_t stream);

}
