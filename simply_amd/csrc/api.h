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
// type first; 2: cap * tanh(. / cap).  algo 0: the library chooses; 1: the generic 32-bit-ALU kernel; 2: the
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
                           hipStream_t stream);
int paged_attention_prefill_group();  // units that one workgroup takes
bool paged_attention_prefill_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride, const void* q,
                                   int64_t out_stride, const void* out);
int paged_attention_prefill(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* units, int unit_begin, int unit_count,
                            void* out, int64_t out_stride, int H, int Kh, int hd, int page_size, int window,
                            float soft_cap, int max_kv_len, int max_q_len, int num_splits, void* workspace, size_t workspace_bytes,
                            hipStream_t stream);
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
                            float soft_cap, hipStream_t stream);
}  // namespace sa
