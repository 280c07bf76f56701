// Error channel and dispatch of the C entry points.
#include <stdarg.h>
#include <stdio.h>

#include "api.h"
#include "common.h"

namespace sa {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return 1;
  }
  return 0;
}

}  // namespace sa

using namespace sa;

extern "C" const char* sa_last_error() { return g_error; }
extern "C" int sa_version() { return 1; }

static int gemm_routed(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C,
                       int c_dtype, int64_t ldc, int M, int N, int K, int epilogue, float cap, int algo,
                       int packed, int shape, void* workspace, int64_t workspace_bytes, int* planes_left,
                       hipStream_t stream) {
  if (planes_left != nullptr) *planes_left = 1;
  if (M == 0 || N == 0) return 0;
  SA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  SA_REQUIRE(lda >= K && ldc >= N, "gemm: leading dimensions lda=%lld ldc=%lld are below K=%d, N=%d", (long long)lda,
             (long long)ldc, K, N);
  const int act = epilogue_activation(epilogue);
  epilogue = epilogue_kind(epilogue);
  SA_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm: unknown epilogue %d", epilogue);
  SA_REQUIRE(act >= 0 && act < kNumActivations && (epilogue == 1 || act == 0), "gemm: unknown activation %d", act);
  SA_REQUIRE(epilogue != 1 || (W2 != nullptr) != (packed != 0),
             "gemm: the gated epilogue takes two row-major weights, or one tiled weight that holds both");
  SA_REQUIRE(epilogue != 2 || cap > 0.f, "gemm: the soft-cap epilogue needs a positive cap");
  SA_REQUIRE(algo >= 0 && algo <= 4, "gemm: unknown algorithm %d", algo);
  const bool bf16_in = a_dtype == kBF16 && w_dtype == kBF16;
  // up to 16 rows, and up to 32 for products without the gated epilogue and with K below 4096 (measured at the
  // 2B, 9B and 27B sizes: the few-rows kernel, whose waves read the activations from L2, beats the kernels with
  // K cut over workgroups there; for longer K, the down projections, it is up to 2x slower).  Not from 8 rows on
  // against so many weight rows that the tiled kernel fills the GPU without a cut of K (the head over a large
  // vocabulary: 7 % faster at 8 rows, 30 % at 16, 80 % at 32; up to 6 rows the few-rows kernel wins).
  // Nor against a very long K (the 27B down projection, 36864: kernels that cut K over workgroups are 15 % faster at
  // one row and 40 % at 16), nor from 9 rows on against K of 8192 and more (the 2B and 9B down projections: the
  // wide kernel with its cut takes 13.0 against 16.8 us and 24.2 against 26.7 at 16 rows; up to 8 rows, where a
  // load of activations serves several chunks of K, the few-rows kernel wins).
  const bool many_weight_rows = packed && epilogue != 1 && M >= 8 && N >= 65536;
  const bool long_k = packed && epilogue != 1 && K >= 24576;
  // (... or against K of 4096 and more where the weight is large, 16 M elements: 27B q/k/v 16.0 against 18.6 us at
  // 16 rows; the same size decides for 17 to 32 rows: 9B q/k/v 16.0 against 22.5 us at 32 rows with the wide kernel,
  // 2B q/k/v 9.5 against 9.8 with the few-rows kernel)
  const bool large = static_cast<int64_t>(N) * K >= (int64_t{16} << 20);
  const bool longish_k = packed && epilogue == 0 && M >= 9 && N <= 16384 && (K >= 8192 || (K >= 4096 && large));
  const bool tiled_first = many_weight_rows || long_k;
  if (algo == 2 ||
      (algo == 0 && bf16_in && !tiled_first && !longish_k &&
       (M <= 16 || (M <= 32 && epilogue != 1 && K < 4096 && !(packed && epilogue == 0 && large && N <= 16384))))) {
    const bool takes = bf16_in && gemm_skinny_takes(M, N, K, lda, A, W, W2);
    SA_REQUIRE(takes || algo == 0,
               "gemm: the few-rows kernel takes bfloat16 with M <= 64, K and lda multiples of 8 and 16-byte aligned "
               "operands; got M=%d K=%d lda=%lld", M, K, (long long)lda);
    if (takes)
      return gemm_skinny(A, lda, W, W2, C, c_dtype, ldc, M, N, K, epilogue, act, cap, packed, shape, stream);
  }
  // once the product is no longer bound by streaming the weights: the wide tiles (both operands through LDS); and
  // the gated product from 17 rows on, whose very many weight rows fill the GPU with the wide kernel's workgroups
  // without a cut of K (measured at 32 and 64 rows: 10-20 % faster than the tiled kernel with its sum kernel at the
  // 2B, 9B and 27B sizes)
  const int NW = epilogue == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  // 17 to 1,536 rows without an epilogue (q/k/v, output and down projections of portions of prompts and of many
  // decoding requests): the wide kernel with a tile and a cut of K that it chooses for the sizes (2B down projection:
  // 13 us at 17 rows, 15 at 64, 36 at 512, against 19, 23 and 55 for the tiled kernel with its cut)
  // ... and up to 16 rows against a very long K (the 27B down projection: 62 us against 67 for the tiled kernel
  // with its cut and 74 to 84 for the few-rows kernel)
  const bool small_wide = epilogue == 0 && N <= 16384 && ((M >= 17 && M <= 1536) || (long_k && M <= 16) || longish_k);
  const bool wide_first = !gemm_streams_weights(M, NW, K) || (epilogue == 1 && M > 16) || small_wide;
  if (algo == 4 || (algo == 0 && bf16_in && packed && wide_first)) {
    const bool takes = bf16_in && gemm_wide_takes(M, N, K, lda, ldc, A, W, W2, C, c_dtype, epilogue, packed);
    SA_REQUIRE(takes || algo == 0,
               "gemm: the wide MFMA kernel takes bfloat16 in and out with tiled weights, no soft-cap, K a multiple of "
               "64, N and ldc of 4, lda of 8; got N=%d K=%d lda=%lld ldc=%lld tiled=%d", N, K, (long long)lda,
               (long long)ldc, packed);
    // (a shape given by the caller may carry a cut of K in front: cuts * 10000000 + shape)
    if (takes)
      return gemm_wide(A, lda, W, C, ldc, M, N, K, epilogue, act, algo == 4 ? shape % 10000000 : 0,
                       algo == 4 ? shape / 10000000 : 1, workspace,
                       static_cast<size_t>(workspace_bytes < 0 ? 0 : workspace_bytes), stream, planes_left);
  }
  if (algo == 3 || (algo == 0 && bf16_in && packed && (M > 16 || tiled_first))) {
    const bool takes = bf16_in && gemm_tiled_takes(M, N, K, lda, A, W, W2, packed);
    SA_REQUIRE(takes || algo == 0,
               "gemm: the tiled MFMA kernel takes bfloat16 with tiled weights, K and lda multiples of 8 and 16-byte "
               "aligned operands; got K=%d lda=%lld tiled=%d", K, (long long)lda, packed);
    if (takes)
      return gemm_tiled(A, lda, W, C, c_dtype, ldc, M, N, K, epilogue, act, cap, shape, workspace,
                        static_cast<size_t>(workspace_bytes < 0 ? 0 : workspace_bytes), stream);
  }
  return gemm_generic(A, a_dtype, lda, W, W2, w_dtype, C, c_dtype, ldc, M, N, K, epilogue, act, cap, packed, stream);
}

extern "C" int sa_gemm(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C,
                       int c_dtype, int64_t ldc, int M, int N, int K, int epilogue, float cap, int algo,
                       int packed, int shape, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  return gemm_routed(A, a_dtype, lda, W, W2, w_dtype, C, c_dtype, ldc, M, N, K, epilogue, cap, algo, packed, shape,
                     workspace, workspace_bytes, nullptr, stream);
}

extern "C" int sa_sum_planes(const float* planes, int count, void* C, int c_dtype, int64_t ldc, int M, int N,
                             hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  SA_REQUIRE(planes != nullptr && count >= 1 && M > 0 && N > 0 && ldc >= N, "sum_planes: bad sizes %d x [%d, %d]",
             count, M, N);
  return gemm_sum_partials(planes, count, C, c_dtype, ldc, M, N, N, 0, 0, 0.f, stream);
}

extern "C" int sa_gemm_planes(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype,
                              void* C, int c_dtype, int64_t ldc, int M, int N, int K, int epilogue, float cap,
                              int algo, int packed, int shape, void* workspace, int64_t workspace_bytes, int* planes,
                              hipStream_t stream) {
  SA_REQUIRE(planes != nullptr, "gemm_planes: nowhere to put the number of planes");
  return gemm_routed(A, a_dtype, lda, W, W2, w_dtype, C, c_dtype, ldc, M, N, K, epilogue, cap, algo, packed, shape,
                     workspace, workspace_bytes, planes, stream);
}

extern "C" int sa_paged_attention(const void* q, int dtype, int64_t q_stride, const void* k_pages,
                                  const void* v_pages, const int* block_table, int table_stride, const int* token_seq,
                                  const int* positions, void* out, int64_t out_stride, int T, int H, int Kh, int hd,
                                  int page_size, int window, float soft_cap, int algo, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(dtype == kF32 || dtype == kBF16, "paged_attention: unknown dtype %d", dtype);
  SA_REQUIRE(T > 0 && H > 0 && Kh > 0 && hd > 0 && page_size > 0, "paged_attention: bad sizes T=%d H=%d K=%d hd=%d P=%d",
             T, H, Kh, hd, page_size);
  SA_REQUIRE(H % Kh == 0, "paged_attention: %d query heads do not split over %d key heads", H, Kh);
  SA_REQUIRE(q_stride >= static_cast<int64_t>(H) * hd && out_stride >= static_cast<int64_t>(H) * hd,
             "paged_attention: row strides are below heads * head size");
  SA_REQUIRE(window >= 0 && table_stride > 0, "paged_attention: bad window or table stride");
  SA_REQUIRE(algo >= 0 && algo <= 1, "paged_attention: unknown algorithm %d", algo);
  return paged_attention_generic(q, dtype, q_stride, k_pages, v_pages, block_table, table_stride, token_seq, positions,
                                 out, out_stride, T, H, Kh, hd, page_size, window, soft_cap, stream);
}

extern "C" int sa_paged_attention_decode(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                         const int* block_table, int table_stride, const int* seq_meta, int seq_begin,
                                         int seq_count, void* out, int64_t out_stride, int H, int Kh, int hd,
                                         int page_size, int window, float soft_cap, int max_kv_len, int max_q_len,
                                         int num_splits, void* workspace, int64_t workspace_bytes,
                                         hipStream_t stream) {
  if (seq_count == 0) return 0;
  SA_REQUIRE(seq_count > 0 && seq_begin >= 0 && H > 0 && Kh > 0 && H % Kh == 0, "paged_attention_decode: bad counts");
  SA_REQUIRE(window >= 0 && table_stride > 0 && max_kv_len > 0, "paged_attention_decode: bad window, table or length");
  SA_REQUIRE(paged_attention_decode_takes(H, Kh, hd, page_size, max_q_len, q_stride, q),
             "paged_attention_decode takes head size 64, 128 or 256, a page size that is a multiple of 16 and "
             "(heads per key head) * tokens <= 16; got hd=%d P=%d G=%d tokens=%d", hd, page_size, H / Kh, max_q_len);
  SA_REQUIRE(out_stride >= static_cast<int64_t>(H) * hd, "paged_attention_decode: output rows are too short");
  return paged_attention_decode(q, q_stride, k_pages, v_pages, block_table, table_stride, seq_meta, seq_begin, seq_count,
                                out, out_stride, H, Kh, hd, page_size, window, soft_cap, max_kv_len, max_q_len, num_splits,
                                workspace, static_cast<size_t>(workspace_bytes < 0 ? 0 : workspace_bytes), stream);
}

extern "C" int sa_paged_attention_decode_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride,
                                               const void* q) {
  return H > 0 && Kh > 0 && H % Kh == 0 && paged_attention_decode_takes(H, Kh, hd, page_size, max_q_len, q_stride, q);
}

extern "C" int sa_paged_attention_prefill_group() { return paged_attention_prefill_group(); }

extern "C" int sa_paged_attention_prefill(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                          const int* block_table, int table_stride, const int* seq_meta, int unit_begin,
                                          int unit_count, void* out, int64_t out_stride, int H, int Kh, int hd,
                                          int page_size, int window, float soft_cap, int max_kv_len, int max_q_len,
                                          int num_splits, void* workspace, int64_t workspace_bytes,
                                          hipStream_t stream) {
  if (unit_count == 0) return 0;
  SA_REQUIRE(unit_count > 0 && unit_count % paged_attention_prefill_group() == 0 && unit_begin >= 0 && H > 0 && Kh > 0 &&
                 H % Kh == 0,
             "paged_attention_prefill: bad counts (units come in groups of %d)", paged_attention_prefill_group());
  SA_REQUIRE(window >= 0 && table_stride > 0 && max_kv_len > 0, "paged_attention_prefill: bad window, table or length");
  SA_REQUIRE(paged_attention_prefill_takes(H, Kh, hd, page_size, max_q_len, q_stride, q, out_stride, out),
             "paged_attention_prefill takes head size 64, 128 or 256, a page size that is a multiple of 16 and "
             "(heads per key head) * tokens <= 16 per unit; got hd=%d P=%d G=%d tokens=%d", hd, page_size, H / Kh,
             max_q_len);
  SA_REQUIRE(out_stride >= static_cast<int64_t>(H) * hd, "paged_attention_prefill: output rows are too short");
  return paged_attention_prefill(q, q_stride, k_pages, v_pages, block_table, table_stride, seq_meta, unit_begin,
                                 unit_count, out, out_stride, H, Kh, hd, page_size, window, soft_cap, max_kv_len,
                                 max_q_len, num_splits, workspace, static_cast<size_t>(workspace_bytes < 0 ? 0 : workspace_bytes),
                                 stream);
}
