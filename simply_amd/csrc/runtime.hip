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
  const size_t ws_bytes = static_cast<size_t>(workspace_bytes < 0 ? 0 : workspace_bytes);
  // Which of the three bfloat16 kernels take these arguments; a kernel that the caller names must take them.
  const bool skinny_ok = bf16_in && gemm_skinny_takes(M, N, K, lda, A, W, W2);
  const bool wide_ok = bf16_in && gemm_wide_takes(M, N, K, lda, ldc, A, W, W2, C, c_dtype, epilogue, packed);
  const bool tiled_ok = bf16_in && gemm_tiled_takes(M, N, K, lda, A, W, W2, packed);
  SA_REQUIRE(algo != 2 || skinny_ok,
             "gemm: the few-rows kernel takes bfloat16 with M <= 64, K and lda multiples of 8 and 16-byte aligned "
             "operands; got M=%d K=%d lda=%lld", M, K, (long long)lda);
  SA_REQUIRE(algo != 4 || wide_ok,
             "gemm: the wide MFMA kernel takes bfloat16 in and out with tiled weights, no soft-cap, K a multiple of "
             "64, N and ldc of 4, lda of 8; got N=%d K=%d lda=%lld ldc=%lld tiled=%d", N, K, (long long)lda,
             (long long)ldc, packed);
  SA_REQUIRE(algo != 3 || tiled_ok,
             "gemm: the tiled MFMA kernel takes bfloat16 with tiled weights, K and lda multiples of 8 and 16-byte "
             "aligned operands; got K=%d lda=%lld tiled=%d", K, (long long)lda, packed);
  int kernel = algo;
  if (algo == 0) {
    // The kernel that is expected to be fastest: every kernel says how long it expects to take for these sizes (a
    // model of its own time, fitted to measurements, beside its code), and the smallest figure wins.  No size of any
    // model stands here.
    kernel = 1;
    double best = -1.0;
    const double us[3] = {skinny_ok ? gemm_skinny_predict_us(M, N, K, epilogue) : -1.0,
                          tiled_ok ? gemm_tiled_predict_us(M, N, K, epilogue) : -1.0,
                          wide_ok ? gemm_wide_predict_us(M, N, K, epilogue, workspace != nullptr, ws_bytes) : -1.0};
    for (int i = 0; i < 3; ++i)
      if (us[i] >= 0.0 && (best < 0.0 || us[i] < best)) {
        best = us[i];
        kernel = 2 + i;
      }
  }
  if (kernel == 2)
    return gemm_skinny(A, lda, W, W2, C, c_dtype, ldc, M, N, K, epilogue, act, cap, packed, shape, stream);
  // (a shape given by the caller for the wide kernel may carry a cut of K in front: cuts * 10000000 + shape)
  if (kernel == 4)
    return gemm_wide(A, lda, W, C, ldc, M, N, K, epilogue, act, algo == 4 ? shape % 10000000 : 0,
                     algo == 4 ? shape / 10000000 : 1, workspace, ws_bytes, stream, planes_left);
  if (kernel == 3)
    return gemm_tiled(A, lda, W, C, c_dtype, ldc, M, N, K, epilogue, act, cap, shape, workspace, ws_bytes, stream);
  return gemm_generic(A, a_dtype, lda, W, W2, w_dtype, C, c_dtype, ldc, M, N, K, epilogue, act, cap, packed, stream);
}

extern "C" int sa_gemm(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C,
                       int c_dtype, int64_t ldc, int M, int N, int K, int epilogue, float cap, int algo,
                       int packed, int shape, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  return gemm_routed(A, a_dtype, lda, W, W2, w_dtype, C, c_dtype, ldc, M, N, K, epilogue, cap, algo, packed, shape,
                     workspace, workspace_bytes, nullptr, stream);
}

extern "C" int sa_gemm_plan(int M, int N, int K, int epilogue, int c_dtype, int64_t workspace_bytes, double* us_out) {
  if (M < 1 || N < 1 || K < 1) return 0;
  const int epi = epilogue_kind(epilogue);
  const size_t ws_bytes = static_cast<size_t>(workspace_bytes < 0 ? 0 : workspace_bytes);
  alignas(16) static const char aligned_stand_in[16] = {};   // an address that every alignment test passes
  const void* p = aligned_stand_in;
  const int64_t lda = K, ldc = N;
  const bool skinny_ok = gemm_skinny_takes(M, N, K, lda, p, p, nullptr);
  const bool wide_ok = gemm_wide_takes(M, N, K, lda, ldc, p, p, nullptr, p, c_dtype, epi, 1);
  const bool tiled_ok = gemm_tiled_takes(M, N, K, lda, p, p, nullptr, 1);
  const double us[3] = {skinny_ok ? gemm_skinny_predict_us(M, N, K, epi) : -1.0,
                        tiled_ok ? gemm_tiled_predict_us(M, N, K, epi) : -1.0,
                        wide_ok ? gemm_wide_predict_us(M, N, K, epi, ws_bytes > 0, ws_bytes) : -1.0};
  int kernel = 1;
  double best = -1.0;
  for (int i = 0; i < 3; ++i) {
    if (us_out != nullptr) us_out[i] = us[i];
    if (us[i] >= 0.0 && (best < 0.0 || us[i] < best)) {
      best = us[i];
      kernel = 2 + i;
    }
  }
  return kernel;
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
