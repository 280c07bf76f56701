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

extern "C" int sa_gemm(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C,
                       int c_dtype, int64_t ldc, int M, int N, int K, int epilogue, float cap, int algo,
                       hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  SA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  SA_REQUIRE(lda >= K && ldc >= N, "gemm: leading dimensions lda=%lld ldc=%lld are below K=%d, N=%d", (long long)lda,
             (long long)ldc, K, N);
  SA_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm: unknown epilogue %d", epilogue);
  SA_REQUIRE(epilogue != 1 || W2 != nullptr, "gemm: the gated epilogue needs a second weight");
  SA_REQUIRE(epilogue != 2 || cap > 0.f, "gemm: the soft-cap epilogue needs a positive cap");
  SA_REQUIRE(algo >= 0 && algo <= 1, "gemm: unknown algorithm %d", algo);
  return gemm_generic(A, a_dtype, lda, W, W2, w_dtype, C, c_dtype, ldc, M, N, K, epilogue, cap, stream);
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
