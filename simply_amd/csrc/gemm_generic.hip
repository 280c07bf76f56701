// C[M, N] = epilogue(A[M, K] . W[N, K]^T): the matrix product for every size and
// both element types, on the vector ALU in 32-bit (products and sums in float,
// no reduced-precision matrix mode).  Each output element is summed over k in
// increasing order whatever M is, so a row's result does not depend on which
// other rows are in the batch.  This is the kernel of the 32-bit path and the
// fallback of the bfloat16 path for shapes that the MFMA kernels refuse.
#include "api.h"
#include "common.h"

namespace sa {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

// Index of W[n][k] in memory: row-major, or tiled [N / 16][chunks][kq 4][row 16][8] (chunks = ceil(K / 32)).  With
// `paired` (the gated epilogue on tiled weights) the tiles of the gate and of the other factor alternate: the gate's
// tile n / 16 is tile 2 (n / 16), the factor's follows it.
template <bool PACKED>
__device__ inline size_t w_index(int n, int k, int K, int chunks, int paired = 0, int second = 0) {
  if (!PACKED) return static_cast<size_t>(n) * K + k;
  const size_t tile = paired ? 2 * static_cast<size_t>(n / 16) + second : static_cast<size_t>(n / 16);
  return ((tile * chunks + k / 32) * 64 + ((k % 32) / 8) * 16 + n % 16) * 8 + k % 8;
}

// EPI: 0 plain, 1 gated (C = act(A.W^T) * (A.W2^T)), 2 soft-cap (C = cap * tanh(A.W^T / cap))
template <typename TA, typename TW, typename TC, int EPI, bool PACKED>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A, int64_t lda,
                                                           const TW* __restrict__ W, const TW* __restrict__ W2,
                                                           TC* __restrict__ C, int64_t ldc, int M, int N, int K,
                                                           float cap, int act) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  __shared__ float W2s[EPI == 1 ? BK : 1][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[TM][TN] = {};
  float acc2[EPI == 1 ? TM : 1][TN] = {};
  const int chunks = (K + 31) / 32;
  const int lr = tid / 4;         // tile row 0..63
  const int lk = (tid % 4) * 4;   // k offset 0,4,8,12
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      const int m = m0 + lr, n = n0 + lr;
      As[lk + i][lr] = (m < M && k < K) ? to_float(A[static_cast<size_t>(m) * lda + k]) : 0.f;
      Ws[lk + i][lr] = (n < N && k < K) ? to_float(W[w_index<PACKED>(n, k, K, chunks, EPI == 1, 0)]) : 0.f;
      if (EPI == 1)
        W2s[lk + i][lr] = (n < N && k < K) ? to_float((PACKED ? W : W2)[w_index<PACKED>(n, k, K, chunks, 1, 1)]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[TM], b[TN], b2[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[k][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Ws[k][tx * TN + j];
      if (EPI == 1) {
#pragma unroll
        for (int j = 0; j < TN; ++j) b2[j] = W2s[k][tx * TN + j];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
          if (EPI == 1) acc2[i][j] = fmaf(a[i], b2[j], acc2[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (EPI == 1) {
        // both products are rounded to the activation type first, as separate matrix products would be
        v = gated_activation_exact(act, to_float(from_float<TC>(v))) * to_float(from_float<TC>(acc2[i][j]));
      } else if (EPI == 2) {
        v = cap * tanhf(v / cap);
      }
      C[static_cast<size_t>(m) * ldc + n] = from_float<TC>(v);
    }
  }
}

template <typename TA, typename TW, typename TC, bool PACKED>
static void launch_generic(const void* A, int64_t lda, const void* W, const void* W2, void* C, int64_t ldc, int M, int N,
                           int K, int epi, int act, float cap, hipStream_t stream) {
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  const TA* a = static_cast<const TA*>(A);
  const TW* w = static_cast<const TW*>(W);
  const TW* w2 = static_cast<const TW*>(W2);
  TC* c = static_cast<TC*>(C);
  if (epi == 0)
    gemm_generic_kernel<TA, TW, TC, 0, PACKED><<<grid, 256, 0, stream>>>(a, lda, w, w2, c, ldc, M, N, K, cap, act);
  else if (epi == 1)
    gemm_generic_kernel<TA, TW, TC, 1, PACKED><<<grid, 256, 0, stream>>>(a, lda, w, w2, c, ldc, M, N, K, cap, act);
  else
    gemm_generic_kernel<TA, TW, TC, 2, PACKED><<<grid, 256, 0, stream>>>(a, lda, w, w2, c, ldc, M, N, K, cap, act);
}

int gemm_generic(const void* A, int a_dtype, int64_t lda, const void* W, const void* W2, int w_dtype, void* C,
                 int c_dtype, int64_t ldc, int M, int N, int K, int epi, int act, float cap, int packed,
                 hipStream_t stream) {
  if (a_dtype == kF32 && w_dtype == kF32 && c_dtype == kF32 && !packed)
    launch_generic<float, float, float, false>(A, lda, W, W2, C, ldc, M, N, K, epi, act, cap, stream);
  else if (a_dtype == kBF16 && w_dtype == kBF16 && c_dtype == kBF16 && !packed)
    launch_generic<bf16, bf16, bf16, false>(A, lda, W, W2, C, ldc, M, N, K, epi, act, cap, stream);
  else if (a_dtype == kBF16 && w_dtype == kBF16 && c_dtype == kF32 && !packed)
    launch_generic<bf16, bf16, float, false>(A, lda, W, W2, C, ldc, M, N, K, epi, act, cap, stream);
  else if (a_dtype == kBF16 && w_dtype == kBF16 && c_dtype == kBF16 && packed)
    launch_generic<bf16, bf16, bf16, true>(A, lda, W, W2, C, ldc, M, N, K, epi, act, cap, stream);
  else if (a_dtype == kBF16 && w_dtype == kBF16 && c_dtype == kF32 && packed)
    launch_generic<bf16, bf16, float, true>(A, lda, W, W2, C, ldc, M, N, K, epi, act, cap, stream);
  else {
    set_error("gemm: unsupported element types a=%d w=%d c=%d (tiled weights: bfloat16 only)", a_dtype, w_dtype,
              c_dtype);
    return 1;
  }
  return check_launch("gemm_generic");
}

}  // namespace sa
