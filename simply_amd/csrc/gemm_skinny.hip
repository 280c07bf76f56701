// C[M, N] = epilogue(A[M, K] . W[N, K]^T) in bfloat16 for few rows (M <= 64): the decode step's
// matrix products, which are bound by reading W once from HBM.
//
// Work is cut into (16 weight rows) x (a range of K) units, one per wavefront.  A wave streams its
// 16 rows of W straight from global memory into MFMA operand registers (16-byte loads, each row's
// four lanes reading 64 contiguous bytes), takes the matching activations from the cache hierarchy
// (they are small and shared by all waves), and accumulates with v_mfma_f32_16x16x32_bf16: the
// weight rows are the MFMA's A operand, up to four blocks of 16 activation rows its B operands.
// The four waves of a workgroup take four consecutive K ranges of the same rows and add their
// results through LDS; if K is cut over more workgroups than one (needed to fill 256 CUs when N is
// small), each writes its partial tile to a workspace and the workgroup that finishes last adds
// the partials in a fixed order, so the result does not depend on timing.
#include "api.h"
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

__device__ inline float gelu_tanh_f(float x) {
  const float k = 0.7978845608028654f;
  return 0.5f * x * (1.f + tanhf(k * (x + 0.044715f * x * x * x)));
}

__device__ inline bf16x8 load_frag(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }

constexpr int kUnroll = 4;

template <int MB, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16* __restrict__ A, int64_t lda,
                                                          const bf16* __restrict__ W, const bf16* __restrict__ W2,
                                                          void* __restrict__ C, int c_dtype, int64_t ldc, int M, int N,
                                                          int K, int chunks, float cap, float* __restrict__ workspace,
                                                          unsigned* __restrict__ counters) {
  constexpr int NP = EPI == 1 ? 2 : 1;  // planes: gate and up for the gated epilogue
  __shared__ float red[4][NP][MB][16 * 17];
  __shared__ int is_last_s;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int r = lane % 16, kq = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int S = gridDim.y * 4, s = blockIdx.y * 4 + wave;
  const int c0 = static_cast<int>(static_cast<int64_t>(chunks) * s / S);
  const int c1 = static_cast<int>(static_cast<int64_t>(chunks) * (s + 1) / S);

  floatx4 acc[NP][MB];
#pragma unroll
  for (int p = 0; p < NP; ++p)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[p][mb] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bool row_ok = n0 + r < N;
  const bf16* wrow = W + static_cast<size_t>(row_ok ? n0 + r : 0) * K;
  const bf16* w2row = EPI == 1 ? W2 + static_cast<size_t>(row_ok ? n0 + r : 0) * K : nullptr;
  const bf16x8 zero = {};

  for (int c = c0; c < c1; c += kUnroll) {
    bf16x8 a[kUnroll], a2[kUnroll], b[kUnroll][MB];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int k = (c + u) * 32 + kq * 8;
      const bool ok = c + u < c1 && k < K;
      a[u] = (ok && row_ok) ? load_frag(wrow + k) : zero;
      if (EPI == 1) a2[u] = (ok && row_ok) ? load_frag(w2row + k) : zero;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = mb * 16 + r;
        b[u][mb] = (ok && m < M) ? load_frag(A + static_cast<size_t>(m) * lda + k) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        acc[0][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][mb], acc[0][mb], 0, 0, 0);
        if (EPI == 1) acc[1][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[u], b[u][mb], acc[1][mb], 0, 0, 0);
      }
  }

  // lane holds D[n = 4 * (lane / 16) + v][m = lane % 16]
#pragma unroll
  for (int p = 0; p < NP; ++p)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave][p][mb][(4 * kq + v) * 17 + r] = acc[p][mb][v];
  __syncthreads();

  const int ml = tid / 16, nl = tid % 16;  // this thread's output element within each 16 x 16 block
  float sum[NP][MB];
#pragma unroll
  for (int p = 0; p < NP; ++p)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      sum[p][mb] = ((red[0][p][mb][nl * 17 + ml] + red[1][p][mb][nl * 17 + ml]) + red[2][p][mb][nl * 17 + ml]) +
                   red[3][p][mb][nl * 17 + ml];

  const int KS = gridDim.y;
  const int Mpad = MB * 16;
  if (KS > 1) {
    // partial tile -> workspace[plane][split][m][n]; the last workgroup of this tile adds them up in order
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        if (n0 + nl < N)
          workspace[((static_cast<size_t>(p) * KS + blockIdx.y) * Mpad + mb * 16 + ml) * N + n0 + nl] = sum[p][mb];
    __threadfence();
    __syncthreads();
    if (tid == 0) is_last_s = atomicAdd(&counters[blockIdx.x], 1u) == static_cast<unsigned>(KS - 1);
    __syncthreads();
    if (!is_last_s) return;
    __threadfence();
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        float t = 0.f;
        if (n0 + nl < N)
          for (int y = 0; y < KS; ++y)
            t += __builtin_nontemporal_load(
                &workspace[((static_cast<size_t>(p) * KS + y) * Mpad + mb * 16 + ml) * N + n0 + nl]);
        sum[p][mb] = t;
      }
    if (tid == 0) counters[blockIdx.x] = 0u;  // ready for the next launch
  }

#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + ml, n = n0 + nl;
    if (m >= M || n >= N) continue;
    float v = sum[0][mb];
    if (EPI == 1) {
      // both products are rounded to bfloat16 first, as separate matrix products would be
      v = gelu_tanh_f(to_float(float_to_bf16(v))) * to_float(float_to_bf16(sum[NP - 1][mb]));
    } else if (EPI == 2) {
      v = cap * tanhf(v / cap);
    }
    store_f(C, c_dtype, static_cast<size_t>(m) * ldc + n, v);
  }
}

// How many ways to cut K (a multiple of 4: the waves of a workgroup), so that about 8 waves per CU are in
// flight and no wave gets less than two 32-wide chunks.
static int choose_splits(int tiles, int chunks, int planes) {
  const int target_waves = 256 * 12;
  int S = (target_waves + tiles - 1) / tiles;
  S = (S + 3) / 4 * 4;
  const int max_s = chunks * planes / 2;  // at least ~2 KB of weights per wave
  if (S > max_s) S = max_s / 4 * 4;
  if (S < 4) S = 4;
  if (S > 64) S = 64;
  return S;
}

template <int MB>
static void launch_skinny(const bf16* A, int64_t lda, const bf16* W, const bf16* W2, void* C, int c_dtype, int64_t ldc,
                          int M, int N, int K, int epi, float cap, float* ws, unsigned* counters, int S,
                          hipStream_t stream) {
  const int chunks = (K + 31) / 32;
  const dim3 grid((N + 15) / 16, S / 4);
  if (epi == 0)
    gemm_skinny_kernel<MB, 0><<<grid, 256, 0, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K, chunks, cap, ws,
                                                        counters);
  else if (epi == 1)
    gemm_skinny_kernel<MB, 1><<<grid, 256, 0, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K, chunks, cap, ws,
                                                        counters);
  else
    gemm_skinny_kernel<MB, 2><<<grid, 256, 0, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K, chunks, cap, ws,
                                                        counters);
}

bool gemm_skinny_takes(int M, int N, int K, int64_t lda, const void* A, const void* W, const void* W2) {
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  return M >= 1 && M <= 64 && K % 8 == 0 && lda % 8 == 0 && aligned(A) && aligned(W) && (W2 == nullptr || aligned(W2));
}

int gemm_skinny(const void* A, int64_t lda, const void* W, const void* W2, void* C, int c_dtype, int64_t ldc, int M,
                int N, int K, int epi, float cap, void* workspace, size_t workspace_bytes, void* counters,
                int num_counters, int splits, hipStream_t stream) {
  const int tiles = (N + 15) / 16, chunks = (K + 31) / 32, planes = epi == 1 ? 2 : 1;
  int S = splits > 0 ? (splits + 3) / 4 * 4 : choose_splits(tiles, chunks, planes);
  if (S > chunks) S = (chunks + 3) / 4 * 4;
  if (S < 4) S = 4;
  // fewer cuts if the workspace cannot hold the partial tiles (none needed with one workgroup per tile)
  const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);  // as the kernel's template pads it
  const size_t per_split = static_cast<size_t>(planes) * Mpad * N * sizeof(float);
  while (S > 4 && (workspace == nullptr || counters == nullptr || tiles > num_counters ||
                   per_split * (S / 4) > workspace_bytes))
    S -= 4;
  const bf16* a = static_cast<const bf16*>(A);
  const bf16* w = static_cast<const bf16*>(W);
  const bf16* w2 = static_cast<const bf16*>(W2);
  float* ws = static_cast<float*>(workspace);
  unsigned* cn = static_cast<unsigned*>(counters);
  if (M <= 16) launch_skinny<1>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, epi, cap, ws, cn, S, stream);
  else if (M <= 32) launch_skinny<2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, epi, cap, ws, cn, S, stream);
  else launch_skinny<4>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, epi, cap, ws, cn, S, stream);
  return check_launch("gemm_skinny");
}

}  // namespace sa
