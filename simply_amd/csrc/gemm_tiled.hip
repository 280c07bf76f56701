// C[M, N] = epilogue(A[M, K] . W[N, K]^T) in bfloat16 for many rows (portions of prompts): bound by
// the MFMA units.  W is in the tiled layout (16 x 32 blocks in MFMA operand order, see
// simply_amd/kernels/packing.py), A is row-major.
//
// A workgroup of four waves (2 x 2) owns BM x 128 outputs; a wave owns (WM * 16) x 64 of them as WM x 4
// tiles of v_mfma_f32_16x16x32_bf16.  Per step of 32 along K a wave needs WM fragments of A and 4 of W:
//   * A goes through LDS: the workgroup copies a BM x 64 slab with 16-byte loads (eight lanes per row:
//     whole 128-byte lines), one slab ahead in registers while the current one is multiplied; rows are
//     padded to 144 bytes so that the fragment reads (ds_read_b128) hit all 64 banks once.
//   * W fragments are loaded straight from global memory into operand registers (a fragment is one
//     contiguous KiB of the tiled layout), one step ahead, and never touch LDS.
// With WM = 8 this is 8 KiB of LDS reads and 4 KiB of global loads per 32 MFMAs (512 cycles) and wave:
// half of a CU's LDS and L1 bandwidth.
//
// Epilogues: none; gated (two weight matrices, C = gelu_tanh(A.W^T) * (A.W2^T), both rounded to bfloat16
// first); soft-cap (C = cap * tanh(. / cap), float32 out).
#include "api.h"
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

namespace tiled {

constexpr int BK = 64;          // columns of A per LDS slab
constexpr int PITCH = BK + 8;   // elements per LDS row: 144 bytes

__device__ inline float gelu_tanh_f(float x) {
  const float k = 0.7978845608028654f;
  return 0.5f * x * (1.f + tanhf(k * (x + 0.044715f * x * x * x)));
}

// WAVES_N: 2 = waves as 2 x 2 (BM = 2 * WM * 16 rows, 128 columns); 4 = waves as 1 x 4 (BM = WM * 16 rows, 256
// columns: for few rows, every W fragment is loaded by one wave only).  gridDim.z > 1 cuts K over workgroups: each
// writes its float32 partial tile to `partials` [z][plane][M][N] and gemm_reduce_kernel adds them up.
template <int WM, int PLANES, int EPI, int WAVES_N>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16* __restrict__ A, int64_t lda,
                                                         const bf16* __restrict__ W, const bf16* __restrict__ W2,
                                                         void* __restrict__ C, int c_dtype, int64_t ldc, int M, int N,
                                                         int K, int chunks, float cap, float* __restrict__ partials) {
  constexpr int WAVES_M = 4 / WAVES_N;
  constexpr int BM = WAVES_M * WM * 16;
  constexpr int BNW = WAVES_N * 64;  // output columns per workgroup
  constexpr int APT = (BM + 31) / 32;  // 16-byte pieces of a slab per thread
  __shared__ __attribute__((aligned(16))) bf16 As[BM * PITCH];

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int r = lane % 16, grp = lane / 16;
  const int m_base = blockIdx.y * BM;
  const int ntiles = (N + 15) / 16;
  const int nt0 = blockIdx.x * (BNW / 16) + wn * 4;  // this wave's first 16-column tile

  floatx4 acc[PLANES][WM][4];
#pragma unroll
  for (int p = 0; p < PLANES; ++p)
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[p][i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // ---- A: global -> registers -> LDS.  Piece q of this thread: row (tid / 8) + 32 q, columns (tid % 8) * 8 .. + 8.
  const int a_row = tid / 8, a_kg = tid % 8;
  bf16x8 areg[APT];
  const bf16x8 zero = {};
  auto load_a = [&](int stage) {
    const int k = stage * BK + a_kg * 8;
#pragma unroll
    for (int q = 0; q < APT; ++q) {
      const int m = m_base + a_row + 32 * q;
      areg[q] = (m < M && a_row + 32 * q < BM && k < K)
                    ? *reinterpret_cast<const bf16x8*>(A + static_cast<size_t>(m) * lda + k) : zero;
    }
  };
  auto store_a = [&]() {
#pragma unroll
    for (int q = 0; q < APT; ++q)
      if (a_row + 32 * q < BM) *reinterpret_cast<bf16x8*>(As + (a_row + 32 * q) * PITCH + a_kg * 8) = areg[q];
  };

  // ---- W fragments: tile nt, chunk c is the KiB at ((nt * chunks + c) * 512) elements; this lane's 16 bytes at lane * 8
  bf16x8 wreg[2][PLANES][4];
  auto load_w = [&](int buf, int chunk) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int nt = nt0 + j;
      const bool ok = nt < ntiles && chunk < chunks;
      const size_t off = (static_cast<size_t>(ok ? nt : 0) * chunks + (ok ? chunk : 0)) * 512 + lane * 8;
      wreg[buf][0][j] = ok ? *reinterpret_cast<const bf16x8*>(W + off) : zero;
      if (PLANES == 2) wreg[buf][1][j] = ok ? *reinterpret_cast<const bf16x8*>(W2 + off) : zero;
    }
  };

  const int all_stages = (K + BK - 1) / BK;
  const int s0 = static_cast<int>(static_cast<int64_t>(all_stages) * blockIdx.z / gridDim.z);
  const int nstages = static_cast<int>(static_cast<int64_t>(all_stages) * (blockIdx.z + 1) / gridDim.z);
  load_a(s0);
  load_w(0, s0 * 2);
  store_a();
  __syncthreads();

  for (int s = s0; s < nstages; ++s) {
    if (s + 1 < nstages) load_a(s + 1);
#pragma unroll
    for (int kc = 0; kc < 2; ++kc) {
      const int chunk = s * 2 + kc;
      const int buf = kc;  // chunk parity
      load_w(buf ^ 1, chunk + 1);
      bf16x8 af[WM];
#pragma unroll
      for (int i = 0; i < WM; ++i)
        af[i] = *reinterpret_cast<const bf16x8*>(As + ((wm * WM + i) * 16 + r) * PITCH + kc * 32 + grp * 8);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int p = 0; p < PLANES; ++p)
            acc[p][i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], wreg[buf][p][j], acc[p][i][j], 0, 0, 0);
    }
    __syncthreads();
    if (s + 1 < nstages) {
      store_a();
      __syncthreads();
    }
  }

  // ---- epilogue.  acc[.][i][j][v] is C[m = tile i row 4 * grp + v][n = tile j column r]
  if (gridDim.z > 1) {
#pragma unroll
    for (int p = 0; p < PLANES; ++p)
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = m_base + (wm * WM + i) * 16 + 4 * grp + v;
          if (m >= M) continue;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int n = (nt0 + j) * 16 + r;
            if (n < N) partials[((static_cast<size_t>(blockIdx.z) * PLANES + p) * M + m) * N + n] = acc[p][i][j][v];
          }
        }
    return;
  }
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int m = m_base + (wm * WM + i) * 16 + 4 * grp + v;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = (nt0 + j) * 16 + r;
        if (n >= N) continue;
        float x = acc[0][i][j][v];
        if (EPI == 1) x = gelu_tanh_f(to_float(float_to_bf16(x))) * to_float(float_to_bf16(acc[PLANES - 1][i][j][v]));
        else if (EPI == 2) x = cap * tanhf(x / cap);
        store_f(C, c_dtype, static_cast<size_t>(m) * ldc + n, x);
      }
    }
}

// C = epilogue(sum over z of partials[z][plane]), one thread per output element.
template <int EPI>
__global__ void gemm_reduce_kernel(const float* __restrict__ partials, int KS, void* __restrict__ C, int c_dtype,
                                   int64_t ldc, int M, int N, float cap) {
  constexpr int PLANES = EPI == 1 ? 2 : 1;
  const size_t plane = static_cast<size_t>(M) * N;
  for (size_t e = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; e < plane;
       e += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float x = 0.f, y = 0.f;
    for (int z = 0; z < KS; ++z) {
      x += partials[(static_cast<size_t>(z) * PLANES) * plane + e];
      if (EPI == 1) y += partials[(static_cast<size_t>(z) * PLANES + 1) * plane + e];
    }
    if (EPI == 1) x = gelu_tanh_f(to_float(float_to_bf16(x))) * to_float(float_to_bf16(y));
    else if (EPI == 2) x = cap * tanhf(x / cap);
    store_f(C, c_dtype, (e / N) * ldc + e % N, x);
  }
}

template <int WM, int PLANES, int EPI, int WAVES_N>
static void launch(const bf16* A, int64_t lda, const bf16* W, const bf16* W2, void* C, int c_dtype, int64_t ldc, int M,
                   int N, int K, float cap, int ks, float* partials, hipStream_t stream) {
  constexpr int BM = (4 / WAVES_N) * WM * 16, BNW = WAVES_N * 64;
  const dim3 grid((N + BNW - 1) / BNW, (M + BM - 1) / BM, ks);
  gemm_tiled_kernel<WM, PLANES, EPI, WAVES_N><<<grid, 256, 0, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K,
                                                                        (K + 31) / 32, cap, partials);
  if (ks > 1) {
    const size_t plane = static_cast<size_t>(M) * N;
    const int blocks = static_cast<int>((plane + 255) / 256 > 4096 ? 4096 : (plane + 255) / 256);
    gemm_reduce_kernel<EPI><<<blocks, 256, 0, stream>>>(partials, ks, C, c_dtype, ldc, M, N, cap);
  }
}

}  // namespace tiled

bool gemm_tiled_takes(int M, int N, int K, int64_t lda, const void* A, const void* W, const void* W2, int packed) {
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  return packed && M >= 1 && K % 8 == 0 && lda % 8 == 0 && aligned(A) && aligned(W) && (W2 == nullptr || aligned(W2));
}

// ksplit > 0 fixes the number of cuts of K.
int gemm_tiled(const void* A, int64_t lda, const void* W, const void* W2, void* C, int c_dtype, int64_t ldc, int M,
               int N, int K, int epi, float cap, int ksplit, void* workspace, size_t workspace_bytes,
               hipStream_t stream) {
  const bf16* a = static_cast<const bf16*>(A);
  const bf16* w = static_cast<const bf16*>(W);
  const bf16* w2 = static_cast<const bf16*>(W2);
  float* ws = static_cast<float*>(workspace);
  const int planes = epi == 1 ? 2 : 1;
  const int stages = (K + tiled::BK - 1) / tiled::BK;
  if (M <= 64) {
    // few rows: the product is bound by streaming W, so it needs a workgroup or two per CU even when N is small:
    // waves side by side along N (64 rows x 256 columns per workgroup), K cut over workgroups
    const int tiles = (N + 255) / 256;
    int ks = ksplit > 0 ? ksplit : (512 + tiles - 1) / tiles;
    if (ks > stages / 2) ks = stages / 2;
    if (ks < 1) ks = 1;
    while (ks > 1 && (ws == nullptr || static_cast<size_t>(ks) * planes * M * N * sizeof(float) > workspace_bytes)) --ks;
    if (epi == 1) tiled::launch<4, 2, 1, 4>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
    else if (epi == 2) tiled::launch<4, 1, 2, 4>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
    else tiled::launch<4, 1, 0, 4>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
    return check_launch("gemm_tiled");
  }
  // tall workgroup tiles (256 rows) when there are rows and columns enough to fill the GPU with them
  const bool tall = M > 128 && static_cast<int64_t>((M + 255) / 256) * ((N + 127) / 128) >= 200;
  int ks = ksplit > 0 ? ksplit : 1;
  if (ks > stages) ks = stages;
  while (ks > 1 && (ws == nullptr || static_cast<size_t>(ks) * planes * M * N * sizeof(float) > workspace_bytes)) --ks;
  if (epi == 1) {
    tiled::launch<4, 2, 1, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
  } else if (epi == 2) {
    if (tall) tiled::launch<8, 1, 2, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
    else tiled::launch<4, 1, 2, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
  } else {
    if (tall) tiled::launch<8, 1, 0, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
    else tiled::launch<4, 1, 0, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, ks, ws, stream);
  }
  return check_launch("gemm_tiled");
}

}  // namespace sa
