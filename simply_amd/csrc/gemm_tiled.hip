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
constexpr int BN = 128;         // output columns per workgroup

__device__ inline float gelu_tanh_f(float x) {
  const float k = 0.7978845608028654f;
  return 0.5f * x * (1.f + tanhf(k * (x + 0.044715f * x * x * x)));
}

template <int WM, int PLANES, int EPI>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16* __restrict__ A, int64_t lda,
                                                         const bf16* __restrict__ W, const bf16* __restrict__ W2,
                                                         void* __restrict__ C, int c_dtype, int64_t ldc, int M, int N,
                                                         int K, int chunks, float cap) {
  constexpr int BM = 2 * WM * 16;
  constexpr int APT = BM / 32;  // 16-byte pieces of a slab per thread
  __shared__ __attribute__((aligned(16))) bf16 As[BM * PITCH];

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / 2, wn = wave % 2;
  const int r = lane % 16, grp = lane / 16;
  const int m_base = blockIdx.y * BM;
  const int ntiles = (N + 15) / 16;
  const int nt0 = blockIdx.x * (BN / 16) + wn * 4;  // this wave's first 16-column tile

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
      areg[q] = (m < M && k < K) ? *reinterpret_cast<const bf16x8*>(A + static_cast<size_t>(m) * lda + k) : zero;
    }
  };
  auto store_a = [&]() {
#pragma unroll
    for (int q = 0; q < APT; ++q)
      *reinterpret_cast<bf16x8*>(As + (a_row + 32 * q) * PITCH + a_kg * 8) = areg[q];
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

  const int nstages = (K + BK - 1) / BK;
  load_a(0);
  load_w(0, 0);
  store_a();
  __syncthreads();

  for (int s = 0; s < nstages; ++s) {
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

template <int WM, int PLANES, int EPI>
static void launch(const bf16* A, int64_t lda, const bf16* W, const bf16* W2, void* C, int c_dtype, int64_t ldc, int M,
                   int N, int K, float cap, hipStream_t stream) {
  constexpr int BM = 2 * WM * 16;
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  gemm_tiled_kernel<WM, PLANES, EPI><<<grid, 256, 0, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K, (K + 31) / 32,
                                                               cap);
}

}  // namespace tiled

bool gemm_tiled_takes(int M, int N, int K, int64_t lda, const void* A, const void* W, const void* W2, int packed) {
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  return packed && M >= 1 && K % 8 == 0 && lda % 8 == 0 && aligned(A) && aligned(W) && (W2 == nullptr || aligned(W2));
}

int gemm_tiled(const void* A, int64_t lda, const void* W, const void* W2, void* C, int c_dtype, int64_t ldc, int M,
               int N, int K, int epi, float cap, hipStream_t stream) {
  const bf16* a = static_cast<const bf16*>(A);
  const bf16* w = static_cast<const bf16*>(W);
  const bf16* w2 = static_cast<const bf16*>(W2);
  // tall workgroup tiles (256 rows) when there are rows and columns enough to fill the GPU with them
  const bool tall = M > 128 && static_cast<int64_t>((M + 255) / 256) * ((N + 127) / 128) >= 200;
  if (epi == 1) {
    tiled::launch<4, 2, 1>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, stream);
  } else if (epi == 2) {
    if (tall) tiled::launch<8, 1, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, stream);
    else tiled::launch<4, 1, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, stream);
  } else {
    if (tall) tiled::launch<8, 1, 0>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, stream);
    else tiled::launch<4, 1, 0>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, cap, stream);
  }
  return check_launch("gemm_tiled");
}

}  // namespace sa
