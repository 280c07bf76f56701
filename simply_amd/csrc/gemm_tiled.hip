// C[M, N] = epilogue(A[M, K] . W[N, K]^T) in bfloat16 for many rows (portions of prompts): bound by
// the MFMA units.  W is in the tiled layout (16 x 32 blocks in MFMA operand order, see
// simply_amd/kernels/packing.py), A is row-major.
//
// A workgroup of four waves (2 x 2) owns 128 x 128 outputs; a wave owns 64 x 64 of them as 4 x 4 tiles of
// v_mfma_f32_16x16x32_bf16.  Per step of 32 along K a wave needs 4 fragments of A and 4 of W:
//   * A goes through LDS: the workgroup copies 128 x 64 slabs with 16-byte loads (eight lanes per row: whole
//     128-byte lines) into two LDS buffers, two slabs ahead of the multiplication (one in registers, one in
//     LDS), with one barrier per slab; rows are padded to 144 bytes so that the fragment reads
//     (ds_read_b128) hit all 64 banks once.
//   * W fragments are loaded straight from global memory into operand registers (a fragment is one
//     contiguous KiB of the tiled layout), a slab ahead, and never touch LDS.
//
// Epilogues: none; gated (C = gelu_tanh(A.Wg^T) * (A.Wu^T), both rounded to bfloat16 first, from one weight
// whose tiles alternate between Wg and Wu); soft-cap (C = cap * tanh(. / cap), float32 out).
#include <cmath>
#include "api.h"
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

namespace tiled {

constexpr int BK = 64;          // columns of A per LDS slab
constexpr int PITCH = BK + 8;   // elements per LDS row: 144 bytes

// WAVES_N: 2 = waves as 2 x 2 (BM = 2 * WM * 16 rows, 128 columns of W tiles); 4 = waves as 1 x 4 (BM = WM * 16 rows,
// 256 columns: for few rows, every W fragment is loaded by one wave only).  gridDim.z > 1 cuts K over workgroups:
// each writes its float32 partial tile to `partials` [z][M][NW] and gemm_reduce_kernel adds them up.
//
// The gated epilogue (EPI 1) reads one weight whose 16-row tiles alternate between the two matrices (tile 2 i:
// rows 16 i .. of the gate, tile 2 i + 1: the same rows of the other factor; pack_gate_up in the Python package):
// a wave's four tiles are two output tiles, and gate and factor meet in the same lane's registers.  NW is the
// number of weight rows (2 N for the gated epilogue, else N).
// TAIL: K is no multiple of the slab, so the loads carry tests against K.
template <int WM, int EPI, int WAVES_N, bool TAIL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void gemm_tiled_kernel(const bf16* __restrict__ A, int64_t lda, const bf16* __restrict__ W, void* __restrict__ C,
                       int c_dtype, int64_t ldc, int M, int N, int K, int chunks, float cap, int act,
                       float* __restrict__ partials) {
  constexpr int WAVES_M = 4 / WAVES_N;
  constexpr int BM = WAVES_M * WM * 16;
  constexpr int BNW = WAVES_N * 64;  // weight rows per workgroup
  static_assert(BM % 32 == 0, "a slab is copied in passes of 32 rows");
  constexpr int APT = BM / 32;  // 16-byte pieces of a slab per thread
  __shared__ __attribute__((aligned(16))) bf16 As[2][BM * PITCH];

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int r = lane % 16, grp = lane / 16;
  // Which tile this workgroup takes.  Workgroups are handed to the eight XCDs in turn, each with an L2 of its own:
  // the numbering is turned round so that an XCD gets a contiguous share of the tiles, and within it tiles go in
  // columns eight wide, rows first: the 32 workgroups that an XCD runs at a time are a 4 x 8 patch that shares its
  // rows of A and of W through that L2.
  int bx = blockIdx.x, by = blockIdx.y;
  {
    const int nx = gridDim.x, ny = gridDim.y, total = nx * ny;
    int l = bx + nx * by;
    if (total % 8 == 0) l = (l % 8) * (total / 8) + l / 8;
    constexpr int GX = 8;
    const int full = nx / GX;
    if (l < full * GX * ny) {
      const int col = l / (GX * ny), rem = l % (GX * ny);
      by = rem / GX;
      bx = col * GX + rem % GX;
    } else {
      const int rem = l - full * GX * ny, width = nx % GX;
      by = rem / width;
      bx = full * GX + rem % width;
    }
  }
  const int m_base = by * BM;
  const int NW = EPI == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  const int ntiles = (NW + 15) / 16;
  const int nt0 = bx * (BNW / 16) + wn * 4;  // this wave's first 16-row tile of W

  floatx4 acc[WM][4];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // ---- A: global -> registers -> LDS.  Piece q of this thread: row (tid / 8) + 32 q, columns (tid % 8) * 8 .. + 8.
  // Rows beyond M read row M - 1 instead (their products are never stored), so that the loop carries no row test;
  // what depends on the thread alone (row offsets) is computed once, the slab's offset is the same for all.
  const int a_row = tid / 8, a_kg = tid % 8;
  bf16x8 areg[APT];
  const bf16x8 zero = {};
  uint32_t a_off[APT];  // elements; the host checks that M * lda fits
#pragma unroll
  for (int q = 0; q < APT; ++q) {
    const int m = m_base + a_row + 32 * q;
    a_off[q] = static_cast<uint32_t>(m < M ? m : M - 1) * static_cast<uint32_t>(lda) + a_kg * 8;
  }
  auto load_a = [&](int stage) {
    const bf16* slab = A + static_cast<size_t>(stage) * BK;  // the same for the whole workgroup
    const bool in_k = !TAIL || stage * BK + a_kg * 8 < K;
#pragma unroll
    for (int q = 0; q < APT; ++q) areg[q] = in_k ? *reinterpret_cast<const bf16x8*>(slab + a_off[q]) : zero;
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int q = 0; q < APT; ++q)
      *reinterpret_cast<bf16x8*>(As[buf] + (a_row + 32 * q) * PITCH + a_kg * 8) = areg[q];
  };

  // ---- W fragments of a whole slab (two steps of 32): tile nt, chunk c is the KiB at ((nt * chunks + c) * 512)
  // elements, this lane's 16 bytes at lane * 8.  They are requested one slab ahead.  Tiles beyond the last read the
  // last tile instead (their products are never stored).
  bf16x8 wreg[2][2][4];
  const bf16* wtile[4];  // the same for the whole wave
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int nt = __builtin_amdgcn_readfirstlane(nt0 + j < ntiles ? nt0 + j : ntiles - 1);
    wtile[j] = W + static_cast<size_t>(nt) * chunks * 512;
  }
  auto load_w = [&](int buf, int stage) {
#pragma unroll
    for (int kc = 0; kc < 2; ++kc) {
      const int chunk = stage * 2 + kc;
      const bool in_k = !TAIL || chunk < chunks;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        wreg[buf][kc][j] =
            in_k ? *reinterpret_cast<const bf16x8*>(wtile[j] + static_cast<size_t>(chunk) * 512 + lane * 8) : zero;
    }
  };
  auto multiply = [&](int wbuf, int abuf) {
#pragma unroll
    for (int kc = 0; kc < 2; ++kc) {
      bf16x8 af[WM];
#pragma unroll
      for (int i = 0; i < WM; ++i)
        af[i] = *reinterpret_cast<const bf16x8*>(As[abuf] + ((wm * WM + i) * 16 + r) * PITCH + kc * 32 + grp * 8);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], wreg[wbuf][kc][j], acc[i][j], 0, 0, 0);
    }
  };

  const int all_stages = (K + BK - 1) / BK;
  const int s0 = static_cast<int>(static_cast<int64_t>(all_stages) * blockIdx.z / gridDim.z);
  const int s1 = static_cast<int>(static_cast<int64_t>(all_stages) * (blockIdx.z + 1) / gridDim.z);
  // slabs s0 and s0 + 1 into the two LDS buffers, W of slab s0 into registers
  load_a(s0);
  load_w(0, s0);
  store_a(0);
  if (s0 + 1 < s1) {
    load_a(s0 + 1);
    store_a(1);
  }
  __syncthreads();
  // two slabs per turn, so that the register and LDS buffers have fixed names
  for (int s = s0; s < s1; s += 2) {
    // slab s: LDS buffer 0, W registers 0
    if (s + 2 < s1) load_a(s + 2);
    if (s + 1 < s1) load_w(1, s + 1);
    multiply(0, 0);
    __syncthreads();                       // all waves are done with LDS buffer 0
    if (s + 2 < s1) store_a(0);
    if (s + 1 >= s1) break;
    // slab s + 1: LDS buffer 1, W registers 1
    if (s + 3 < s1) load_a(s + 3);
    if (s + 2 < s1) load_w(0, s + 2);
    multiply(1, 1);
    __syncthreads();                       // all waves are done with LDS buffer 1; buffer 0 is complete
    if (s + 3 < s1) store_a(1);
  }

  // ---- epilogue.  acc[i][j][v] is the product at row (tile i, 4 * grp + v) and weight row (tile j, r)
  constexpr int OUT_TILES = EPI == 1 ? 2 : 4;  // output tiles of 16 columns per wave
  if (gridDim.z > 1) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = m_base + (wm * WM + i) * 16 + 4 * grp + v;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = (nt0 + j) * 16 + r;
          if (n < NW) partials[(static_cast<size_t>(blockIdx.z) * M + m) * NW + n] = acc[i][j][v];
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
      for (int j = 0; j < OUT_TILES; ++j) {
        const int n = EPI == 1 ? (nt0 / 2 + j) * 16 + r : (nt0 + j) * 16 + r;
        if (n >= N) continue;
        float x;
        if (EPI == 1)
          x = gated_activation(act, to_float(float_to_bf16(acc[i][2 * j][v]))) * to_float(float_to_bf16(acc[i][2 * j + 1][v]));
        else if (EPI == 2) x = cap * tanhf(acc[i][j][v] / cap);
        else x = acc[i][j][v];
        store_f(C, c_dtype, static_cast<size_t>(m) * ldc + n, x);
      }
    }
}

// C = epilogue(sum over z of partials[z]), one thread per output element.  For the gated epilogue the partial
// tiles hold weight rows in the alternating order: output column n has its gate at 32 (n / 16) + n % 16 and its
// factor 16 further.
template <int EPI>
__global__ void gemm_reduce_kernel(const float* __restrict__ partials, int KS, void* __restrict__ C, int c_dtype,
                                   int64_t ldc, int M, int N, int NW, float cap, int act) {
  const size_t total = static_cast<size_t>(M) * N, plane = static_cast<size_t>(M) * NW;
  for (size_t e = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; e < total;
       e += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t m = e / N, n = e % N;
    const size_t col = EPI == 1 ? 32 * (n / 16) + n % 16 : n;
    float x = 0.f, y = 0.f;
    // eight planes at a time: their loads are in flight together, the sums keep the order of the planes
    for (int z0 = 0; z0 < KS; z0 += 8) {
      float px[8], py[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool ok = z0 + j < KS;
        px[j] = ok ? partials[(z0 + j) * plane + m * NW + col] : 0.f;
        py[j] = (EPI == 1 && ok) ? partials[(z0 + j) * plane + m * NW + col + 16] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        x += px[j];
        y += py[j];
      }
    }
    if (EPI == 1) x = gated_activation(act, to_float(float_to_bf16(x))) * to_float(float_to_bf16(y));
    else if (EPI == 2) x = cap * tanhf(x / cap);
    store_f(C, c_dtype, m * ldc + n, x);
  }
}

// The same for four neighbouring columns per thread (N, NW and ldc multiples of 4, C aligned to its four elements):
// 16-byte loads of the partial tiles, one store.  Each column's sum runs over the planes in the same order as above.
template <int EPI>
__global__ __launch_bounds__(256) void gemm_reduce4_kernel(const float* __restrict__ partials, int KS, void* __restrict__ C,
                                                           int c_dtype, int64_t ldc, int M, int N, int NW, float cap,
                                                           int act) {
  const size_t total = static_cast<size_t>(M) * (N / 4), plane = static_cast<size_t>(M) * NW;
  for (size_t e = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; e < total;
       e += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t m = e / (N / 4), n = (e % (N / 4)) * 4;
    const size_t col = EPI == 1 ? 32 * (n / 16) + n % 16 : n;
    float4 x = {0.f, 0.f, 0.f, 0.f}, y = {0.f, 0.f, 0.f, 0.f};
    for (int z0 = 0; z0 < KS; z0 += 8) {
      float4 px[8], py[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool ok = z0 + j < KS;
        const float* at = partials + (z0 + j) * plane + m * NW + col;
        px[j] = ok ? *reinterpret_cast<const float4*>(at) : float4{0.f, 0.f, 0.f, 0.f};
        py[j] = (EPI == 1 && ok) ? *reinterpret_cast<const float4*>(at + 16) : float4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        x.x += px[j].x; x.y += px[j].y; x.z += px[j].z; x.w += px[j].w;
        y.x += py[j].x; y.y += py[j].y; y.z += py[j].z; y.w += py[j].w;
      }
    }
    float r[4] = {x.x, x.y, x.z, x.w};
    const float g[4] = {y.x, y.y, y.z, y.w};
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if (EPI == 1) r[v] = gated_activation(act, to_float(float_to_bf16(r[v]))) * to_float(float_to_bf16(g[v]));
      else if (EPI == 2) r[v] = cap * tanhf(r[v] / cap);
    }
    if (c_dtype == kF32) {
      *reinterpret_cast<float4*>(static_cast<float*>(C) + m * ldc + n) = float4{r[0], r[1], r[2], r[3]};
    } else {
      uint2 packed;
      packed.x = static_cast<uint32_t>(float_to_bf16(r[0]).bits) | (static_cast<uint32_t>(float_to_bf16(r[1]).bits) << 16);
      packed.y = static_cast<uint32_t>(float_to_bf16(r[2]).bits) | (static_cast<uint32_t>(float_to_bf16(r[3]).bits) << 16);
      *reinterpret_cast<uint2*>(static_cast<bf16*>(C) + m * ldc + n) = packed;
    }
  }
}

template <int WM, int EPI, int WAVES_N>
static void launch(const bf16* A, int64_t lda, const bf16* W, void* C, int c_dtype, int64_t ldc, int M, int N, int K,
                   float cap, int act, int ks, float* partials, hipStream_t stream) {
  constexpr int BM = (4 / WAVES_N) * WM * 16, BNW = WAVES_N * 64;
  const int NW = EPI == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  const dim3 grid((NW + BNW - 1) / BNW, (M + BM - 1) / BM, ks);
  if (K % BK == 0)
    gemm_tiled_kernel<WM, EPI, WAVES_N, false><<<grid, 256, 0, stream>>>(A, lda, W, C, c_dtype, ldc, M, N, K, (K + 31) / 32,
                                                                         cap, act, partials);
  else
    gemm_tiled_kernel<WM, EPI, WAVES_N, true><<<grid, 256, 0, stream>>>(A, lda, W, C, c_dtype, ldc, M, N, K, (K + 31) / 32,
                                                                        cap, act, partials);
  if (ks > 1) gemm_sum_partials(partials, ks, C, c_dtype, ldc, M, N, NW, EPI, act, cap, stream);
}

}  // namespace tiled

int gemm_sum_partials(const float* partials, int ks, void* C, int c_dtype, int64_t ldc, int M, int N, int NW, int epi,
                      int act, float cap, hipStream_t stream) {
  const size_t c_bytes = c_dtype == kF32 ? 4 : 2;
  const bool by_four = N % 4 == 0 && NW % 4 == 0 && ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & (4 * c_bytes - 1)) == 0 &&
                       (reinterpret_cast<uintptr_t>(partials) & 15u) == 0;
  const size_t total = by_four ? static_cast<size_t>(M) * (N / 4) : static_cast<size_t>(M) * N;
  const int blocks = static_cast<int>((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
#define SA_SUM(EPI)                                                                                              \
  do {                                                                                                           \
    if (by_four) tiled::gemm_reduce4_kernel<EPI><<<blocks, 256, 0, stream>>>(partials, ks, C, c_dtype, ldc, M, N, NW, cap, act); \
    else tiled::gemm_reduce_kernel<EPI><<<blocks, 256, 0, stream>>>(partials, ks, C, c_dtype, ldc, M, N, NW, cap, act);          \
  } while (0)
  if (epi == 1) SA_SUM(1);
  else if (epi == 2) SA_SUM(2);
  else SA_SUM(0);
#undef SA_SUM
  return check_launch("gemm_sum_partials");
}

// Whether a product of M rows against NW weight rows of length K is better off with 64 rows x 256 weight rows per
// workgroup and K cut over workgroups than with the wide-tile kernel.  Measured at the 2B, 9B and 27B sizes: up to
// 64 rows always; beyond that while M * NW stays below about a million (192 rows of a q/k/v projection, 256 to 384
// of an output projection), and further the longer K is (the down projections: to 384 rows at K = 9216 and 14336,
// to 512 at 36864), where the wide kernel's few tiles would each walk all of K on a fraction of the CUs.
bool gemm_streams_weights(int M, int NW, int K) {
  const double limit = K <= 9216 ? 1.0e6 : 1.0e6 * pow(static_cast<double>(K) / 9216.0, 0.85);
  return M <= 64 || static_cast<double>(M) * NW <= limit;
}

// The time that this kernel is expected to take, in microseconds (see gemm_skinny_predict_us): the weights streamed
// once, or the products at this kernel's rate, whichever takes longer, after a start that includes the sum of the
// cuts of K.  Fitted to the same sweep (within 0.86 to 1.38 of the measured time up to 64 rows).
double gemm_tiled_predict_us(int M, int N, int K, int epi) {
  const double NW = epi == 1 ? 2.0 * ((N + 15) / 16) * 16 : N;
  return 9.0 + 0.08 * (M < 64 ? M : 64) + fmax(2.0 * NW * K / 5.7e6, static_cast<double>(M) * NW * K / (0.6e9 / 2));
}

bool gemm_tiled_takes(int M, int N, int K, int64_t lda, const void* A, const void* W, const void* W2, int packed) {
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  return packed && W2 == nullptr && M >= 1 && K % 8 == 0 && lda % 8 == 0 && aligned(A) && aligned(W) &&
         static_cast<int64_t>(M) * lda < (int64_t{1} << 32);  // row offsets are kept in 32 bits
}

// ksplit > 0 fixes the number of cuts of K.
int gemm_tiled(const void* A, int64_t lda, const void* W, void* C, int c_dtype, int64_t ldc, int M, int N, int K,
               int epi, int act, float cap, int ksplit, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  const bf16* a = static_cast<const bf16*>(A);
  const bf16* w = static_cast<const bf16*>(W);
  float* ws = static_cast<float*>(workspace);
  const int NW = epi == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  const int stages = (K + tiled::BK - 1) / tiled::BK;
  const bool few = gemm_streams_weights(M, NW, K);
  int ks = 1;
  if (ksplit > 0) {
    ks = ksplit;
  } else if (few) {
    // few rows: the product is bound by streaming W, so it needs a workgroup or two per CU even when N is small:
    // waves side by side (64 rows x 256 weight rows per workgroup), K cut over workgroups
    // (measured at 32 and 64 rows at the 2B, 9B and 27B sizes: about a workgroup per CU of at least four slabs
    // each, nearly two per CU where K is long; more cuts cost more in the sum of the partial tiles than they gain)
    const int tiles = (NW + 255) / 256;
    const int target = K >= 8192 ? 440 : 256;
    ks = (target + tiles / 2) / tiles;
    if (ks > stages / 4) ks = stages / 4;
    // ... and no more cuts than keep the partial tiles (written and read again as 32-bit) at half the weights' bytes:
    // at 256 rows of the 2B down projection 9 cuts (38 us) instead of 36 (54 us); at 64 rows nothing changes
    const int by_traffic = static_cast<int>((static_cast<int64_t>(NW) * K * 2) / (2 * static_cast<int64_t>(M) * NW * 4));
    if (ks > by_traffic) ks = by_traffic < 2 ? 2 : by_traffic;
  }
  if (ks > stages) ks = stages;
  if (ks < 1) ks = 1;
  while (ks > 1 && (ws == nullptr || static_cast<size_t>(ks) * M * NW * sizeof(float) > workspace_bytes)) --ks;
#define SA_TILED(WM, WN)                                                                                      \
  do {                                                                                                        \
    if (epi == 1) tiled::launch<WM, 1, WN>(a, lda, w, C, c_dtype, ldc, M, N, K, cap, act, ks, ws, stream);      \
    else if (epi == 2) tiled::launch<WM, 2, WN>(a, lda, w, C, c_dtype, ldc, M, N, K, cap, act, ks, ws, stream); \
    else tiled::launch<WM, 0, WN>(a, lda, w, C, c_dtype, ldc, M, N, K, cap, act, ks, ws, stream);               \
  } while (0)
  if (few) SA_TILED(4, 4);
  else SA_TILED(4, 2);
#undef SA_TILED
  return check_launch("gemm_tiled");
}

}  // namespace sa
