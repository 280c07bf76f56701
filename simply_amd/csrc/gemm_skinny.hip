// C[M, N] = epilogue(A[M, K] . W[N, K]^T) in bfloat16 for few rows (M <= 64): the decode step's
// matrix products, which are bound by reading W once from HBM.
//
// Work is cut into (16 weight rows) x (a range of K) units, one per wavefront.  A wave streams its
// 16 rows of W straight from global memory into MFMA operand registers (16-byte loads, each row's
// four lanes reading 64 contiguous bytes), takes the matching activations from the cache hierarchy
// (they are small and shared by all waves), and accumulates with v_mfma_f32_16x16x32_bf16: the
// weight rows are the MFMA's A operand, up to four blocks of 16 activation rows its B operands.
// W may be row-major [N, K] or tiled (pack_tiles in the Python package): [N / 16][K / 32][64 lanes][8], each
// 1 KiB block being one MFMA operand of 16 rows x 32 columns in register order, so that a wave's load is one
// contiguous KiB (row-major rows give 64-byte pieces, which reach about half the bandwidth).
// The 4 to 16 waves of a workgroup take consecutive K ranges of the same rows and add their results
// through LDS in a fixed order.  When N is small a workgroup owns only 8 or 4 rows (the other
// operand rows are zero), so that there are enough workgroups for 256 CUs without cutting K over
// workgroups: that would need a device-wide fence, which on this GPU writes back the whole L2.
#include "api.h"
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

__device__ inline bf16x8 load_frag(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }

// kUnroll: chunks of 32 columns of K whose loads a wave issues together (one register set).  4 everywhere: sets of 8
// were slower where they could matter (the 2B down projection, 36 chunks a wave: 18.8 us against 15.7).
constexpr int kMaxWaves = 16;

// blockDim.x = 64 * NW (NW waves share the K range); a workgroup owns `tile_rows` (16, 8 or 4) rows of W.
// G (1, 2 or 4; more than 1 only with MB == 1, tiled weights and up to 16 / G rows): a load of activations brings
// G consecutive chunks of K at once, rows 0 .. 16 / G - 1 of chunk g in the operand's columns g * (16 / G) ..: with
// few rows the 16 columns of the operand would otherwise hold copies, and the loads of the activations, which come
// from L2 and are as many as those of the weights, cost a quarter of the kernel (12 against 9 us at the 2B down
// projection without them).  The product of chunk g is right in its own columns only and has an accumulator of its
// own; the G accumulators are added up, column group by column group, after the loop.
template <int MB, int EPI, bool PACKED, int kUnroll, int G>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(const bf16* __restrict__ A, int64_t lda,
                                                           const bf16* __restrict__ W, const bf16* __restrict__ W2,
                                                           void* __restrict__ C, int c_dtype, int64_t ldc, int M, int N,
                                                           int K, int chunks, int tile_rows, float cap, int act) {
  constexpr int NP = EPI == 1 ? 2 : 1;  // planes: gate and up for the gated epilogue
  extern __shared__ float red[];        // [NW][NP][MB][16 * 17]
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // uniform over the wave: kept in a scalar register
  const int NW = blockDim.x / kWave;
  const int r = lane % 16, kq = lane / 16;
  const int n0 = blockIdx.x * tile_rows;
  const int c0 = static_cast<int>(static_cast<int64_t>(chunks) * wave / NW);
  const int c1 = static_cast<int>(static_cast<int64_t>(chunks) * (wave + 1) / NW);

  static_assert(G == 1 || (MB == 1 && PACKED && kUnroll % G == 0), "chunks share a load only for up to 16 rows");
  floatx4 acc[NP][MB * G];  // [p][mb], or [p][g]
#pragma unroll
  for (int p = 0; p < NP; ++p)
#pragma unroll
    for (int mb = 0; mb < MB * G; ++mb) acc[p][mb] = floatx4{0.f, 0.f, 0.f, 0.f};

  const bool row_ok = r < tile_rows && n0 + r < N;
  // row-major W: this lane's row, 8 elements at k.  Tiled W (see pack_tiles): tile (n0 / 16), chunk c is one
  // contiguous 1 KiB block of which this lane owns 16 bytes, padded with zeros beyond N and K.
  // With the gated epilogue a tiled W holds the two matrices' tiles in turn: tile 2 i the gate, 2 i + 1 the factor.
  const size_t tile_elems = static_cast<size_t>(chunks) * 512;
  const size_t tile = (EPI == 1 ? 2 : 1) * static_cast<size_t>(n0 / 16);
  const bf16* wrow = PACKED ? W + tile * tile_elems + lane * 8 : W + static_cast<size_t>(row_ok ? n0 + r : 0) * K;
  const bf16* w2row = EPI != 1 ? nullptr
                      : PACKED ? wrow + tile_elems
                               : W2 + static_cast<size_t>(row_ok ? n0 + r : 0) * K;
  const bf16x8 zero = {};

  // Two register sets of kUnroll chunks each: while one set is multiplied, the loads of the other are in flight.
  bf16x8 a[2][kUnroll], a2[2][kUnroll], b[2][kUnroll][MB];
  auto load_set = [&](int set, int c) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int k = (c + u) * 32 + kq * 8;
      const bool ok = c + u < c1 && k < K;
      if (PACKED) a[set][u] = c + u < c1 ? load_frag(wrow + static_cast<size_t>(c + u) * 512) : zero;
      else a[set][u] = (ok && row_ok) ? load_frag(wrow + k) : zero;
      if (EPI == 1) {
        if (PACKED) a2[set][u] = c + u < c1 ? load_frag(w2row + static_cast<size_t>(c + u) * 512) : zero;
        else a2[set][u] = (ok && row_ok) ? load_frag(w2row + k) : zero;
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = mb * 16 + r;
        b[set][u][mb] = (ok && m < M) ? load_frag(A + static_cast<size_t>(m) * lda + k) : zero;
      }
    }
  };
  auto mul_set = [&](int set) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        acc[0][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[set][u], b[set][u][mb], acc[0][mb], 0, 0, 0);
        if (EPI == 1)
          acc[1][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[set][u], b[set][u][mb], acc[1][mb], 0, 0, 0);
      }
  };
  if (PACKED && K % 32 == 0) {
    // Tiled weights and whole chunks (every real model's sizes): the loop's loads are unconditional, so that it is
    // straight-line code and the compiler counts the loads in flight; with a branch around a load it waits for
    // all of them before the first product, and the two register sets never overlap.  Activation rows beyond M are
    // read from row M - 1: their products land in output rows that are not stored.
    const bf16* arow[MB];
    constexpr int kCols = 16 / G;  // columns of the operand per chunk: lane column r holds row r % kCols of chunk r / kCols
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = mb * 16 + r % kCols;
      arow[mb] = A + static_cast<size_t>(m < M ? m : M - 1) * lda + (r / kCols) * 32 + kq * 8;
    }
    auto load_full = [&](int set, int c) {   // chunks c .. c + kUnroll - 1, all within the wave's range
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        a[set][u] = load_frag(wrow + static_cast<size_t>(c + u) * 512);
        if (EPI == 1) a2[set][u] = load_frag(w2row + static_cast<size_t>(c + u) * 512);
        if (u % G == 0) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) b[set][u / G][mb] = load_frag(arow[mb] + (c + u) * 32);
        }
      }
    };
    auto mul_full = [&](int set) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const int to = G == 1 ? mb : u % G;
          acc[0][to] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[set][u], b[set][u / G][mb], acc[0][to], 0, 0, 0);
          if (EPI == 1)
            acc[1][to] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[set][u], b[set][u / G][mb], acc[1][to], 0, 0, 0);
        }
    };
    const int sets = (c1 - c0) / kUnroll;   // full sets; what is left goes through the loads with tests below
    int s = 0;
    if (sets > 0) {
      load_full(0, c0);
      for (; s + 2 < sets; s += 2) {   // set 0 holds full set s
        // (the scheduling barriers keep the compiler from moving the loads of a set behind the products of the
        // other: it would then wait for them where it has put them, with nothing in flight across iterations)
        load_full(1, c0 + (s + 1) * kUnroll);
        __builtin_amdgcn_sched_barrier(0);
        mul_full(0);
        __builtin_amdgcn_sched_barrier(0);
        load_full(0, c0 + (s + 2) * kUnroll);
        __builtin_amdgcn_sched_barrier(0);
        mul_full(1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (sets - s == 2) {
        load_full(1, c0 + (s + 1) * kUnroll);
        mul_full(0);
        mul_full(1);
      } else {
        mul_full(0);
      }
    }
    if (c0 + sets * kUnroll < c1) {  // (row m in column m: into the first accumulator, whose columns these are)
      load_set(0, c0 + sets * kUnroll);
      mul_set(0);
    }
    if (G > 1) {  // column r of the sum: accumulator g's column g * kCols + r, that is its row of 16 lanes rotated
                  // (a rotation on the vector unit, DPP row_ror, not a shuffle through LDS)
#pragma unroll
      for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          if constexpr (G == 2) {
            acc[p][0][v] += lane_exchange<0x120 + 8>(acc[p][1][v]);
          } else if constexpr (G == 4) {
            acc[p][0][v] += lane_exchange<0x120 + 12>(acc[p][1][v]);
            acc[p][0][v] += lane_exchange<0x120 + 8>(acc[p][2][v]);
            acc[p][0][v] += lane_exchange<0x120 + 4>(acc[p][3][v]);
          }
        }
    }
  } else {
    load_set(0, c0);
    for (int c = c0; c < c1; c += 2 * kUnroll) {
      load_set(1, c + kUnroll);
      mul_set(0);
      load_set(0, c + 2 * kUnroll);
      mul_set(1);
    }
  }

  // lane holds D[n = 4 * (lane / 16) + v][m = lane % 16]; the waves' tiles are added up through LDS, in wave order
  auto red_at = [&](int w, int p, int mb) { return red + ((static_cast<size_t>(w) * NP + p) * MB + mb) * (16 * 17); };
#pragma unroll
  for (int p = 0; p < NP; ++p)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int v = 0; v < 4; ++v) red_at(wave, p, mb)[(4 * kq + v) * 17 + r] = acc[p][mb][v];
  __syncthreads();
  for (int e = tid; e < 256; e += blockDim.x) {
  const int ml = e / 16, nl = e % 16;  // an output element within each 16 x 16 block
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + ml, n = n0 + nl;
    if (m >= M || nl >= tile_rows || n >= N) continue;
    float sum[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      float t = 0.f;
      for (int w = 0; w < NW; ++w) t += red_at(w, p, mb)[nl * 17 + ml];
      sum[p] = t;
    }
    float v = sum[0];
    if (EPI == 1) {
      // both products are rounded to bfloat16 first, as separate matrix products would be
      v = gated_activation(act, to_float(float_to_bf16(v))) * to_float(float_to_bf16(sum[NP - 1]));
    } else if (EPI == 2) {
      v = cap * tanhf(v / cap);
    }
    store_f(C, c_dtype, static_cast<size_t>(m) * ldc + n, v);
  }
  }
}

// Rows of W per workgroup and waves per workgroup; no wave gets less than two 32-wide chunks of K; the LDS for the
// waves' tiles stays under 64 KiB.  Nothing is cut over workgroups: on this GPU a device-wide fence writes the
// whole L2 back.
static void choose_shape(int N, int chunks, int planes, int MB, int* tile_rows, int* waves) {
  // measured on MI355X at M = 8: tiles of 16 rows always win (narrower tiles leave load lanes idle); 8 waves
  // per workgroup while there are few tiles, 4 when there are many
  const int rows = 16;
  const int tiles = (N + rows - 1) / rows;
  int nw = tiles < 1024 ? 8 : 4;
  if (nw > chunks / 2) nw = chunks / 2;
  while (nw > 1 && static_cast<size_t>(nw) * planes * MB * 16 * 17 * sizeof(float) > 60 * 1024) --nw;
  if (nw > kMaxWaves) nw = kMaxWaves;
  if (nw < 1) nw = 1;
  *tile_rows = rows;
  *waves = nw;
}

template <int MB, bool PACKED, int U, int G = 1>
static void launch_skinny(const bf16* A, int64_t lda, const bf16* W, const bf16* W2, void* C, int c_dtype, int64_t ldc,
                          int M, int N, int K, int epi, int act, float cap, int tile_rows, int waves,
                          hipStream_t stream) {
  const int chunks = (K + 31) / 32;
  const dim3 grid((N + tile_rows - 1) / tile_rows);
  const int threads = waves * kWave;
  const size_t lds = static_cast<size_t>(waves) * (epi == 1 ? 2 : 1) * MB * 16 * 17 * sizeof(float);
  if (epi == 0)
    gemm_skinny_kernel<MB, 0, PACKED, U, G><<<grid, threads, lds, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K, chunks,
                                                                      tile_rows, cap, act);
  else if (epi == 1)
    gemm_skinny_kernel<MB, 1, PACKED, U, G><<<grid, threads, lds, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K, chunks,
                                                                      tile_rows, cap, act);
  else
    gemm_skinny_kernel<MB, 2, PACKED, U, G><<<grid, threads, lds, stream>>>(A, lda, W, W2, C, c_dtype, ldc, M, N, K, chunks,
                                                                      tile_rows, cap, act);
}

bool gemm_skinny_takes(int M, int N, int K, int64_t lda, const void* A, const void* W, const void* W2) {
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  // K % 8: a lane's 8 activations lie within its row, and row-major weight rows start at 16-byte boundaries
  return M >= 1 && M <= 64 && K % 8 == 0 && lda % 8 == 0 && aligned(A) && aligned(W) && (W2 == nullptr || aligned(W2));
}

// The time that this kernel is expected to take, in microseconds (the figure by which the library chooses between its
// product kernels), or a negative number for sizes that it would serve badly by construction (more than 16 rows of a
// gated product, more than 32 of any).  A workgroup streams 16 rows of W (32 of a paired weight) over all of K and
// reads the rows of activations from L2; a CU's workgroups share its memory path.  The constants are fitted to a
// sweep over 1 to 64 rows against fifteen weight sizes from 2 MB to 1.2 GB streamed from HBM (among them the q/k/v,
// output, down and gated products of the Gemma 2 2B, 9B and 27B sizes and four sizes of no model): the prediction is
// within 0.83 to 1.27 of the measured time.
double gemm_skinny_predict_us(int M, int N, int K, int epi) {
  if (M > (epi == 1 ? 16 : 32)) return -1.0;
  const double wgs = (N + 15) / 16;
  const double wg_bytes = (epi == 1 ? 32.0 : 16.0) * K * 2;
  const double hbm_us = wgs * wg_bytes / 6.0e6;                            // every weight once, at 6 TB/s
  const double act_us = wgs * M * K * 2 / (M > 8 ? 15.0e6 : 30.0e6);       // the activations, per workgroup, from L2
  // a CU streams 33 GB/s through one of these workgroups after another; rows beyond 8 cost it activation loads of
  // their own (up to 8 rows ride along in the weights' load slots)
  const double rows = M <= 8 ? 1.0 : (M <= 16 ? 1.0 + 0.085 * (M - 8) : 1.68 + 0.045 * (M - 16));
  const double cu_us = ceil(wgs / 256.0) * wg_bytes / 33.0e3 * rows;
  return 2.5 + fmax(hbm_us + act_us, cu_us);
}

// shape > 0 fixes the cut: tile_rows * 100 + waves (for instance 816: 8 rows, 16 waves)
int gemm_skinny(const void* A, int64_t lda, const void* W, const void* W2, void* C, int c_dtype, int64_t ldc, int M,
                int N, int K, int epi, int act, float cap, int packed, int shape, hipStream_t stream) {
  const int chunks = (K + 31) / 32, planes = epi == 1 ? 2 : 1;
  const int MB = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  int tile_rows, waves;
  choose_shape(N, chunks, planes, MB, &tile_rows, &waves);
  if (shape > 0) {
    tile_rows = shape / 100;
    waves = shape % 100;
    if ((tile_rows != 4 && tile_rows != 8 && tile_rows != 16) || (packed && tile_rows != 16) || waves < 1 || waves > kMaxWaves ||
        static_cast<size_t>(waves) * planes * MB * 16 * 17 * sizeof(float) > 64 * 1024) {
      set_error("gemm: bad few-rows shape %d (rows 4, 8 or 16, times 100, plus 1..16 waves)", shape);
      return 1;
    }
  }
  const bf16* a = static_cast<const bf16*>(A);
  const bf16* w = static_cast<const bf16*>(W);
  const bf16* w2 = static_cast<const bf16*>(W2);
#define SA_SKINNY(MBV)                                                                                              \
  do {                                                                                                              \
    if (packed)                                                                                                     \
      launch_skinny<MBV, true, 4>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, epi, act, cap, tile_rows, waves, stream); \
    else                                                                                                            \
      launch_skinny<MBV, false, 4>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, epi, act, cap, tile_rows, waves, stream); \
  } while (0)
  // up to 8 rows against tiled weights: two or four chunks of K to a load of activations
  if (packed && K % 32 == 0 && tile_rows == 16 && M <= 4)
    launch_skinny<1, true, 4, 4>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, epi, act, cap, tile_rows, waves, stream);
  else if (packed && K % 32 == 0 && tile_rows == 16 && M <= 8)
    launch_skinny<1, true, 4, 2>(a, lda, w, w2, C, c_dtype, ldc, M, N, K, epi, act, cap, tile_rows, waves, stream);
  else if (MB == 1) SA_SKINNY(1);
  else if (MB == 2) SA_SKINNY(2);
  else SA_SKINNY(4);
#undef SA_SKINNY
  return check_launch("gemm_skinny");
}

}  // namespace sa
