// C[M, N] = epilogue(A[M, K] . W[N, K]^T) in bfloat16 for very many rows (whole prompts), on tiles wide enough
// that the vector memory path is no longer the bound: the 128 x 128 tiles of the tiled kernel pull 96 KiB per
// slab of 64 columns through a CU's 64 bytes a clock, which caps it at about a third of the MFMA rate.
//
// A workgroup of eight waves (one per CU) owns 256 x 192, 256 x 128, 128 x 256 or 192 x 128 outputs (or one of four
// waves, two per CU, 128 x 192) and takes both operands through LDS, in slabs of 64 columns of K that go round two
// or three buffers, with loads that go from global memory straight into LDS (no registers in between).
//   * Layout in LDS: W as KiB blocks in MFMA operand order (16 rows x 32 columns, lane l holds row l % 16,
//     columns 8 (l / 16) ..), which is how it lies in global memory, so a block is a copy.  A as rows of 128 bytes
//     (eight lanes load a row: whole lines) whose eight 16-byte pieces are permuted by the row's number, so that
//     the 16 rows of a fragment read fall into different banks.  All fragment reads are ds_read_b128 without bank
//     conflicts (measured).
//   * Schedule of a wave: the fragments of the two halves of a slab have registers of their own; the products of
//     the second half are held back until after the next barrier, where they cover the fragment reads of the next
//     slab's first half, and the reads of the second half are covered by the products of the first: between two
//     barriers the MFMA unit always has products to do.  On the larger tiles the reads are issued one by one
//     between those products (a wave issues in order: many reads in a row keep its products back).  The loads of
//     the slab one or two ahead are spread over the products, one after every few: issued together after the
//     barrier, the waves queue up at the memory pipeline (16 cycles a load) while the MFMA unit idles; with two
//     buffers they all go out in the first half of a slab, so that the second half covers the last one's way.
//   * The products are taken transposed (W fragment as the first operand), so that a lane holds four neighbouring
//     columns of one row of C and stores them as one 8-byte piece.
//
// Epilogues: none; gated (C = act(A.Wg^T) * (A.Wu^T), both rounded to bfloat16 first, from one weight whose
// 16-row tiles alternate between Wg and Wu).  K must be a multiple of 64, N and ldc of 4.
//
// K may be cut over gridDim.z workgroups (a few hundred rows against a long K and few weight rows: too few tiles for
// 256 CUs otherwise): each writes its 32-bit partial tile to `partials` [z][M][N], and the tiled kernel's sum kernel
// adds them up.
#include "api.h"
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

namespace wide {

constexpr int BK = 64;
constexpr int kCUs = 256;  // compute units of an MI355X

// s_waitcnt for "at most n vector-memory loads outstanding" and nothing else (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4, lgkmcnt 11:8)
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// The workgroup barrier alone; the empty statements keep the compiler from moving memory accesses across it.
__device__ inline void bare_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
}

// 16 bytes per lane from global memory (base + offset bytes, base the same for the whole wave) into LDS at byte
// address lds + 16 * lane (the same for the whole wave).  Written as an instruction: the compiler counts a load
// into LDS that it knows of as a pending LDS access for as long as the load is under way, and then makes every
// wait for a fragment read a wait for all of them.  It does not know of these loads: the kernel waits for them
// itself (vmcnt) before the barrier that precedes the first read of what they bring.
__device__ __forceinline__ void load_to_lds(const bf16* base, uint32_t offset, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(offset), "s"(base), "s"(lds)
               : "memory");
}

// WM x WN: 16 x 16 tiles of a wave (rows of A x rows of W); WAVES_M x (WAVES / WAVES_M) waves.
template <int WM, int WN, int WAVES_M, int EPI, int NSTAGE, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_wide_kernel(const bf16* __restrict__ A, int64_t lda,
                                                        const bf16* __restrict__ W, bf16* __restrict__ C, int64_t ldc,
                                                        int M, int N, int K, int chunks, int act,
                                                        float* __restrict__ partials) {
  constexpr int WAVES_N = WAVES / WAVES_M;
  constexpr int MT = WAVES_M * WM, NT = WAVES_N * WN;  // 16-row tiles of A and of W per workgroup
  constexpr int BM = MT * 16;
  constexpr int A_BLOCKS = MT * 2, W_BLOCKS = NT * 2;  // KiB blocks of a slab
  static_assert(A_BLOCKS % WAVES == 0 && W_BLOCKS % WAVES == 0, "every wave copies the same number of blocks");
  static_assert(EPI != 1 || WN % 2 == 0, "gate and factor tiles come in pairs");
  constexpr int APW = A_BLOCKS / WAVES, WPW = W_BLOCKS / WAVES;
  constexpr int STAGE = (A_BLOCKS + W_BLOCKS) * 512;  // elements
  __shared__ __attribute__((aligned(16))) __bf16 stages[NSTAGE * STAGE];
  const uint32_t lds_base = static_cast<uint32_t>(
      reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) __bf16*)stages));

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  // Which tile: workgroups go to the eight XCDs in turn, each with an L2 of its own; the numbering is turned round
  // so that an XCD gets a contiguous share of the tiles, and within it tiles go in columns eight wide, rows first.
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
  // this workgroup's share of K: slabs slab0 .. slab0 + slabs
  const int slabs_all = K / BK;
  const int slab0 = static_cast<int>(static_cast<int64_t>(blockIdx.z) * slabs_all / gridDim.z);
  const int slabs = static_cast<int>(static_cast<int64_t>(blockIdx.z + 1) * slabs_all / gridDim.z) - slab0;
  A += static_cast<size_t>(slab0) * BK;
  const int m_base = by * BM;
  const int NW = EPI == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  const int ntiles = (NW + 15) / 16;
  const int nt_base = bx * NT;

  // ---- what this wave copies of every slab: KiB blocks wave + WAVES i of A and of W.
  // A block b is rows 8 (b % 2) .. + 8 of tile b / 2, all 64 columns of the slab: eight lanes per row read its 128
  // bytes, so a load is eight whole lines.  In LDS a row's eight 16-byte pieces are permuted (piece p of row r of
  // the tile lies at p ^ (r / 2)), which makes the fragment reads below (16 rows, one piece each) hit all banks.
  // W block b is tile b / 2, columns 32 (b % 2) .. of the slab: a KiB as it lies in global memory.
  // Rows beyond M read row M - 1, tiles beyond the last the last one (their products are never stored).
  const int half_mine = wave % 2, tile_mine = wave / 2;
  uint32_t a_off[APW];  // bytes; the host checks that M * lda fits
#pragma unroll
  for (int i = 0; i < APW; ++i) {
    const int r = half_mine * 8 + lane / 8;  // row of the tile
    const int m = m_base + (tile_mine + (WAVES / 2) * i) * 16 + r;
    a_off[i] = (static_cast<uint32_t>(m < M ? m : M - 1) * static_cast<uint32_t>(lda) + ((lane % 8) ^ (r / 2)) * 8) * 2;
  }
  const bf16* w_from[WPW];  // the same for the whole wave
#pragma unroll
  for (int i = 0; i < WPW; ++i) {
    const int nt = nt_base + tile_mine + (WAVES / 2) * i;
    const int clamped = __builtin_amdgcn_readfirstlane(nt < ntiles ? nt : ntiles - 1);
    w_from[i] = W + (static_cast<size_t>(clamped) * chunks + half_mine) * 512 + static_cast<size_t>(slab0) * 1024;
  }
  // load n (of LOADS) of slab `slab` into buffer `buf`
  constexpr int LOADS = APW + WPW;
  auto request_one = [&](int n, int slab, int buf) __attribute__((always_inline)) {
    const uint32_t to = lds_base + static_cast<uint32_t>(buf) * (STAGE * 2);
    if (n < APW)
      load_to_lds(A + static_cast<size_t>(slab) * BK, a_off[n], to + ((tile_mine + (WAVES / 2) * n) * 2 + half_mine) * 1024);
    else
      load_to_lds(w_from[n - APW] + static_cast<size_t>(slab) * 1024, lane * 16,
                  to + (A_BLOCKS + (tile_mine + (WAVES / 2) * (n - APW)) * 2 + half_mine) * 1024);
  };

  floatx4 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // this lane's piece of an A fragment (row lane % 16, columns 32 kc + 8 (lane / 16) ..) within its tile, elements
  int a_frag[2];
#pragma unroll
  for (int kc = 0; kc < 2; ++kc) {
    const int r = lane % 16;
    a_frag[kc] = r * 64 + ((kc * 4 + lane / 16) ^ (r / 2)) * 8;
  }
  // Fragments of the two halves of a slab (columns 0 .. 31 and 32 .. 63) in registers of their own.  The products
  // of the second half are held back until after the next barrier, where they cover the time that the fragment
  // reads of the next slab's first half take; the reads of the second half are covered by the products of the
  // first.  So the MFMA unit always has products to do while LDS reads are under way.
  bf16x8 fa[2][WM], fw[2][WN];
  auto read = [&](const __bf16* stage, int kc) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
      fa[kc][i] = *reinterpret_cast<const bf16x8*>(stage + (wm * WM + i) * 1024 + a_frag[kc]);
#pragma unroll
    for (int j = 0; j < WN; ++j)
      fw[kc][j] = *reinterpret_cast<const bf16x8*>(stage + ((A_BLOCKS + (wn * WN + j) * 2 + kc) * 64 + lane) * 8);
  };
  // fragment n of half kc alone: W's first (the first row of products needs them all), then A's
  auto read_one = [&](const __bf16* stage, int kc, int n) __attribute__((always_inline)) {
    if (n < WN)
      fw[kc][n] = *reinterpret_cast<const bf16x8*>(stage + ((A_BLOCKS + (wn * WN + n) * 2 + kc) * 64 + lane) * 8);
    else
      fa[kc][n - WN] = *reinterpret_cast<const bf16x8*>(stage + (wm * WM + n - WN) * 1024 + a_frag[kc]);
  };
  // Tiles with enough products read the fragments of the other half one by one, each after one of the first
  // products of this half, instead of all of them before: a wave issues in order, and sixteen reads in a row keep
  // its products from the MFMA unit for a few hundred cycles.
  constexpr bool INTERLEAVED = WM * WN >= 2 * (WM + WN);
  // The products of half kc (`first`: 0 for the held-back half, which comes first after the barrier; 1 for the
  // other; -1: no loads).  After every EVERY products, counted through the slab, one load of slab `slab` is asked
  // for: spread out, so that the waves do not queue up at the memory pipeline (which takes 16 cycles for each) while
  // the MFMA unit idles, and early: with two buffers all of them among the first half's products, so that the
  // second half's cover the time that the last one takes.
  constexpr int SPAN = NSTAGE == 2 ? WM * WN : 2 * WM * WN;
  constexpr int EVERY = SPAN / LOADS > 0 ? SPAN / LOADS : 1;
  constexpr int PER = SPAN / LOADS > 0 ? 1 : (LOADS + SPAN - 1) / SPAN;  // (small tiles: several loads after each product)
  auto multiply = [&](int kc, int first, int slab, int buf, const __bf16* rstage = nullptr, int rkc = -1)
                      __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[kc][j], fa[kc][i], acc[i][j], 0, 0, 0);
        if (INTERLEAVED && rkc >= 0 && i * WN + j < WM + WN) {
          __builtin_amdgcn_sched_barrier(0);
          read_one(rstage, rkc, i * WN + j);
          __builtin_amdgcn_sched_barrier(0);
        }
        const int q = (first > 0 ? WM * WN : 0) + i * WN + j + 1;  // products of this slab so far
#pragma unroll
        for (int e = 0; e < PER; ++e) {
          const int n = (q / EVERY - 1) * PER + e;
          if (first >= 0 && q % EVERY == 0 && n < LOADS) {
            __builtin_amdgcn_sched_barrier(0);
            request_one(n, slab, buf);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
    }
  };
  // The slabs go round NSTAGE buffers.  Before the barrier of slab s this wave's loads of slab s have arrived (those
  // of the NSTAGE - 2 slabs after it may be under way) and its fragment reads of slab s - 1 are done; after it
  // everyone's, so that the loads of slab s + NSTAGE - 1 may go into the buffer of slab s - 1.  Past the last slab
  // the last one is loaded again (no branch).
#pragma unroll
  for (int p = 0; p < NSTAGE; ++p)
#pragma unroll
    for (int n = 0; n < LOADS; ++n) request_one(n, p < slabs ? p : slabs - 1, p);
  // slab 0: nothing held back yet, and its loads for later are already asked for
  __builtin_amdgcn_s_waitcnt(waitcnt_vm((NSTAGE - 1) * LOADS));
  bare_barrier();
  read(stages, 0);
  read(stages, 1);
  __builtin_amdgcn_sched_barrier(0);
  multiply(0, -1, 0, 0);
  int cur = 1, target = 0;
  for (int s = 1; s < slabs; ++s) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((NSTAGE - 2) * LOADS) & ~(15 << 8));
    bare_barrier();
    const int ahead = s + NSTAGE - 1 < slabs ? s + NSTAGE - 1 : slabs - 1;
    const __bf16* stage = stages + cur * STAGE;
    if (INTERLEAVED) {
      multiply(1, 0, ahead, target, stage, 0);
      __builtin_amdgcn_sched_barrier(0);
      multiply(0, 1, ahead, target, stage, 1);
    } else {
      read(stage, 0);
      __builtin_amdgcn_sched_barrier(0);
      multiply(1, 0, ahead, target);
      __builtin_amdgcn_sched_barrier(0);  // (reads moved up among these products would need registers of their own)
      read(stage, 1);
      __builtin_amdgcn_sched_barrier(0);
      multiply(0, 1, ahead, target);
    }
    target = cur;
    cur = cur + 1 == NSTAGE ? 0 : cur + 1;
  }
  multiply(1, -1, 0, 0);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // the loads asked for beyond the last slab

  // ---- epilogue.  acc[i][j][v] is the product at row (tile i, lane % 16) of A and row (tile j, 4 (lane / 16) + v)
  // of W.
  const int row = lane % 16, quad = lane / 16;
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int m = m_base + (wm * WM + i) * 16 + row;
    if (m >= M) continue;
    if (EPI == 3) {  // this workgroup's share of the sum, as it is
      float* p_row = partials + (static_cast<size_t>(blockIdx.z) * M + m) * N;
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const int n = (nt_base + wn * WN + j) * 16 + quad * 4;
        if (n < N) *reinterpret_cast<floatx4*>(p_row + n) = acc[i][j];
      }
      continue;
    }
    bf16* c_row = C + static_cast<size_t>(m) * ldc;
    constexpr int OUT = EPI == 1 ? WN / 2 : WN;
#pragma unroll
    for (int j = 0; j < OUT; ++j) {
      const int tile = EPI == 1 ? (nt_base + wn * WN) / 2 + j : nt_base + wn * WN + j;
      const int n = tile * 16 + quad * 4;
      if (n >= N) continue;
      float x[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        if (EPI == 1)
          x[v] = gated_activation(act, to_float(float_to_bf16(acc[i][2 * j][v]))) *
                 to_float(float_to_bf16(acc[i][2 * j + 1][v]));
        else
          x[v] = acc[i][j][v];
      }
      uint2 packed;
      packed.x = static_cast<uint32_t>(float_to_bf16(x[0]).bits) | (static_cast<uint32_t>(float_to_bf16(x[1]).bits) << 16);
      packed.y = static_cast<uint32_t>(float_to_bf16(x[2]).bits) | (static_cast<uint32_t>(float_to_bf16(x[3]).bits) << 16);
      *reinterpret_cast<uint2*>(c_row + n) = packed;
    }
  }
}

template <int WM, int WN, int WAVES_M, int NSTAGE, int WAVES = 8>
static void launch(const bf16* A, int64_t lda, const bf16* W, bf16* C, int64_t ldc, int M, int N, int K, int epi,
                   int act, int ks, float* partials, hipStream_t stream) {
  constexpr int BM = WAVES_M * WM * 16, BNW = (WAVES / WAVES_M) * WN * 16;
  const int NW = epi == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  const dim3 grid((NW + BNW - 1) / BNW, (M + BM - 1) / BM, ks);
  if (epi == 1)
    gemm_wide_kernel<WM, WN, WAVES_M, 1, NSTAGE, WAVES><<<grid, WAVES * 64, 0, stream>>>(A, lda, W, C, ldc, M, N, K, K / 32,
                                                                                         act, nullptr);
  else if (ks > 1)
    gemm_wide_kernel<WM, WN, WAVES_M, 3, NSTAGE, WAVES><<<grid, WAVES * 64, 0, stream>>>(A, lda, W, C, ldc, M, N, K, K / 32,
                                                                                         act, partials);
  else
    gemm_wide_kernel<WM, WN, WAVES_M, 0, NSTAGE, WAVES><<<grid, WAVES * 64, 0, stream>>>(A, lda, W, C, ldc, M, N, K, K / 32,
                                                                                         act, nullptr);
}

}  // namespace wide

bool gemm_wide_takes(int M, int N, int K, int64_t lda, int64_t ldc, const void* A, const void* W, const void* W2,
                     const void* C, int c_dtype, int epi, int packed) {
  auto aligned = [](const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
  return packed && W2 == nullptr && (epi == 0 || epi == 1) && c_dtype == kBF16 && M >= 1 && K % wide::BK == 0 &&
         N % 4 == 0 && lda % 8 == 0 && ldc % 4 == 0 && aligned(A, 16) && aligned(W, 16) && aligned(C, 8) &&
         static_cast<int64_t>(M) * lda < (int64_t{1} << 31);  // byte offsets of rows are kept in 32 bits
}

// The tile and the cut of K for a product whose caller fixes neither, and the time that this kernel is expected to
// take with them in microseconds (the figure by which the library chooses between its product kernels).
static double plan_shape(int M, int N, int K, int epi, bool have_workspace, size_t workspace_bytes, int& shape, int& ks) {
  const int NW_all = epi == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  // without a fitted model below: the weights streamed once at the rate this kernel reaches for few rows, or the
  // products at its rate for many, whichever takes longer, after its start
  double us = 5.0 + 0.02 * (M < 64 ? M : 64) +
              fmax(2.0 * NW_all * K / 5.8e6, static_cast<double>(M) * NW_all * K / (1.05e9 / 2));
  // The cost of a shape: the workgroups that the busiest CU gets times the size of the tile; of equals the first.
  // Workgroups of four waves run two to a CU, where one's epilogue and first loads overlap the other's
  // products (measured: 7-9 % faster than one workgroup of twice the tile once every CU has two of them;
  // slower when it has one; from one and a half per CU on it is also the best for few rows of very many weight
  // rows, which are bound by streaming them).
  const int NW = epi == 1 ? 2 * ((N + 15) / 16) * 16 : N;
  const int shapes[5][4] = {{2128192, 128, 192, 93}, {2256192, 256, 192, 100}, {3256128, 256, 128, 100},
                            {3128256, 128, 256, 100}, {3192128, 192, 128, 100}};
  int64_t best = -1;
  for (const auto& sh : shapes) {
    const int64_t tiles = static_cast<int64_t>((M + sh[1] - 1) / sh[1]) * ((NW + sh[2] - 1) / sh[2]);
    if (sh[3] < 100 && tiles < wide::kCUs * 3 / 2) continue;
    const int64_t cost = ((tiles + wide::kCUs - 1) / wide::kCUs) * sh[1] * sh[2] * sh[3];
    if (best < 0 || cost < best) {
      best = cost;
      shape = sh[0];
    }
  }
  // A gated product of few rows whose tiles of 128 weight rows make one round at most (the 2B and 9B feed-forward
  // for up to 128 decoding requests) streams its weights: rows of 64 (or 128) with the deepest pipeline that fits
  // are 5 to 25 % faster there than the large tiles (2B at 64 rows: 23 against 28 us; 9B: 39 against 48).
  if (epi == 1 && M <= 128) {
    const int rows = M <= 64 ? 64 : 128;
    if (static_cast<int64_t>((M + rows - 1) / rows) * ((NW + 127) / 128) <= wide::kCUs) shape = M <= 64 ? 6064128 : 3128128;
  }
  // 17 to 1,536 rows without an epilogue (portions of prompts, many decoding requests): the tiles above are too few
  // for 256 CUs, and every workgroup walks all of K at the pace of its own slabs.  Smaller tiles with deeper
  // pipelines, and K cut over workgroups so that about one round of them covers the GPU, chosen by a model of the
  // time fitted to measurements at the 2B, 9B and 27B sizes (64 to 2,048 rows, seven tiles, one to fourteen cuts;
  // it is within 6 % of the best measured choice nearly everywhere, and a fifth faster in sum than either the
  // uncut tiles above or the tiled kernel with its cut: the 2B down projection at 512 rows takes 36 us against 55).
  if (epi == 0 && M <= 1536) {  // (fewer than 17 rows come here only against a very long K)
    struct Tile { int code, rows, wrows; double eff, start; };  // share of the MFMA rate in the loop; us to start
    static const Tile tiles[7] = {{3128128, 128, 128, 0.425, 1.44}, {3128256, 128, 256, 0.535, 2.03},
                                  {3192128, 192, 128, 0.535, 1.25}, {3256128, 256, 128, 0.615, 1.58},
                                  {5128064, 128, 64, 0.326, 0.85},  {6064064, 64, 64, 0.234, 0.80},
                                  {6064128, 64, 128, 0.277, 1.08}};
    const int slabs = K / wide::BK;
    double best_us = -1.0;
    int best_ks = 1;
    for (const Tile& t : tiles) {
      const int64_t count = static_cast<int64_t>((M + t.rows - 1) / t.rows) * ((N + t.wrows - 1) / t.wrows);
      const int cuts[3] = {1, static_cast<int>(wide::kCUs / count), static_cast<int>(2 * wide::kCUs / count)};
      for (int c = 0; c < 3; ++c) {
        const int cut = cuts[c];
        if (cut < 1 || (c > 0 && (cut < 2 || cut == cuts[c - 1])) || cut > slabs / 4) continue;
        const double partial_bytes = static_cast<double>(cut) * M * N * 4;
        if (cut > 1 && (!have_workspace || partial_bytes > static_cast<double>(workspace_bytes))) continue;
        const int64_t rounds = (count * cut + wide::kCUs - 1) / wide::kCUs;
        const int per = (slabs + cut - 1) / cut;
        // a CU's MFMA rate: 4.9 M multiply-adds of bfloat16 a microsecond
        double us = rounds * (static_cast<double>(per) * t.rows * t.wrows * wide::BK / (4.9e6 * t.eff) + t.start) + 3.2;
        if (cut > 1) us += partial_bytes / 5.5e6 + partial_bytes / 4.9e6 + 3.7;  // written, read again, the sum kernel
        if (best_us < 0 || us < best_us) {
          best_us = us;
          shape = t.code;
          best_ks = cut;
        }
      }
    }
    if (ks == 1) ks = best_ks;
    // (the model of the tiles knows nothing of memory: the weights streamed once from HBM are a floor under it)
    if (best_us >= 0) us = fmax(best_us, 5.0 + 0.02 * (M < 64 ? M : 64) + 2.0 * NW_all * K / 5.8e6);
  }
  return us;
}

// shape: 0: chosen here; else stages * 1000000 + rows * 1000 + weight rows of a workgroup's tile (2256192, 3256128,
// 3128256, 3192128; 2128192: workgroups of four waves, two to a CU).
// ks > 1 cuts K over that many workgroups per tile (no epilogue only; the partial tiles go through `workspace`,
// which must hold ks * M * N floats).
int gemm_wide(const void* A, int64_t lda, const void* W, void* C, int64_t ldc, int M, int N, int K, int epi, int act,
              int shape, int ks, void* workspace, size_t workspace_bytes, hipStream_t stream, int* planes_left) {
  if (ks < 1) ks = 1;
  if (ks > K / wide::BK) ks = K / wide::BK;
  if (ks > 1 && (epi != 0 || workspace == nullptr || static_cast<size_t>(ks) * M * N * sizeof(float) > workspace_bytes)) {
    set_error("gemm: the wide kernel cuts K only without an epilogue and with a workspace of ks * M * N floats");
    return 1;
  }
  float* ws = static_cast<float*>(workspace);
  const bf16* a = static_cast<const bf16*>(A);
  const bf16* w = static_cast<const bf16*>(W);
  bf16* c = static_cast<bf16*>(C);
  if (shape == 0) plan_shape(M, N, K, epi, ws != nullptr, workspace_bytes, shape, ks);
  switch (shape) {
    case 2256192: wide::launch<4, 6, 4, 2>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 3256128: wide::launch<4, 4, 4, 3>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 3128256: wide::launch<4, 4, 2, 3>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 3192128: wide::launch<3, 4, 4, 3>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 2128192: wide::launch<4, 6, 2, 2, 4>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;  // two workgroups per CU
    // small tiles, for products of a few hundred rows whose large tiles would leave most CUs idle (two or more
    // workgroups per CU fit: 36 to 72 KiB of LDS each)
    case 3128128: wide::launch<2, 4, 4, 3>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 3128064: wide::launch<2, 2, 4, 3>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 3064128: wide::launch<1, 4, 4, 3>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 3064064: wide::launch<1, 2, 4, 3>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 6064064: wide::launch<1, 2, 4, 6>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 5128064: wide::launch<2, 2, 4, 5>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 4128128: wide::launch<2, 4, 4, 4>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    case 6064128: wide::launch<1, 4, 4, 6>(a, lda, w, c, ldc, M, N, K, epi, act, ks, ws, stream); break;
    default:
      set_error("gemm: unknown wide tile %d", shape);
      return 1;
  }
  if (check_launch("gemm_wide")) return 1;
  if (planes_left != nullptr) {  // the caller adds the cuts' partial results up itself (ks planes of [M, N] floats)
    *planes_left = ks;
    return 0;
  }
  if (ks > 1) return gemm_sum_partials(ws, ks, C, kBF16, ldc, M, N, N, 0, 0, 0.f, stream);
  return 0;
}


double gemm_wide_predict_us(int M, int N, int K, int epi, bool have_workspace, size_t workspace_bytes) {
  int shape = 0, ks = 1;
  return plan_shape(M, N, K, epi, have_workspace, workspace_bytes, shape, ks);
}

}  // namespace sa
