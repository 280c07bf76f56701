// The decode step's "norm, then matrix product" in one kernel, for up to 16 rows in bfloat16:
//
//     h_out = h_in + norm_post(y)                  (y null: h_out = h_in and nothing is written)
//     a     = norm_next(h_out)                     bfloat16, kept in LDS
//     C     = epilogue(a . W^T)                    W tiled; epilogue none, gated (paired tiles) or soft-cap
//
// where norm(x; w) = x * rsqrt(mean(x^2) + eps) * (w + plus_one), all in float32.  It replaces the separate
// residual-and-norm kernel that would otherwise run between every two products of a block: at a handful of
// rows that kernel is pure launch latency.  Every workgroup recomputes the two norms of all rows (the rows are
// a few KiB and lie in L2), puts the activations into LDS, from where they feed the MFMA as the B operand, and
// then streams 16-row tiles of W as the few-rows product kernel does.  At most one workgroup per compute unit
// is launched and each takes several tiles, so that the norms are redone 256 times at most.  Workgroup 0 also writes h_out,
// to a buffer other than h_in: workgroups start at different times, so h_in must stay what it was.
#include "api.h"
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

namespace normed {

constexpr int kWaves = 8;
constexpr int kMaxGroups = 256;  // one workgroup per compute unit; each takes the same number of tiles, or one fewer

__device__ inline bf16x8 load_frag(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }

// What the rotary epilogue (EPI 3) needs: the product is the fused q/k/v projection of an attention layer, columns
// [H query heads | Kh key heads | Kh value heads] of hd each.  Query and key heads are rotated by the token's
// position (pairs (i, i + hd / 2), angle position / timescale[i] / scale_factor), queries divided by q_div and
// written to C, keys and values written into the cache pages at slot_mapping[row] (as the separate rotary kernel
// does, from the product rounded to bfloat16 as that kernel reads it).
struct RotaryArgs {
  const int* positions;
  const float* timescale;       // [hd / 2], or null: no rotation
  float inv_scale_factor, q_div;
  const int64_t* slot_mapping;  // null: nothing is written into the cache
  bf16* k_pages;
  bf16* v_pages;
  int H, Kh, hd, page_size;
};

// NCH: 256-element pieces of a row (K <= 256 * NCH): 10, 14 or 18
// kUnroll: fragments of a register set (chunks of 32 columns of K whose loads a wave issues together); 4: sets of 5,
// two to a tile at the 2B width instead of three, were no faster (q/k/v 8.8 against 8.1 us at one row)
template <int EPI, int NCH, bool EXACT, int kUnroll>
__global__ __launch_bounds__(kWaves* kWave) void gemm_normed_kernel(
    const bf16* __restrict__ y, const float* __restrict__ h_in, float* __restrict__ h_out,
    const void* __restrict__ w_post, int w_post_dtype, float eps_post, float plus_post,
    const void* __restrict__ w_next, int w_next_dtype, float eps_next, float plus_next, const bf16* __restrict__ W,
    void* __restrict__ C, int c_dtype, int64_t ldc, int M, int N, int K, int chunks, int act_rows, float cap,
    int activation, RotaryArgs rot) {
  constexpr int NP = (EPI == 1 || EPI == 3) ? 2 : 1;  // tiles of W that a workgroup multiplies side by side
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int pitch = K + 8;                               // elements per row of activations in LDS
  bf16* act = reinterpret_cast<bf16*>(smem);             // [act_rows][pitch]
  float* red = reinterpret_cast<float*>(smem + static_cast<size_t>(act_rows) * pitch * sizeof(bf16));  // [waves][NP][16 * 17]

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r = lane % 16, kq = lane / 16;

  // ---- set-up of the product: a workgroup takes the 16-row tiles of W (pairs of tiles for the gated epilogue)
  // blockIdx.x, blockIdx.x + gridDim.x, ...; K is cut over the waves.  The first fragments of W are asked for
  // before the norms, so that their way from HBM overlaps the norms' trips to L2.
  // work items: 16-row tiles of W; pairs (2 i, 2 i + 1) for the gated epilogue; for the rotary epilogue pairs
  // (t, t + hd / 32) of a head's tiles, which hold the two dimensions of every rotated pair
  const int half_tiles = EPI == 3 ? rot.hd / 32 : 1;
  const int ntiles = EPI == 3 ? (rot.H + 2 * rot.Kh) * half_tiles : (N + 15) / 16;
  const int c0 = static_cast<int>(static_cast<int64_t>(chunks) * wave / kWaves);
  const int c1 = static_cast<int>(static_cast<int64_t>(chunks) * (wave + 1) / kWaves);
  const size_t tile_elems = static_cast<size_t>(chunks) * 512;
  const size_t pair_off = (EPI == 3 ? half_tiles : 1) * tile_elems;  // from the first tile of an item to its second
  auto tile_ptr = [&](int item) {
    const int first = EPI == 1 ? 2 * item : EPI == 3 ? (item / half_tiles) * 2 * half_tiles + item % half_tiles : item;
    return W + static_cast<size_t>(first) * tile_elems + lane * 8;
  };
  const bf16* wrow = tile_ptr(blockIdx.x);
  const bf16* w2row = wrow + pair_off;
  const bf16* arow = act + static_cast<size_t>(r) * pitch + kq * 8;
  const bool a_ok = r < act_rows;
  const bf16x8 zero = {};
  floatx4 acc[NP];

  bf16x8 a[2][kUnroll], a2[2][kUnroll];
  auto load_set = [&](int set, int c) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const bool ok = c + u < c1;
      a[set][u] = ok ? load_frag(wrow + static_cast<size_t>(c + u) * 512) : zero;
      if (NP == 2) a2[set][u] = ok ? load_frag(w2row + static_cast<size_t>(c + u) * 512) : zero;
    }
  };
  auto mul_set = [&](int set, int c) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      // beyond the wave's range the W fragment is zero; the activations read there are finite (zero padded rows)
      const int k = (c + u < c1 ? c + u : c0) * 32;
      const bf16x8 b = a_ok ? load_frag(arow + k) : zero;
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[set][u], b, acc[0], 0, 0, 0);
      if (NP == 2) acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[set][u], b, acc[1], 0, 0, 0);
    }
  };
  const int nseg = (c1 - c0 + kUnroll - 1) / kUnroll;  // sets of fragments per tile for this wave
  // (rows of more than 3584 elements leave no registers for the second set during the norms)
  constexpr bool kBothSetsFirst = NCH <= 14;
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  const bool add = y != nullptr, post = add && w_post != nullptr;
  if constexpr (EXACT) {
    // The first fragments of W are asked for before the norms are computed, so that their way from HBM overlaps the
    // norms; but after the loads of the wave's first row: loads come back in the order in which they were asked
    // for, and the norms, whose operands lie in L2, must not wait for the weights.  Unconditional loads (a chunk
    // beyond the wave's share reads the last chunk and is set to zero afterwards): with a branch around a load the
    // compiler waits for all loads in flight where it next uses one.
    // (`from`: the tile's first fragment of this lane, through a value that the compiler cannot see through and that
    // is made after the row's loads: it would otherwise move the weights' loads up to the kernel's start)
    auto load_first = [&](int set, int c, const bf16* from) __attribute__((always_inline)) {
  #pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const size_t at = static_cast<size_t>(c + u < chunks ? c + u : chunks - 1) * 512;
        a[set][u] = load_frag(from + at);
        if (NP == 2) a2[set][u] = load_frag(from + pair_off + at);
      }
    };
    auto zero_beyond = [&](int set, int c) __attribute__((always_inline)) {
  #pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        a[set][u] = c + u < c1 ? a[set][u] : zero;
        if (NP == 2) a2[set][u] = c + u < c1 ? a2[set][u] : zero;
      }
    };

    // ---- the two norms, one wave per row.  A lane holds 4 consecutive elements of each 256-element piece of the
    // row; all loads of a row are issued before the first use, so a row costs one trip to L2.
    // (rows of more than 2560 elements: the norms' scale factors are read where they are used, from L1 after the
    // first row, instead of ahead with the row: the registers do not hold both)
    constexpr bool kAhead = NCH <= 10;
    float4 hv[NCH];
    bf16x4 yv[NCH], wpv[kAhead ? NCH : 1], wnv[kAhead ? NCH : 1];
    const bf16* wp16 = static_cast<const bf16*>(w_post);
    const bf16* wn16 = static_cast<const bf16*>(w_next);
    // what is not there (no y, no post-norm) is read from what is, and not used: every load is unconditional
    const bf16* y_from = add ? y : reinterpret_cast<const bf16*>(h_in);
    const bf16* wp_from = post ? wp16 : wn16;
    auto ask_row = [&](int m) __attribute__((always_inline)) {
      const size_t rb = static_cast<size_t>(m < M ? m : M - 1) * K;
  #pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = c * 256 + lane * 4, at = (EXACT || d < K) ? d : 0;
        hv[c] = *reinterpret_cast<const float4*>(h_in + rb + at);
        yv[c] = *reinterpret_cast<const bf16x4*>(y_from + rb + at);
        if constexpr (kAhead) {
          wpv[c] = *reinterpret_cast<const bf16x4*>(wp_from + at);
          wnv[c] = *reinterpret_cast<const bf16x4*>(wn16 + at);
        }
      }
    };
    // (No branch between a row's loads and their first use: the compiler would move the loads into the branch, behind
    // the weights' loads.  What a branch would skip is computed and dropped by a select.)
    auto norm_row = [&](int m) __attribute__((always_inline)) {
      bf16* dst = act + static_cast<size_t>(m) * pitch;
      const bool valid = m < M;
      const size_t rb = static_cast<size_t>(valid ? m : M - 1) * K;
      auto post_scale = [&](int c, int d) __attribute__((always_inline)) {
        if constexpr (kAhead) return wpv[c];
        else return *reinterpret_cast<const bf16x4*>(wp_from + d);
      };
      auto next_scale = [&](int c, int d) __attribute__((always_inline)) {
        if constexpr (kAhead) return wnv[c];
        else return *reinterpret_cast<const bf16x4*>(wn16 + d);
      };
      float ss = 0.f;
  #pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const bool in_row = EXACT || c * 256 + lane * 4 < K;  // (pieces beyond the row were read from its start: zeros in the sums)
  #pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = in_row ? static_cast<float>(yv[c][e]) : 0.f;
          ss += v * v;
        }
      }
      const float rr = post ? rsqrtf(wave_sum(ss) / static_cast<float>(K) + eps_post) : 1.f;
      // (the row's y is converted to float again below, from a value that the compiler takes for a new one: it would
      // otherwise keep the first loop's 4 NCH floats alive through the sum, which at 14 and 18 pieces is what spills)
      if constexpr (NCH > 10) {
  #pragma unroll
        for (int c = 0; c < NCH; ++c) asm volatile("" : "+v"(yv[c]));
      }
      float ss2 = 0.f;
  #pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = c * 256 + lane * 4;
        const bool in_row = EXACT || d < K;
        float* h = reinterpret_cast<float*>(&hv[c]);
        const bf16x4 ws = post_scale(c, in_row ? d : 0);
  #pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = static_cast<float>(yv[c][e]);
          const float t = post ? v * rr * (static_cast<float>(ws[e]) + plus_post) : v;
          h[e] = in_row ? h[e] + (add ? t : 0.f) : 0.f;
          ss2 += h[e] * h[e];
        }
      }
      if (add && blockIdx.x == 0 && valid) {
  #pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int d = c * 256 + lane * 4;
          if (EXACT || d < K) *reinterpret_cast<float4*>(h_out + rb + d) = hv[c];
        }
      }
      const float r2 = rsqrtf(wave_sum(ss2) / static_cast<float>(K) + eps_next);
  #pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = c * 256 + lane * 4;
        if (!EXACT && d >= K) continue;
        const float* h = reinterpret_cast<const float*>(&hv[c]);
        const bf16x4 ws = next_scale(c, d);
  #pragma unroll
        for (int e = 0; e < 4; ++e)
          dst[d + e] = float_to_bf16(valid ? h[e] * r2 * (static_cast<float>(ws[e]) + plus_next) : 0.f);
      }
      for (int d = K + lane; d < pitch; d += kWave) dst[d] = float_to_bf16(0.f);
    };
    auto zero_row = [&](int m) __attribute__((always_inline)) {
      bf16* dst = act + static_cast<size_t>(m) * pitch;
      for (int d = lane; d < pitch; d += kWave) dst[d] = float_to_bf16(0.f);
    };
    // A wave without a row (fewer rows than waves) asks for no row: the loads of a workgroup's eight waves go through
    // one path of 64 bytes a clock, and eight copies of a row (a single request decoding) would hold the weights up.
    int lane_elems = lane * 8;
    if (wave < M) {
      ask_row(wave);
      asm volatile("" : "+v"(lane_elems));
      const bf16* first_from = wrow - lane * 8 + lane_elems;
      __builtin_amdgcn_sched_barrier(0);
      load_first(0, c0, first_from);
      __builtin_amdgcn_sched_barrier(0);
      norm_row(wave);
    } else {
      load_first(0, c0, wrow);
      zero_row(wave);
    }
    asm volatile("" : "+v"(lane_elems));
    const bf16* second_from = wrow - lane * 8 + lane_elems;
    __builtin_amdgcn_sched_barrier(0);
    if (kBothSetsFirst) load_first(1, c0 + kUnroll, second_from);   // on its way during the further rows, the barrier and the first set's products
    for (int m = wave + kWaves; m < act_rows; m += kWaves) {
      if (m < M) {
        ask_row(m);
        norm_row(m);
      } else {
        zero_row(m);
      }
    }
    zero_beyond(0, c0);
    if (kBothSetsFirst) zero_beyond(1, c0 + kUnroll);
  } else {
    // both sets of fragments are asked for before the norms: a wave's share of a tile is two or three sets, so most
    // of the first tile is on its way while the norms are computed
    load_set(0, c0);
    if (kBothSetsFirst && nseg >= 2) load_set(1, c0 + kUnroll);

    // ---- the two norms, one wave per row.  A lane holds 4 consecutive elements of each 256-element piece of the
    // row; all loads of a row are issued before the first use, so a row costs one trip to L2.
    for (int m = wave; m < act_rows; m += kWaves) {
      bf16* dst = act + static_cast<size_t>(m) * pitch;
      if (m >= M) {
        for (int d = lane; d < pitch; d += kWave) dst[d] = float_to_bf16(0.f);
        continue;
      }
      const size_t rb = static_cast<size_t>(m) * K;
      // (rows of more than 2560 elements: the norms' scale factors are read where they are used, from L1 after the
      // first row, instead of ahead with the row: the registers do not hold both)
      constexpr bool kAhead = NCH <= 10;
      float4 hv[NCH];
      bf16x4 yv[NCH], wpv[kAhead ? NCH : 1], wnv[kAhead ? NCH : 1];
      const bf16* wp16 = static_cast<const bf16*>(w_post);
      const bf16* wn16 = static_cast<const bf16*>(w_next);
  #pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = c * 256 + lane * 4;
        hv[c] = d < K ? *reinterpret_cast<const float4*>(h_in + rb + d) : float4{0.f, 0.f, 0.f, 0.f};
        yv[c] = (add && d < K) ? *reinterpret_cast<const bf16x4*>(y + rb + d) : bf16x4{};
        if constexpr (kAhead) {
          wpv[c] = (post && d < K) ? *reinterpret_cast<const bf16x4*>(wp16 + d) : bf16x4{};
          wnv[c] = d < K ? *reinterpret_cast<const bf16x4*>(wn16 + d) : bf16x4{};
        }
      }
      auto post_scale = [&](int c, int d) __attribute__((always_inline)) {
        if constexpr (kAhead) return wpv[c];
        else return *reinterpret_cast<const bf16x4*>(wp16 + d);
      };
      auto next_scale = [&](int c, int d) __attribute__((always_inline)) {
        if constexpr (kAhead) return wnv[c];
        else return *reinterpret_cast<const bf16x4*>(wn16 + d);
      };
      if (add) {
        float rr = 1.f;
        if (post) {
          float ss = 0.f;
  #pragma unroll
          for (int c = 0; c < NCH; ++c)
  #pragma unroll
            for (int e = 0; e < 4; ++e) ss += static_cast<float>(yv[c][e]) * static_cast<float>(yv[c][e]);
          rr = rsqrtf(wave_sum(ss) / static_cast<float>(K) + eps_post);
        }
  #pragma unroll
        for (int c = 0; c < NCH; ++c) {
          const int d = c * 256 + lane * 4;
          if (d >= K) continue;
          float* h = reinterpret_cast<float*>(&hv[c]);
          const bf16x4 ws = post ? post_scale(c, d) : bf16x4{};
  #pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float v = static_cast<float>(yv[c][e]);
            h[e] += post ? v * rr * (static_cast<float>(ws[e]) + plus_post) : v;
          }
          if (blockIdx.x == 0) *reinterpret_cast<float4*>(h_out + rb + d) = hv[c];
        }
      }
      float ss2 = 0.f;
  #pragma unroll
      for (int c = 0; c < NCH; ++c) ss2 += hv[c].x * hv[c].x + hv[c].y * hv[c].y + hv[c].z * hv[c].z + hv[c].w * hv[c].w;
      const float r2 = rsqrtf(wave_sum(ss2) / static_cast<float>(K) + eps_next);
  #pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d = c * 256 + lane * 4;
        if (d >= K) continue;
        const float* h = reinterpret_cast<const float*>(&hv[c]);
        const bf16x4 ws = next_scale(c, d);
  #pragma unroll
        for (int e = 0; e < 4; ++e)
          dst[d + e] = float_to_bf16(h[e] * r2 * (static_cast<float>(ws[e]) + plus_next));
      }
      for (int d = K + lane; d < pitch; d += kWave) dst[d] = float_to_bf16(0.f);
    }
  }
  if (!kBothSetsFirst && nseg >= 2) load_set(1, c0 + kUnroll);
  __syncthreads();

  for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
#pragma unroll
    for (int p = 0; p < NP; ++p) acc[p] = floatx4{0.f, 0.f, 0.f, 0.f};
    const bool more = tile + static_cast<int>(gridDim.x) < ntiles;
    const bf16* const here = wrow;
    const bf16* const next = tile_ptr(tile + gridDim.x);
    // at the start of a tile set 0 holds its first fragments and set 1 its second ones; each set is asked for
    // again as soon as it has been used: for two sets further on in this tile, or for the next tile's start
    auto refill = [&](int set, int seg) {
      if (seg < nseg) {
        load_set(set, c0 + seg * kUnroll);
      } else if (more && set < nseg) {  // set 0 takes the next tile's first fragments, set 1 its second ones
        wrow = next;
        w2row = next + pair_off;
        load_set(set, c0 + set * kUnroll);
        wrow = here;
        w2row = here + pair_off;
      }
    };
    for (int seg = 0; seg < nseg; seg += 2) {
      mul_set(0, c0 + seg * kUnroll);
      refill(0, seg + 2);
      if (seg + 1 < nseg) {
        mul_set(1, c0 + (seg + 1) * kUnroll);
        refill(1, seg + 3);
      }
    }
    wrow = next;
    w2row = next + pair_off;

    // ---- lane holds D[n = 4 * kq + v][m = r]; the waves' tiles are added up through LDS, in wave order
    __syncthreads();  // the previous tile's sums have been read
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[(wave * NP + p) * (16 * 17) + (4 * kq + v) * 17 + r] = acc[p][v];
    __syncthreads();
    if (EPI == 3) {
      const int ml = tid / 16, nl = tid % 16;
      if (tid < 256 && ml < M) {
        float x[2];
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          float t = 0.f;
          for (int w = 0; w < kWaves; ++w) t += red[(w * NP + p) * (16 * 17) + nl * 17 + ml];
          x[p] = to_float(float_to_bf16(t));
        }
        const int head = tile / half_tiles, i = (tile % half_tiles) * 16 + nl, half = rot.hd / 2;
        float o1 = x[0], o2 = x[1];
        if (head < rot.H + rot.Kh && rot.timescale != nullptr) {
          float sn, cs;
          sincosf(static_cast<float>(rot.positions[ml]) / rot.timescale[i] * rot.inv_scale_factor, &sn, &cs);
          o1 = x[0] * cs - x[1] * sn;
          o2 = x[1] * cs + x[0] * sn;
        }
        if (head < rot.H) {
          const size_t at = static_cast<size_t>(ml) * ldc + static_cast<size_t>(head) * rot.hd + i;
          store_f(C, c_dtype, at, o1 / rot.q_div);
          store_f(C, c_dtype, at + half, o2 / rot.q_div);
        } else if (rot.slot_mapping != nullptr && rot.slot_mapping[ml] >= 0) {
          const int64_t slot = rot.slot_mapping[ml];
          const int64_t page = slot / rot.page_size;
          const int koff = static_cast<int>(slot % rot.page_size);
          if (head < rot.H + rot.Kh) {
            bf16* dst = rot.k_pages + (page * rot.Kh + (head - rot.H)) * rot.page_size * rot.hd;
            const bool tiled = keys_tiled(rot.page_size, rot.hd);
            dst[key_index(tiled, rot.page_size, rot.hd, koff, i)] = float_to_bf16(o1);
            dst[key_index(tiled, rot.page_size, rot.hd, koff, i + half)] = float_to_bf16(o2);
          } else {  // value pages are [page, head, hd, page_size]
            bf16* dst = rot.v_pages + (page * rot.Kh + (head - rot.H - rot.Kh)) * rot.page_size * rot.hd + koff;
            dst[static_cast<size_t>(i) * rot.page_size] = float_to_bf16(x[0]);
            dst[static_cast<size_t>(i + half) * rot.page_size] = float_to_bf16(x[1]);
          }
        }
      }
    } else if (tid < 256) {
      const int ml = tid / 16, nl = tid % 16, n = tile * 16 + nl;
      if (ml < M && n < N) {
        float sum[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
          float t = 0.f;
          for (int w = 0; w < kWaves; ++w) t += red[(w * NP + p) * (16 * 17) + nl * 17 + ml];
          sum[p] = t;
        }
        float v = sum[0];
        if (EPI == 1) v = gated_activation(activation, to_float(float_to_bf16(v))) * to_float(float_to_bf16(sum[NP - 1]));
        else if (EPI == 2) v = cap * tanhf(v / cap);
        store_f(C, c_dtype, static_cast<size_t>(ml) * ldc + n, v);
      }
    }
  }
}

template <int EPI, int NCH, bool EXACT = false, int kUnroll = 4>
static int launch(const bf16* y, const float* h_in, float* h_out, const void* w_post, int w_post_dtype, float eps_post,
                  float plus_post, const void* w_next, int w_next_dtype, float eps_next, float plus_next, const bf16* W,
                  void* C, int c_dtype, int64_t ldc, int M, int N, int K, float cap, int activation,
                  const RotaryArgs& rot, hipStream_t stream) {
  const int act_rows = M <= 8 ? 8 : 16;
  const size_t lds = static_cast<size_t>(act_rows) * (K + 8) * sizeof(bf16) +
                     static_cast<size_t>(kWaves) * ((EPI == 1 || EPI == 3) ? 2 : 1) * 16 * 17 * sizeof(float);
  auto kernel = gemm_normed_kernel<EPI, NCH, EXACT, kUnroll>;
  if (lds > 64 * 1024) {
    static bool raised = false;  // per instantiation
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        set_error("gemm_normed: the GPU refuses %zu bytes of LDS", lds);
        return 1;
      }
      raised = true;
    }
  }
  const int ntiles = EPI == 3 ? (rot.H + 2 * rot.Kh) * (rot.hd / 32) : (N + 15) / 16;
  const int grid = (ntiles + (ntiles + kMaxGroups - 1) / kMaxGroups - 1) / ((ntiles + kMaxGroups - 1) / kMaxGroups);
  kernel<<<grid, kWaves * kWave, lds, stream>>>(y, h_in, h_out, w_post, w_post_dtype, eps_post, plus_post, w_next,
                                                         w_next_dtype, eps_next, plus_next, W, C, c_dtype, ldc, M, N, K,
                                                         (K + 31) / 32, act_rows, cap, activation, rot);
  return check_launch("gemm_normed");
}

}  // namespace normed
}  // namespace sa

using namespace sa;

extern "C" int sa_gemm_normed_max_rows() { return 16; }

extern "C" int sa_gemm_normed_takes(int M, int N, int K) {
  const size_t lds = static_cast<size_t>(M <= 8 ? 8 : 16) * (K + 8) * 2 + 8 * 2 * 16 * 17 * 4;
  return M >= 1 && M <= sa_gemm_normed_max_rows() && K % 32 == 0 && K <= 256 * 18 && lds <= 160 * 1024;
}

// Widths of a whole number of 256-element pieces for which the prologue without per-piece tests is instantiated
// (SA_NORMED_K and the rotary dispatch below name the same ones).
static bool has_exact_prologue(int K) {
  switch (K) {
    case 2048: case 2304: case 2560: case 3072: case 3584: case 4096: case 4608: return true;
    default: return false;
  }
}

extern "C" int sa_gemm_normed_pays(int M, int N, int K) {
  // Up to 2560 wide every width gains (8.1 against 13.3 us for q/k/v at one row of 2304).  Wider rows leave the
  // kernel too few registers to have its first weights on their way during the norms unless the prologue has no
  // per-piece tests (5 to 25 % faster than the separate kernels at 3584 and 4608, slower without).  Against very many
  // weight rows (a head over a large vocabulary) the kernels that fill the GPU without the norms in front win.
  return sa_gemm_normed_takes(M, N, K) && (K <= 2560 || has_exact_prologue(K)) && N <= 16 * 8192;
}

extern "C" int sa_gemm_normed(const void* y, const float* h_in, float* h_out, const void* w_post, int w_post_dtype,
                              float eps_post, int plus_one_post, const void* w_next, int w_next_dtype, float eps_next,
                              int plus_one_next, const void* W, void* C, int c_dtype, int64_t ldc, int M, int N, int K,
                              int epilogue, float cap, hipStream_t stream) {
  SA_REQUIRE(sa_gemm_normed_takes(M, N, K),
             "gemm_normed takes 1..16 rows and a width that is a multiple of 32, at most 4608, and fits in LDS; got M=%d K=%d", M, K);
  SA_REQUIRE(N > 0 && ldc >= N && w_next != nullptr && h_in != nullptr && W != nullptr, "gemm_normed: bad arguments");
  SA_REQUIRE(w_next_dtype == kBF16 && (w_post == nullptr || w_post_dtype == kBF16),
             "gemm_normed: the norm weights must be bfloat16");
  SA_REQUIRE(y == nullptr || (h_out != nullptr && h_out != h_in),
             "gemm_normed: with y the updated residual goes to a buffer other than the input");
  const int activation = epilogue_activation(epilogue);
  epilogue = epilogue_kind(epilogue);
  SA_REQUIRE(epilogue >= 0 && epilogue <= 2 && (epilogue != 2 || cap > 0.f), "gemm_normed: bad epilogue");
  SA_REQUIRE(activation >= 0 && activation < kNumActivations && (epilogue == 1 || activation == 0),
             "gemm_normed: unknown activation %d", activation);
  const bf16* yb = static_cast<const bf16*>(y);
  const bf16* w = static_cast<const bf16*>(W);
  const float pp = plus_one_post ? 1.f : 0.f, pn = plus_one_next ? 1.f : 0.f;
#define SA_NORMED(EPI, NCH)                                                                                      \
  return normed::launch<EPI, NCH>(yb, h_in, h_out, w_post, w_post_dtype, eps_post, pp, w_next, w_next_dtype, eps_next, \
                                  pn, w, C, c_dtype, ldc, M, N, K, cap, activation, normed::RotaryArgs{}, stream)
#define SA_NORMED_EXACT(EPI, NCH)                                                                                  \
  return normed::launch<EPI, NCH, true>(yb, h_in, h_out, w_post, w_post_dtype, eps_post, pp, w_next, w_next_dtype,   \
                                        eps_next, pn, w, C, c_dtype, ldc, M, N, K, cap, activation, normed::RotaryArgs{}, \
                                        stream)
#define SA_NORMED_K(EPI)          \
  do {                            \
    /* rows of a whole number of 256-element pieces, up to 2560 wide: the prologue without per-piece tests */     \
    if (K == 2048) SA_NORMED_EXACT(EPI, 8);                                                                        \
    if (K == 2304) SA_NORMED_EXACT(EPI, 9);                                                                        \
    if (K == 2560) SA_NORMED_EXACT(EPI, 10);                                                                       \
    if (K == 3072) SA_NORMED_EXACT(EPI, 12);                                                                       \
    if (K == 3584) SA_NORMED_EXACT(EPI, 14);                                                                       \
    if (K == 4096) SA_NORMED_EXACT(EPI, 16);                                                                       \
    if (K == 4608) SA_NORMED_EXACT(EPI, 18);                                                                       \
    if (K <= 2560) SA_NORMED(EPI, 10); \
    if (K <= 3584) SA_NORMED(EPI, 14); \
    SA_NORMED(EPI, 18);           \
  } while (0)
  if (epilogue == 0) SA_NORMED_K(0);
  if (epilogue == 1) SA_NORMED_K(1);
  SA_NORMED_K(2);
#undef SA_NORMED_K
#undef SA_NORMED_EXACT
#undef SA_NORMED
}

// The fused q/k/v projection of an attention layer with the norms in front (as sa_gemm_normed) and, behind it, the
// rotation of queries and keys, the query scale and the write of keys and values into the cache pages (as
// sa_rope_cache_write): C receives the queries only, [M, >= H * hd] with rows of ldc elements.  W has (H + 2 Kh) * hd
// rows; hd is a multiple of 32.  timescale null: no rotation; slot_mapping null: nothing is written into the cache.
extern "C" int sa_gemm_normed_rotary(const void* y, const float* h_in, float* h_out, const void* w_post, int w_post_dtype,
                                     float eps_post, int plus_one_post, const void* w_next, int w_next_dtype,
                                     float eps_next, int plus_one_next, const void* W, void* C, int c_dtype, int64_t ldc,
                                     int M, int K, const int* positions, const float* timescale, float scale_factor,
                                     float q_div, const int64_t* slot_mapping, void* k_pages, void* v_pages, int H,
                                     int Kh, int hd, int page_size, hipStream_t stream) {
  SA_REQUIRE(H >= 0 && Kh >= 0 && H + 2 * Kh > 0 && hd > 0 && hd % 32 == 0,
             "gemm_normed_rotary: bad head counts, or a head size that is no multiple of 32 (H=%d K=%d hd=%d)", H, Kh, hd);
  const int N = (H + 2 * Kh) * hd;
  SA_REQUIRE(sa_gemm_normed_takes(M, N, K),
             "gemm_normed takes 1..16 rows and a width that is a multiple of 32, at most 4608, and fits in LDS; got M=%d K=%d", M, K);
  SA_REQUIRE(ldc >= static_cast<int64_t>(H) * hd && w_next != nullptr && h_in != nullptr && W != nullptr && C != nullptr &&
                 positions != nullptr,
             "gemm_normed_rotary: bad arguments");
  SA_REQUIRE(w_next_dtype == kBF16 && (w_post == nullptr || w_post_dtype == kBF16),
             "gemm_normed: the norm weights must be bfloat16");
  SA_REQUIRE(y == nullptr || (h_out != nullptr && h_out != h_in),
             "gemm_normed: with y the updated residual goes to a buffer other than the input");
  SA_REQUIRE(page_size > 0 && scale_factor > 0.f && q_div > 0.f, "gemm_normed_rotary: bad page size, scale factor or query scale");
  SA_REQUIRE(slot_mapping == nullptr || (k_pages != nullptr && v_pages != nullptr),
             "gemm_normed_rotary: slots come with key and value pages");
  normed::RotaryArgs rot{positions, timescale, 1.f / scale_factor, q_div, slot_mapping, static_cast<bf16*>(k_pages),
                         static_cast<bf16*>(v_pages), H, Kh, hd, page_size};
#define SA_ROTARY(NCH)                                                                                              \
  return normed::launch<3, NCH>(static_cast<const bf16*>(y), h_in, h_out, w_post, w_post_dtype, eps_post,             \
                                plus_one_post ? 1.f : 0.f, w_next, w_next_dtype, eps_next, plus_one_next ? 1.f : 0.f, \
                                static_cast<const bf16*>(W), C, c_dtype, ldc, M, N, K, 0.f, 0, rot, stream)
#define SA_ROTARY_EXACT(NCH)                                                                                        \
  return normed::launch<3, NCH, true>(static_cast<const bf16*>(y), h_in, h_out, w_post, w_post_dtype, eps_post,        \
                                      plus_one_post ? 1.f : 0.f, w_next, w_next_dtype, eps_next,                       \
                                      plus_one_next ? 1.f : 0.f, static_cast<const bf16*>(W), C, c_dtype, ldc, M, N, K, \
                                      0.f, 0, rot, stream)
  if (K == 2048) SA_ROTARY_EXACT(8);
  if (K == 2304) SA_ROTARY_EXACT(9);
  if (K == 2560) SA_ROTARY_EXACT(10);
  if (K == 3072) SA_ROTARY_EXACT(12);
  if (K == 3584) SA_ROTARY_EXACT(14);
  if (K == 4096) SA_ROTARY_EXACT(16);
  if (K == 4608) SA_ROTARY_EXACT(18);
#undef SA_ROTARY_EXACT
  if (K <= 2560) SA_ROTARY(10);
  if (K <= 3584) SA_ROTARY(14);
  SA_ROTARY(18);
#undef SA_ROTARY
}
