// Paged attention in bfloat16 for portions of prompts: many query tokens of one request over the keys that the
// request has so far.  Bound by the matrix cores and the softmax arithmetic, no longer by reading the keys: a
// workgroup of four waves takes 4 consecutive units of up to 16 query rows each (rows = tokens x query heads of
// one key/value head; the host cuts a request's tokens into such units) and one key/value head, and walks over the
// keys once for all 64 rows.  Each tile of 32 keys and its values go through LDS:
//
//     global -> registers         issued one tile ahead, while the current tile is computed
//     registers -> LDS            keys stay in their 16-key x 32-dimension blocks of MFMA operand order (a plain
//                                 copy); values, stored [hd, page_size] in their pages, are re-ordered into operand
//                                 blocks of 16 dimensions x 32 keys on the way
//     LDS -> MFMA                 every wave reads every block with one 16-byte read per lane and computes, for
//                                 its own 16 rows, S^T = K . Q^T, the soft-cap, mask and online softmax in float32,
//                                 and O^T += V^T . P^T, exactly as the few-rows kernel does
//
// A wave skips tiles that none of its rows can see, and the mask arithmetic on tiles that all of its rows see
// whole.  The exponentials are taken to base 2 with log2(e) folded into the constants.  When few workgroups would
// result (a short portion over a long context), the keys are also cut into ranges over workgroups, and the ranges
// are merged by the second kernel of the few-rows path.
#include "api.h"
#include "attention_common.h"

namespace sa {
namespace prefill {

constexpr int kUnitsPerGroup = 4;  // waves of a workgroup, each with a unit of up to 16 rows
constexpr float kLog2e = 1.4426950408889634f;

template <int NDC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void paged_attention_prefill_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const SeqMeta* __restrict__ units, int unit_begin,
    bf16* __restrict__ out, int64_t out_stride, int Kh, int G, int page_size, int window, float soft_cap,
    float* __restrict__ workspace) {
  constexpr int HD = NDC * 32;
  constexpr int NDB = HD / 16;          // output blocks of 16 dimensions
  constexpr int PPT = NDC / 2;          // 16-byte pieces of keys (and of values) per thread and tile
  constexpr int SUB = NDC * 64;         // pieces in a sub-tile of 16 keys
  static_assert(NDC % 2 == 0, "head size must be a multiple of 64");
  __shared__ __attribute__((aligned(16))) __bf16 k_s[2 * NDC * 512];  // [sub-tile][dc][lane][8]
  __shared__ __attribute__((aligned(16))) __bf16 v_s[NDB * 512];      // [db][lane][8]: 16 dimensions x 32 keys

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r = lane % 16, grp = lane / 16;
  const int split = blockIdx.x, num_splits = gridDim.x, kh = blockIdx.y;
  const int u0 = unit_begin + blockIdx.z * kUnitsPerGroup;

  // the keys that some row of the workgroup sees: [lo_g, hi_g)
  int lo_g = 0x7fffffff, hi_g = 0, slot = 0;
#pragma unroll
  for (int w = 0; w < kUnitsPerGroup; ++w) {
    const SeqMeta m = units[u0 + w];
    if (m.q_len > 0) {
      const int lo_w = (window > 0 && m.pos0 - window + 1 > 0) ? m.pos0 - window + 1 : 0;
      lo_g = lo_w < lo_g ? lo_w : lo_g;
      hi_g = m.pos0 + m.q_len > hi_g ? m.pos0 + m.q_len : hi_g;
      slot = m.slot;
    }
  }
  if (hi_g == 0) return;  // no rows at all (uniform over the workgroup)
  const int* table = block_table + static_cast<size_t>(slot) * table_stride;
  const int tile0 = lo_g / kTile, tile1 = (hi_g + kTile - 1) / kTile;
  const int ntiles = tile1 - tile0;
  const int tb = tile0 + static_cast<int>(static_cast<int64_t>(ntiles) * split / num_splits);
  const int te = tile0 + static_cast<int>(static_cast<int64_t>(ntiles) * (split + 1) / num_splits);

  // this wave's unit and this lane's row of it: query token qi, query head g of the group
  const SeqMeta sm = units[u0 + wave];
  const int rows = G * sm.q_len;  // <= 16
  const int qi = r / G, g = r % G;
  const bool row_ok = r < rows;
  const int pos_r = sm.pos0 + qi;
  const int lo_r = (window > 0 && pos_r - window + 1 > 0) ? pos_r - window + 1 : 0;
  // over the wave's rows: positions [pos_first, pos_last], lower bounds [lo_first, lo_last]
  const int pos_first = sm.pos0, pos_last = sm.pos0 + sm.q_len - 1;
  const int lo_first = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int lo_last = (window > 0 && pos_last - window + 1 > 0) ? pos_last - window + 1 : 0;

  // Q as B operands: lane (row r, grp) holds Q[row r][dc * 32 + grp * 8 .. + 8]
  bf16x8 qf[NDC];
  {
    const bf16* qp = q + static_cast<size_t>(sm.q_start + (row_ok ? qi : 0)) * q_stride +
                     static_cast<size_t>(kh * G + (row_ok ? g : 0)) * HD + grp * 8;
#pragma unroll
    for (int dc = 0; dc < NDC; ++dc) qf[dc] = row_ok ? *reinterpret_cast<const bf16x8*>(qp + dc * 32) : bf16x8{};
  }

  floatx4 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) acc[db] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;  // per row, in units of log2; l_run is this lane group's share

  // scores in base-2 units: y = log2(e) * cap * tanh(s / cap) = c2 - 2 * c2 / (2^(s * c1) + 1), or log2(e) * s
  const float c1 = soft_cap > 0.f ? 2.f * kLog2e / soft_cap : kLog2e;
  const float c2 = soft_cap * kLog2e;

  bf16x8 kreg[PPT], vreg[PPT];
  const bf16x8 zero8 = {};
  // global -> registers: piece p of the tile is 16 bytes of sub-tile p / SUB; of the keys it is piece p % SUB of
  // the sub-tile's contiguous blocks, of the values it is keys 8h .. 8h+7 of dimension d (p % SUB = 2 * d + h)
  auto fetch = [&](int tile) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int p = i * 256 + tid;
      const int t = p / SUB, w = p % SUB;
      const int sk0 = tile * kTile + t * 16;
      const bool ok = sk0 < hi_g && sk0 + 16 > lo_g;
      kreg[i] = zero8;
      vreg[i] = zero8;
      if (ok) {
        const int page = table[sk0 / page_size];
        const int off = sk0 % page_size;  // a multiple of 16
        const size_t head = static_cast<size_t>(page) * Kh + kh;
        const int d = w / 2, h = w % 2;
        kreg[i] = *reinterpret_cast<const bf16x8*>(k_pages + head * page_size * HD +
                                                   static_cast<size_t>(off / 16) * (NDC * 512) + w * 8);
        vreg[i] = *reinterpret_cast<const bf16x8*>(v_pages + (head * HD + d) * page_size + off + h * 8);
        if (sk0 + h * 8 + 8 > hi_g) {  // keys at or beyond hi_g may be unwritten: their values count as 0
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (sk0 + h * 8 + e >= hi_g) vreg[i][e] = to_bf16_raw(0.f);
        }
      }
    }
  };
  // registers -> LDS
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int p = i * 256 + tid;
      const int t = p / SUB, w = p % SUB;
      *reinterpret_cast<bf16x8*>(k_s + static_cast<size_t>(p) * 8) = kreg[i];
      const int d = w / 2, h = w % 2;
      const int db = d / 16, dr = d % 16;
      const bf16x4 first = {vreg[i][0], vreg[i][1], vreg[i][2], vreg[i][3]};
      const bf16x4 second = {vreg[i][4], vreg[i][5], vreg[i][6], vreg[i][7]};
      // operand lane (grp', dr) holds keys 4 * grp' .. + 3 of each sub-tile: elements t * 4 .. + 3
      *reinterpret_cast<bf16x4*>(v_s + ((db * 64 + (2 * h) * 16 + dr) * 8 + t * 4)) = first;
      *reinterpret_cast<bf16x4*>(v_s + ((db * 64 + (2 * h + 1) * 16 + dr) * 8 + t * 4)) = second;
    }
  };
  // one tile from LDS, for this wave's rows
  auto compute = [&](int tile) {
    const int key0 = tile * kTile;
    if (rows == 0 || key0 > pos_last || key0 + kTile <= lo_first) return;  // no row of the wave sees a key of it
    floatx4 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dc = 0; dc < NDC; ++dc) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(k_s + ((t * NDC + dc) * 64 + lane) * 8);
        s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[dc], s[t], 0, 0, 0);
      }
    }
    // every row of the wave sees every key of the tile: no mask
    const bool whole = rows == 16 && key0 + kTile - 1 <= pos_first && key0 >= lo_last;
    float y[2][4];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float x = s[t][v] * c1;
        if (soft_cap > 0.f) x = c2 - 2.f * c2 * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x) + 1.f);
        if (!whole) {
          const int key = key0 + t * 16 + grp * 4 + v;
          x = (row_ok && key <= pos_r && key >= lo_r) ? x : -INFINITY;
        }
        y[t][v] = x;
        mx = fmaxf(mx, x);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m_run, mx);
    // a row that has seen no visible key yet keeps m = -inf; 2^(-inf - -inf) must not appear
    const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float e = __builtin_amdgcn_exp2f(y[t][v] - m_use);  // 2^-inf = 0
        psum += e;
        pf[t * 4 + v] = to_bf16_raw(e);
      }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;  // rarely, once the maxima have settled
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      const bf16x8 vf = *reinterpret_cast<const bf16x8*>(v_s + (db * 64 + lane) * 8);
      if (rescale) {
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[db][v] *= alpha;
      }
      acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc[db], 0, 0, 0);
    }
  };

  if (tb < te) {
    fetch(tb);
    stash();
    __syncthreads();
    for (int tile = tb; tile < te; ++tile) {
      const bool more = tile + 1 < te;
      if (more) fetch(tile + 1);
      compute(tile);
      __syncthreads();  // every wave has read the tile
      if (more) stash();
      __syncthreads();
    }
  }

  // acc[db][v] is O^T[d = db * 16 + 4 * grp + v][row r]
  l_run += __shfl_xor(l_run, 16, kWave);
  l_run += __shfl_xor(l_run, 32, kWave);
  if (!row_ok) return;
  if (num_splits == 1) {
    bf16* op = out + static_cast<size_t>(sm.q_start + qi) * out_stride + static_cast<size_t>(kh * G + g) * HD;
    const float inv = 1.f / l_run;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      const bf16x4 o4 = {to_bf16_raw(acc[db][0] * inv), to_bf16_raw(acc[db][1] * inv), to_bf16_raw(acc[db][2] * inv),
                         to_bf16_raw(acc[db][3] * inv)};
      *reinterpret_cast<bf16x4*>(op + db * 16 + 4 * grp) = o4;
    }
  } else {
    // the merge kernel works with natural logarithms
    const size_t row_words = HD + 2;
    const size_t unit = static_cast<size_t>(blockIdx.z * kUnitsPerGroup + wave) * Kh + kh;
    float* wp = workspace + ((unit * num_splits + split) * 16 + r) * row_words;
#pragma unroll
    for (int db = 0; db < NDB; ++db) *reinterpret_cast<floatx4*>(wp + db * 16 + 4 * grp) = acc[db];
    if (grp == 0) {
      wp[HD] = m_run * (1.f / kLog2e);
      wp[HD + 1] = l_run;
    }
  }
}

}  // namespace prefill

bool paged_attention_prefill_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride, const void* q,
                                   int64_t out_stride, const void* out) {
  const int G = H / Kh;
  return (hd == 64 || hd == 128 || hd == 256) && page_size % 16 == 0 && G * max_q_len <= 16 && q_stride % 8 == 0 &&
         (reinterpret_cast<uintptr_t>(q) & 15u) == 0 && out_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 7u) == 0;
}

int paged_attention_prefill(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* units, int unit_begin, int unit_count,
                            void* out, int64_t out_stride, int H, int Kh, int hd, int page_size, int window,
                            float soft_cap, int max_kv_len, int num_splits, void* workspace, size_t workspace_bytes,
                            hipStream_t stream) {
  using prefill::kUnitsPerGroup;
  if (unit_count == 0) return 0;
  const int G = H / Kh;
  const int groups = unit_count / kUnitsPerGroup;
  int span = window > 0 && window < max_kv_len ? window + 16 * kUnitsPerGroup : max_kv_len;  // keys a workgroup reads at most
  if (span < 1) span = 1;
  const int max_tiles = (span + kTile - 1) / kTile + 1;
  int KS = num_splits;
  if (KS <= 0) {
    const int wgs = groups * Kh;
    KS = wgs >= 192 ? 1 : (256 + wgs / 2) / wgs;  // about one workgroup per CU at least
    const int cap_by_work = (max_tiles + 15) / 16;  // at least 16 tiles (512 keys) per workgroup
    if (KS > cap_by_work) KS = cap_by_work;
  }
  if (KS > max_tiles) KS = max_tiles;
  if (KS > kMaxSplits) KS = kMaxSplits;
  if (KS < 1) KS = 1;
  const size_t per_split = static_cast<size_t>(unit_count) * Kh * 16 * (hd + 2) * sizeof(float);
  while (KS > 1 && (workspace == nullptr || per_split * KS > workspace_bytes)) --KS;
  const dim3 grid(KS, Kh, groups);
  const bf16* qp = static_cast<const bf16*>(q);
  const bf16* kp = static_cast<const bf16*>(k_pages);
  const bf16* vp = static_cast<const bf16*>(v_pages);
  const SeqMeta* um = reinterpret_cast<const SeqMeta*>(units);
  bf16* op = static_cast<bf16*>(out);
  float* ws = static_cast<float*>(workspace);
#define SA_LAUNCH(NDC)                                                                                          \
  prefill::paged_attention_prefill_kernel<NDC><<<grid, 256, 0, stream>>>(qp, q_stride, kp, vp, block_table,      \
                                                                         table_stride, um, unit_begin, op,      \
                                                                         out_stride, Kh, G, page_size, window,  \
                                                                         soft_cap, ws)
  if (hd == 64) SA_LAUNCH(2);
  else if (hd == 128) SA_LAUNCH(4);
  else if (hd == 256) SA_LAUNCH(8);
  else {
    set_error("paged_attention_prefill: head size %d is not 64, 128 or 256", hd);
    return 1;
  }
#undef SA_LAUNCH
  if (check_launch("paged_attention_prefill")) return 1;
  if (KS > 1) return attention_merge_ranges(ws, KS, hd, um, unit_begin, unit_count, op, out_stride, Kh, G, stream);
  return 0;
}

}  // namespace sa
