// Paged attention in bfloat16 for requests that bring few query tokens (decode: one token): bound
// by reading each request's keys and values once.
//
// One workgroup of four waves takes one (request, key/value head, range of keys).  All G query
// heads of the key/value head and all of the request's q_len query tokens are the G * q_len <= 16
// columns of one MFMA tile, so keys and values are read once for all of them.  Per tile of 32 keys a
// wave computes
//     S^T[key, row] = K[key, :] . Q[row, :]     v_mfma_f32_16x16x32_bf16, K rows as the A operand,
//                                               loaded straight from the page, where 16 keys x 32
//                                               dimensions are stored as one operand (a contiguous KiB)
//     soft-cap, mask, running maximum and sum per row (float32)
//     O^T[d, row]  += V^T[d, key] . P^T[key, row]
// The second product needs no data movement: S^T comes out of the first MFMA in the register
// layout that the second MFMA wants for its B operand, and value pages are stored transposed
// ([hd, page_size]) so that the A operand is a plain load as well.  The four waves take tiles in
// turn and merge their (maximum, sum, output) through LDS; key ranges are merged by a second, small
// kernel from a workspace, in a fixed order (a merge by the workgroup that finishes last would need a
// device-wide fence, which on this GPU writes back the whole L2).
#include <mutex>

#include "api.h"
#include "attention_common.h"

// Scratch memory of sa_paged_attention_decode_static (below): the partial results of the key ranges.  Every GPU that
// the library runs on holds its own copy, at its own address, until the process ends.
constexpr size_t kStaticScratchBytes = size_t(16) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace sa {

// Sub-tiles of 16 keys whose page a workgroup looks up once, into LDS, before its loop: 32768 keys.
constexpr int kMaxRangeSubTiles = 2048;

__device__ inline float fast_tanh(float x) {
  // tanh(x) = 1 - 2 / (exp(2x) + 1); exact at both ends, relative error ~1e-6 in between
  const float e = __expf(2.f * x);
  return 1.f - 2.f / (e + 1.f);
}

// NDC = head size / 32
template <int NDC>
__global__ __launch_bounds__(256) void paged_attention_decode_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const SeqMeta* __restrict__ seq_meta, int seq_begin,
    bf16* __restrict__ out, int64_t out_stride, int Kh, int G, int page_size, int window, float soft_cap,
    float* __restrict__ workspace) {
  constexpr int HD = NDC * 32;
  constexpr int NDB = HD / 16;  // output blocks of 16 dimensions
  __shared__ __align__(16) float o_s[2][16][HD + 4];   // a wave's output [row][d], while two waves are merged (rows of 16-byte pieces)
  __shared__ float m_s[2][16], l_s[2][16];
  __shared__ int2 where_s[kMaxRangeSubTiles];  // per sub-tile of this workgroup's range: its page, its block within it

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // the same for the whole wave: kept in a scalar register
  const int r = lane % 16, grp = lane / 16;
  const int split = blockIdx.x, num_splits = gridDim.x, kh = blockIdx.y, seq = seq_begin + blockIdx.z;
  const SeqMeta sm = seq_meta[seq];
  const int rows = G * sm.q_len;  // <= 16
  const int* table = block_table + static_cast<size_t>(sm.slot) * table_stride;

  // this lane's row of the tile: query token qi, query head g of the group
  const int qi = r / G, g = r % G;
  const bool row_ok = r < rows;
  const int pos_r = sm.pos0 + qi;
  const int hi = sm.pos0 + sm.q_len;  // keys [lo, hi) are visible to some row
  const int lo = (window > 0 && sm.pos0 - window + 1 > 0) ? sm.pos0 - window + 1 : 0;
  const int lo_r = (window > 0 && pos_r - window + 1 > 0) ? pos_r - window + 1 : 0;

  // tiles of 32 keys aligned to absolute positions; this workgroup's share, then this wave's
  const int tile0 = lo / kTile, tile1 = (hi + kTile - 1) / kTile;
  const int ntiles = tile1 - tile0;
  const int tb = tile0 + static_cast<int>(static_cast<int64_t>(ntiles) * split / num_splits);
  const int te = tile0 + static_cast<int>(static_cast<int64_t>(ntiles) * (split + 1) / num_splits);

  // Where every sub-tile of 16 keys of the range lies is looked up once per pass, into LDS, so that the loop below
  // has no load whose address depends on another load.  (A sub-tile lies within one page: page_size is a multiple
  // of 16.)  The host cuts the keys so that a range fits one pass; a range that is longer all the same (a caller
  // that understates max_kv_len) takes further passes, each with its own look-up, instead of reading beyond the
  // array.
  // (the queries are asked for first: their load is under way during the look-up)
  // Q as B operands: lane (row r, grp) holds Q[row r][dc * 32 + grp * 8 .. + 8]
  bf16x8 qf[NDC];
  {
    const bf16* qp = q + static_cast<size_t>(sm.q_start + (row_ok ? qi : 0)) * q_stride +
                     static_cast<size_t>(kh * G + (row_ok ? g : 0)) * HD + grp * 8;
#pragma unroll
    for (int dc = 0; dc < NDC; ++dc)
      qf[dc] = row_ok ? *reinterpret_cast<const bf16x8*>(qp + dc * 32) : bf16x8{};
  }
  constexpr int kPassTiles = kMaxRangeSubTiles / 2;
  int pass_b = tb;                                        // this pass covers tiles [pass_b, pass_e)
  int pass_e = te - tb > kPassTiles ? tb + kPassTiles : te;
  int sub0 = 2 * pass_b;
  auto look_up = [&]() {
    // (at least the first entry is written, also for a range without tiles: loads that are not needed go there)
    const int nsub = pass_e > pass_b ? 2 * (pass_e - pass_b) : 1;
    for (int i = tid; i < nsub; i += 256) {
      const int key = (sub0 + i) * 16;
      int2 w = {0, 0};
      if (key < hi && key + 16 > lo) {
        const int block = key / page_size;
        w.x = table[block];
        w.y = (key - block * page_size) / 16;
      }
      where_s[i] = w;
    }
    __syncthreads();
  };
  look_up();

  floatx4 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) acc[db] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;  // per row (lane % 16); l_run is this lane group's share

  // The loop is software-pipelined over two sets of registers (A and B), each holding the keys and the values of
  // one tile: while a tile is computed from one set, the loads of the next tile are in flight into the other, and
  // each half of a set (keys, values) is requested again for the tile after next as soon as it has been used.  A
  // wave thus keeps about 48 KiB of loads in flight; with one workgroup per CU that is what hides the latency.
  struct SubTile {
    bool ok;            // some key of the sub-tile is in [lo, hi): its page exists
    const bf16* k;      // this lane's 16 bytes of the sub-tile's first key block
    const bf16* v;      // this lane's value row (dimension r of block 0), at its 4 keys
  };
  auto locate = [&](int tile, int t) {
    SubTile st;
    const int sk0 = tile * kTile + t * 16;
    st.ok = tile < pass_e && sk0 < hi && sk0 + 16 > lo;  // wave-uniform
    // A sub-tile outside the range is loaded all the same, from where this pass's first sub-tile lies: every load of
    // the loop is unconditional, the loop straight-line code, and the compiler counts the loads in flight (with a
    // branch around a load it waits for all of them, and loads and products do not overlap).  What is loaded there
    // is never used: its scores are masked and its values replaced by zeros.  (Not from one place for everybody,
    // such as the pool's first page: with a tile or two to a wave, as for a single request, every wave of the GPU
    // has such loads, and a thousand waves on the same sixteen KiB queue up at its few channels of L2; a
    // workgroup's own first sub-tile is in its CU's cache.)
    const int2 w = where_s[st.ok ? 2 * tile + t - sub0 : 0];
    const size_t head = static_cast<size_t>(w.x) * Kh + kh;
    const int blk = w.y;
    // keys are stored in 16-key x 32-dimension blocks of operand order: block (blk, dc) is a contiguous KiB
    st.k = k_pages + head * page_size * HD + static_cast<size_t>(blk) * (NDC * 512) + lane * 8;
    st.v = v_pages + (head * HD + r) * page_size + blk * 16 + grp * 4;
    return st;
  };
  struct TileRegs {
    SubTile st[2];
    bf16x8 kf[2][NDC];
    bf16x4 vf[2][NDB];
  };
  auto request_keys = [&](TileRegs& b, int tile) {
    b.st[0] = locate(tile, 0);
    b.st[1] = locate(tile, 1);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int dc = 0; dc < NDC; ++dc)
        b.kf[t][dc] = *reinterpret_cast<const bf16x8*>(b.st[t].k + dc * 512);
  };
  auto request_values = [&](TileRegs& b) {  // of the tile whose keys were requested last
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int db = 0; db < NDB; ++db)
        b.vf[t][db] = *reinterpret_cast<const bf16x4*>(b.st[t].v + static_cast<size_t>(db) * 16 * page_size);
  };
  // One tile from the registers of `b`; its keys, then its values, are requested anew for tile `next`.
  auto process = [&](TileRegs& b, int tile, int next) {
    const int key0 = tile * kTile;
    const bool sub_ok[2] = {b.st[0].ok, b.st[1].ok};
    // ---- scores of the two sub-tiles of 16 keys
    floatx4 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dc = 0; dc < NDC; ++dc) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.kf[t][dc], qf[dc], s[t], 0, 0, 0);
    }
    // the values of this tile are still needed: only the key half of the set is requested now
    bf16x4 vcur[2][NDB];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int db = 0; db < NDB; ++db) vcur[t][db] = b.vf[t][db];
    request_keys(b, next);
    // ---- cap, mask, online softmax.  Lane (row r, grp) holds keys sk0 + 4 * grp + v of each sub-tile.
    float p[2][4];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int key = key0 + t * 16 + grp * 4 + v;
        float x = s[t][v];
        if (soft_cap > 0.f) x = soft_cap * fast_tanh(x / soft_cap);
        const bool vis = sub_ok[t] && row_ok && key <= pos_r && key >= lo_r;
        x = vis ? x : -INFINITY;
        p[t][v] = x;
        mx = fmaxf(mx, x);
      }
    mx = max_over_row_lanes(mx);
    const float m_new = fmaxf(m_run, mx);
    // a row that has seen no visible key yet keeps m = -inf; exp(-inf - -inf) must not appear
    const float alpha = m_new == -INFINITY ? 1.f : __expf(m_run - m_new);
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float e = p[t][v] == -INFINITY ? 0.f : __expf(p[t][v] - m_new);
        psum += e;
        pf[t * 4 + v] = to_bf16_raw(e);
      }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    // ---- output: O^T[d][row] = alpha * O^T + V^T[d][keys] . P^T[keys][row]
    // lane (d = r, grp) of the A operand holds V^T[db * 16 + r][the same 8 keys as pf]
    const bool tail = key0 + kTile > hi;  // keys at or beyond hi may be unwritten: their values count as 0
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      bf16x8 a;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) a[t * 4 + v] = vcur[t][db][v];
      if (tail || !sub_ok[0] || !sub_ok[1]) {  // (wave-uniform, and rare: the range's first and last tile)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int key = key0 + (e / 4) * 16 + grp * 4 + (e % 4);
          if (key >= hi || !sub_ok[e / 4]) a[e] = to_bf16_raw(0.f);
        }
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[db][v] *= alpha;
      acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pf, acc[db], 0, 0, 0);
    }
    request_values(b);
  };

  TileRegs A, B;
  for (;;) {
    int tile = pass_b + wave;
    request_keys(A, tile);
    request_values(A);
    request_keys(B, tile + 4);
    request_values(B);
    for (; tile < pass_e; tile += 8) {
      process(A, tile, tile + 8);
      if (tile + 4 < pass_e) process(B, tile + 4, tile + 12);
    }
    if (pass_e >= te) break;  // (the usual case: one pass)
    __syncthreads();          // every wave has done with this pass's look-ups
    pass_b = pass_e;
    pass_e = te - pass_b > kPassTiles ? pass_b + kPassTiles : te;
    sub0 = 2 * pass_b;
    look_up();
  }

  // ---- merge the four waves in two rounds through LDS (waves 2, 3 into 0, 1; then 1 into 0).
  // acc[db][v] is O^T[d = db * 16 + 4 * grp + v][row r].
  l_run = sum_over_row_lanes(l_run);
  // (acc[db] is four consecutive dimensions: one 16-byte piece of LDS; rows beyond the request's hold nothing)
  auto put = [&](int slot) {
    if (row_ok) {
#pragma unroll
      for (int db = 0; db < NDB; ++db) *reinterpret_cast<floatx4*>(&o_s[slot][r][db * 16 + 4 * grp]) = acc[db];
      if (grp == 0) {
        m_s[slot][r] = m_run;
        l_s[slot][r] = l_run;
      }
    }
  };
  auto take = [&](int slot) {
    if (!row_ok) return;
    const float m_o = m_s[slot][r], l_o = l_s[slot][r];
    const float M = fmaxf(m_run, m_o);
    const float a = m_run == -INFINITY ? 0.f : __expf(m_run - M);
    const float b = m_o == -INFINITY ? 0.f : __expf(m_o - M);
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      const floatx4 o = *reinterpret_cast<const floatx4*>(&o_s[slot][r][db * 16 + 4 * grp]);
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[db][v] = acc[db][v] * a + o[v] * b;
    }
    l_run = l_run * a + l_o * b;
    m_run = M;
  };
  if (wave >= 2) put(wave - 2);
  __syncthreads();
  if (wave < 2) take(wave);
  __syncthreads();
  if (wave == 1) put(0);
  __syncthreads();
  if (wave == 0) take(0);

  const int KS = num_splits;
  const size_t row_words = HD + kRowExtra;  // output, maximum, sum
  const size_t unit = (static_cast<size_t>(blockIdx.z) * Kh + kh);
  if (wave == 0 && row_ok) {
    if (KS == 1) {
      bf16* op = out + static_cast<size_t>(sm.q_start + qi) * out_stride + static_cast<size_t>(kh * G + g) * HD;
      const float inv = 1.f / l_run;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int v = 0; v < 4; ++v) op[db * 16 + 4 * grp + v] = float_to_bf16(acc[db][v] * inv);
    } else {
      float* wp = workspace + ((unit * KS + split) * 16 + r) * row_words;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int v = 0; v < 4; ++v) wp[db * 16 + 4 * grp + v] = acc[db][v];
      if (grp == 0) {
        wp[HD] = m_run;
        wp[HD + 1] = l_run;
      }
    }
  }
}

// Adds up the key ranges of each (request, head, row), in their order: one workgroup per row, one thread per
// output dimension; the ranges' weights exp(m_y - max) are computed once into LDS.
__global__ __launch_bounds__(256) void paged_attention_merge_kernel(const float* __restrict__ workspace, int KS, int HD,
                                                                    const SeqMeta* __restrict__ seq_meta, int seq_begin,
                                                                    bf16* __restrict__ out, int64_t out_stride, int Kh,
                                                                    int G, int chunk_tiles, int group, int window) {
  __shared__ float w_s[kMaxSplits];
  __shared__ float scratch[16];
  __shared__ float4 part_s[256];
  const int tid = threadIdx.x, kh = blockIdx.x, z = blockIdx.y, orow = blockIdx.z;
  const SeqMeta sm = seq_meta[seq_begin + z];
  if (orow >= G * sm.q_len) return;
  const size_t row_words = HD + kRowExtra;
  const size_t unit = static_cast<size_t>(z) * Kh + kh;
  const float* base = workspace + (unit * KS * 16 + orow) * row_words;
  const size_t stride = 16 * row_words;
  if (chunk_tiles > 0) {  // the ranges that this unit's group has; one: it has written its output itself
    int lo, hi, slot;
    group_keys(seq_meta, seq_begin + z / group * group, group, window, &lo, &hi, &slot);
    KS = key_chunks(lo, hi, chunk_tiles);
    if (KS <= 1) return;
  }
  const float my = tid < KS ? base[tid * stride + HD] : -INFINITY;
  const float ly = tid < KS ? base[tid * stride + HD + 1] : 0.f;
  // The threads are `parts` groups of HD / 4: group p adds up ranges p, p + parts, ... for four dimensions per
  // thread, then group 0 adds the groups up in order.  The first kAhead ranges of a thread are asked for here,
  // before the weights are known: their loads are under way together with those of the maxima and sums above, so
  // the kernel waits for memory once, not twice.
  constexpr int kAhead = 16;
  const int quarter = HD / 4, parts = 256 / quarter;
  const int c = tid % quarter, part = tid / quarter;
  float4 ahead[kAhead];
#pragma unroll
  for (int i = 0; i < kAhead; ++i) {
    const int y = part + i * parts;
    ahead[i] = (part < parts && y < KS) ? *reinterpret_cast<const float4*>(base + y * stride + 4 * c)
                                        : float4{0.f, 0.f, 0.f, 0.f};
  }
  // maximum over the ranges
  float mx = wave_max(my);
  if (tid % kWave == 0) scratch[tid / kWave] = mx;
  __syncthreads();
  const float Mg = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
  const float wy = my == -INFINITY ? 0.f : __expf(my - Mg);
  if (tid < KS) w_s[tid] = wy;
  const float Lg = block_sum(ly * wy, scratch + 4);  // has its own barriers; w_s is complete after them
  float4 o = {0.f, 0.f, 0.f, 0.f};
  if (part < parts) {
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      const int y = part + i * parts;
      const float w = y < KS ? w_s[y] : 0.f;
      o.x += ahead[i].x * w;
      o.y += ahead[i].y * w;
      o.z += ahead[i].z * w;
      o.w += ahead[i].w * w;
    }
    for (int y = part + kAhead * parts; y < KS; y += parts) {
      const float4 v = *reinterpret_cast<const float4*>(base + y * stride + 4 * c);
      const float w = w_s[y];
      o.x += v.x * w;
      o.y += v.y * w;
      o.z += v.z * w;
      o.w += v.w * w;
    }
    part_s[tid] = o;
  }
  __syncthreads();
  if (part != 0) return;
  for (int p = 1; p < parts; ++p) {
    const float4 v = part_s[p * quarter + c];
    o.x += v.x;
    o.y += v.y;
    o.z += v.z;
    o.w += v.w;
  }
  const int oq = orow / G, og = orow % G;
  bf16* op = out + static_cast<size_t>(sm.q_start + oq) * out_stride + static_cast<size_t>(kh * G + og) * HD;
  const float inv = 1.f / Lg;
  op[4 * c] = float_to_bf16(o.x * inv);
  op[4 * c + 1] = float_to_bf16(o.y * inv);
  op[4 * c + 2] = float_to_bf16(o.z * inv);
  op[4 * c + 3] = float_to_bf16(o.w * inv);
}

bool paged_attention_decode_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride, const void* q) {
  const int G = H / Kh;
  return (hd == 64 || hd == 128 || hd == 256) && page_size % 16 == 0 && G * max_q_len <= 16 && q_stride % 8 == 0 &&
         (reinterpret_cast<uintptr_t>(q) & 15u) == 0;
}

// Tiles of kTile keys that a request reads at most.
static int decode_max_tiles(int window, int max_kv_len) {
  int span = window > 0 && window < max_kv_len ? window + 16 : max_kv_len;
  if (span < 1) span = 1;
  return (span + kTile - 1) / kTile + 1;
}

// Into how many ranges the keys of each request are cut (num_splits > 0 asks for that many).
int paged_attention_decode_ranges(int seq_count, int Kh, int window, int max_kv_len, int num_splits) {
  const int units = seq_count * Kh;
  const int max_tiles = decode_max_tiles(window, max_kv_len);
  int KS = num_splits;
  if (KS <= 0) {
    // One workgroup per CU at most, and as many as that allows: longer ranges amortise the set-up, and a few
    // workgroups beyond the CUs would run as a round of their own (6 requests of 8,192 keys at the 2B shape: 42 us
    // with 240 workgroups, 58 with 264; 24 requests: 144 with 192, 188 with 288).
    KS = 256 / units;
    const int cap_by_work = (max_tiles + 1) / 2;  // at least 2 tiles (64 keys) per workgroup
    if (KS > cap_by_work) KS = cap_by_work;
    // ... and no more than 64 ranges, or ranges of 16 tiles: a thread of the second kernel has 16 ranges' partial
    // results on their way at once (one request of 8,192 keys at the 2B shape: 18.5 us with 64 ranges, 19.4 with 32)
    const int cap_by_merge = max_tiles / 16 > 64 ? max_tiles / 16 : 64;
    if (KS > cap_by_merge) KS = cap_by_merge;
  }
  // (a workgroup looks up the pages of at most kMaxRangeSubTiles sub-tiles: two more than its share of the tiles has)
  const int least = (2 * max_tiles + kMaxRangeSubTiles - 3) / (kMaxRangeSubTiles - 2);
  if (KS < least) KS = least;
  if (KS > max_tiles) KS = max_tiles;
  if (KS > kMaxSplits) KS = kMaxSplits;
  if (KS < 1) KS = 1;
  return KS;
}

int paged_attention_decode(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                           const int* block_table, int table_stride, const int* seq_meta, int seq_begin, int seq_count,
                           void* out, int64_t out_stride, int H, int Kh, int hd, int page_size, int window,
                           float soft_cap, int max_kv_len, int max_q_len, int num_splits, void* workspace, size_t workspace_bytes,
                           hipStream_t stream) {
  if (seq_count == 0) return 0;
  const int G = H / Kh;
  const int units = seq_count * Kh;
  int KS = paged_attention_decode_ranges(seq_count, Kh, window, max_kv_len, num_splits);
  const size_t per_split = static_cast<size_t>(units) * 16 * (hd + kRowExtra) * sizeof(float);
  while (KS > 1 && (workspace == nullptr || per_split * KS > workspace_bytes)) --KS;
  // (ranges of more than kMaxRangeSubTiles sub-tiles, which a small workspace or a caller's own num_splits may
  // leave, take several passes inside the kernel)
  const dim3 grid(KS, Kh, seq_count);
  const bf16* qp = static_cast<const bf16*>(q);
  const bf16* kp = static_cast<const bf16*>(k_pages);
  const bf16* vp = static_cast<const bf16*>(v_pages);
  const SeqMeta* sm = reinterpret_cast<const SeqMeta*>(seq_meta);
  bf16* op = static_cast<bf16*>(out);
  float* ws = static_cast<float*>(workspace);
#define SA_LAUNCH(NDC)                                                                                              \
  paged_attention_decode_kernel<NDC><<<grid, 256, 0, stream>>>(qp, q_stride, kp, vp, block_table, table_stride, sm, \
                                                               seq_begin, op, out_stride, Kh, G, page_size, window,  \
                                                               soft_cap, ws)
  if (hd == 64) SA_LAUNCH(2);
  else if (hd == 128) SA_LAUNCH(4);
  else if (hd == 256) SA_LAUNCH(8);
  else {
    set_error("paged_attention_decode: head size %d is not 64, 128 or 256", hd);
    return 1;
  }
#undef SA_LAUNCH
  if (check_launch("paged_attention_decode")) return 1;
  if (KS > 1) return attention_merge_ranges(ws, KS, hd, sm, seq_begin, seq_count, max_q_len, op, out_stride, Kh, G, stream);
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// The same attention with the partial results of the key ranges in memory that the library owns: for callers that
// cannot allocate.  `scratch` is a host-side stand-in for a device array; its device address on each GPU is asked
// for once per device (hipGetSymbolAddress) and only that address is ever handed to kernels.
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// The address of `scratch` on the current device (asked for at the first call on that device), or null after
// set_error().
static void* static_scratch() {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
    set_error("paged_attention_decode_static: no current device (%s, device %d, at most %d devices)",
              hipGetErrorString(e), device, kMaxDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(::scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("paged_attention_decode_static: the address of the scratch array on device %d is not known: %s",
                device, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[device] = ptr;
  }
  return g_scratch_ptr[device];
}

int paged_attention_decode_static(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                  const int* block_table, int table_stride, const int* seq_meta, int seq_begin,
                                  int seq_count, void* out, int64_t out_stride, int H, int Kh, int hd, int page_size,
                                  int window, float soft_cap, int max_kv_len, int max_q_len, int num_splits,
                                  hipStream_t stream) {
  if (seq_count == 0) return 0;
  // the ranges that the entry point with a workspace chooses when it has room for all of them; here they must fit
  const int KS = paged_attention_decode_ranges(seq_count, Kh, window, max_kv_len, num_splits);
  const size_t need = KS > 1 ? static_cast<size_t>(seq_count) * Kh * KS * 16 * (hd + kRowExtra) * sizeof(float) : 0;
  if (need > kStaticScratchBytes) {
    set_error("paged_attention_decode_static: %d requests x %d key heads x %d key ranges of head size %d need %zu bytes "
              "of partial results, the library's own scratch memory holds %zu: fewer requests at a time, or fewer "
              "ranges (num_splits)", seq_count, Kh, KS, hd, need, kStaticScratchBytes);
    return 1;
  }
  void* ptr = static_scratch();
  if (ptr == nullptr) return 1;
  return paged_attention_decode(q, q_stride, k_pages, v_pages, block_table, table_stride, seq_meta, seq_begin, seq_count,
                                out, out_stride, H, Kh, hd, page_size, window, soft_cap, max_kv_len, max_q_len, KS, ptr,
                                kStaticScratchBytes, stream);
}

// The same for units with many rows (portions of prompts): one workgroup per (unit, head) takes all 16 rows, 16
// threads per row, each with its share of the output dimensions in pieces of four.
__global__ __launch_bounds__(256) void paged_attention_merge_rows_kernel(const float* __restrict__ workspace, int KS,
                                                                         int HD, const SeqMeta* __restrict__ seq_meta,
                                                                         int seq_begin, bf16* __restrict__ out,
                                                                         int64_t out_stride, int Kh, int G,
                                                                         int chunk_tiles, int group, int window) {
  const int tid = threadIdx.x, kh = blockIdx.x, z = blockIdx.y;
  const SeqMeta sm = seq_meta[seq_begin + z];
  const int orow = tid / 16, part = tid % 16;
  if (orow >= G * sm.q_len) return;
  const size_t row_words = HD + kRowExtra;
  const size_t unit = static_cast<size_t>(z) * Kh + kh;
  const float* base = workspace + (unit * KS * 16 + orow) * row_words;
  const size_t stride = 16 * row_words;
  if (chunk_tiles > 0) {  // the ranges that this unit's group has; one: it has written its output itself
    int lo, hi, slot;
    group_keys(seq_meta, seq_begin + z / group * group, group, window, &lo, &hi, &slot);
    KS = key_chunks(lo, hi, chunk_tiles);
    if (KS <= 1) return;
  }
  float Mg = -INFINITY;
  for (int y = 0; y < KS; ++y) Mg = fmaxf(Mg, base[y * stride + HD]);
  float Lg = 0.f;
  for (int y = 0; y < KS; ++y) {
    const float my = base[y * stride + HD];
    Lg += my == -INFINITY ? 0.f : base[y * stride + HD + 1] * __expf(my - Mg);
  }
  const float inv = 1.f / Lg;
  const int oq = orow / G, og = orow % G;
  bf16* op = out + static_cast<size_t>(sm.q_start + oq) * out_stride + static_cast<size_t>(kh * G + og) * HD;
  for (int d = part * 4; d < HD; d += 64) {
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    for (int y = 0; y < KS; ++y) {
      const float my = base[y * stride + HD];
      const float wy = my == -INFINITY ? 0.f : __expf(my - Mg);
      const float4 v = *reinterpret_cast<const float4*>(base + y * stride + d);
      o[0] += v.x * wy;
      o[1] += v.y * wy;
      o[2] += v.z * wy;
      o[3] += v.w * wy;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) op[d + e] = float_to_bf16(o[e] * inv);
  }
}

int attention_merge_ranges(const float* workspace, int num_ranges, int hd, const SeqMeta* units, int unit_begin,
                           int unit_count, int max_q_len, bf16* out, int64_t out_stride, int Kh, int G,
                           hipStream_t stream, int chunk_tiles, int group, int window) {
  const int max_rows = G * max_q_len < 16 ? G * max_q_len : 16;
  if (max_rows > 4 && num_ranges <= 64) {
    paged_attention_merge_rows_kernel<<<dim3(Kh, unit_count), 256, 0, stream>>>(
        workspace, num_ranges, hd, units, unit_begin, out, out_stride, Kh, G, chunk_tiles, group, window);
    return check_launch("paged_attention_merge_rows");
  }
  // one workgroup per row: rows beyond the longest unit's are not launched
  paged_attention_merge_kernel<<<dim3(Kh, unit_count, max_rows), 256, 0, stream>>>(
      workspace, num_ranges, hd, units, unit_begin, out, out_stride, Kh, G, chunk_tiles, group, window);
  return check_launch("paged_attention_merge");
}

}  // namespace sa

extern "C" int sa_paged_attention_decode_static_bytes() { return static_cast<int>(kStaticScratchBytes); }

extern "C" int sa_paged_attention_decode_static(const void* q, int64_t q_stride, const void* k_pages,
                                                const void* v_pages, const int* block_table, int table_stride,
                                                const int* seq_meta, int seq_begin, int seq_count, void* out,
                                                int64_t out_stride, int H, int Kh, int hd, int page_size, int window,
                                                float soft_cap, int max_kv_len, int max_q_len, int num_splits,
                                                hipStream_t stream) {
  using namespace sa;
  if (seq_count == 0) return 0;
  SA_REQUIRE(seq_count > 0 && seq_begin >= 0 && H > 0 && Kh > 0 && H % Kh == 0,
             "paged_attention_decode_static: bad counts");
  SA_REQUIRE(window >= 0 && table_stride > 0 && max_kv_len > 0,
             "paged_attention_decode_static: bad window, table or length");
  SA_REQUIRE(num_splits <= kMaxSplits, "paged_attention_decode_static: at most %d key ranges", kMaxSplits);
  SA_REQUIRE(paged_attention_decode_takes(H, Kh, hd, page_size, max_q_len, q_stride, q),
             "paged_attention_decode_static takes head size 64, 128 or 256, a page size that is a multiple of 16 and "
             "(heads per key head) * tokens <= 16; got hd=%d P=%d G=%d tokens=%d", hd, page_size, H / Kh, max_q_len);
  SA_REQUIRE(out_stride >= static_cast<int64_t>(H) * hd, "paged_attention_decode_static: output rows are too short");
  return paged_attention_decode_static(q, q_stride, k_pages, v_pages, block_table, table_stride, seq_meta, seq_begin,
                                       seq_count, out, out_stride, H, Kh, hd, page_size, window, soft_cap, max_kv_len,
                                       max_q_len, num_splits, stream);
}
