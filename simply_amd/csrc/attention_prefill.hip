// Paged attention in bfloat16 for portions of prompts: many query tokens of one request over the keys that the
// request has so far.  Bound by the matrix cores and the softmax arithmetic, no longer by reading the keys: a
// workgroup of four waves takes 4 * R consecutive units of up to 16 query rows each (rows = tokens x query heads of
// one key/value head; the host cuts a request's tokens into such units) and one key/value head, and walks over
// the keys once for all of its rows.
//
// Keys and values go from the pages straight into LDS (global_load_lds: no staging registers), into two buffers
// of one 32-key tile each, so that the loads of the next tile are in flight while one tile is computed (they are
// asked for one by one among the tile's first products; a third buffer, loads two tiles ahead, was slower); two
// workgroups fit on a compute unit and fill each other's waits.  Both lie in LDS as they lie in their pages: keys in 16-key x 32-dimension blocks of MFMA operand
// order, values per 16-key sub-tile as blocks of 16 dimensions, [keys 0..7 | keys 8..15][dimension][8 keys].  Every wave reads every block of a tile and computes,
// for its own rows,
//     S^T = K . Q^T            keys as the A operand, one 16-byte LDS read per lane and block
//     soft-cap, mask and online softmax in float32 (base-2 exponentials, log2(e) folded into the constants)
//     O^T += V^T . P^T         S^T comes out of the first product in the layout that the second wants for P^T;
//                              the value operand is two 8-byte LDS reads per lane, one from each sub-tile
// exactly as the few-rows kernel does from global memory.  A wave with R units keeps R tiles of rows and uses each
// operand it reads for all of them.  A wave skips tiles that none of its rows can see and the mask arithmetic on
// tiles that all of its rows see whole.
//
// The two buffers are kept in step by one workgroup barrier per tile.  The barrier is the bare instruction, with the
// count of outstanding loads given by hand: the usual barrier with its fence would wait for all loads in flight,
// which is the pipeline.  The loads are written as instructions that the compiler does not know of (load_to_lds below).
//
// When few workgroups would result (a short portion over a long context), the keys are also cut into ranges over
// workgroups, and the ranges are merged by the second kernel of the few-rows path.
#include "api.h"
#include "attention_common.h"

namespace sa {
namespace prefill {

constexpr int kWaves = 4;
constexpr float kLog2e = 1.4426950408889634f;

// s_waitcnt for "at most n vector-memory loads outstanding" and nothing else (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4, lgkmcnt 11:8)
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// The workgroup barrier alone; the empty statements keep the compiler from moving memory accesses across it.
__device__ inline void bare_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
}

// 16 bytes per lane from global memory (an address per lane) into LDS at byte address lds + 16 * lane (lds is the
// same for the whole wave).  Written as an instruction: the compiler counts a load into LDS that it knows of as a
// pending LDS access for as long as the load is under way, and then makes every wait for an operand read a wait for
// all of them.  It does not know of these loads: the kernel waits for them itself (vmcnt) before the barrier that
// precedes the first read of what they bring.
__device__ __forceinline__ void load_to_lds(const bf16* src, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds) : "memory");
}

template <int NDC, int R, bool CAP>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(R == 1 ? 2 : 1, R == 1 ? 2 : 1))) void paged_attention_prefill_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const SeqMeta* __restrict__ units, int unit_begin,
    bf16* __restrict__ out, int64_t out_stride, int Kh, int G, int page_size, int window, float soft_cap,
    float* __restrict__ workspace, int chunk_tiles) {
  constexpr int HD = NDC * 32;
  constexpr int NDB = HD / 16;            // output blocks of 16 dimensions
  constexpr int CPW = NDC / 2;            // KiB chunks of keys (and of values) per wave and tile
  constexpr int HALF = NDC * 1024;        // elements of a tile's keys (and of its values) in a buffer: 2 * NDC KiB
  constexpr int GROUP = kWaves * R;       // units per workgroup
  static_assert(NDC % 2 == 0, "head size must be a multiple of 64");
  // [keys: sub-tile, dc, lane, 8][values: sub-tile, d, 16]
  __shared__ __attribute__((aligned(16))) __bf16 stage0[2 * HALF];
  __shared__ __attribute__((aligned(16))) __bf16 stage1[2 * HALF];
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) __bf16*)stage0));
  const uint32_t lds1 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) __bf16*)stage1));

  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int r = lane % 16, grp = lane / 16;
  const int split = blockIdx.y, num_splits = gridDim.y, kh = blockIdx.x;
  // later units of a prompt see more keys: they are started first
  const int group = gridDim.z - 1 - blockIdx.z;
  const int u0 = unit_begin + group * GROUP;

  // the keys that some row of the workgroup sees, in ranges of chunk_tiles tiles: this workgroup takes range `split`
  int lo_g, hi_g, slot = 0;
  if (!group_keys(units, u0, GROUP, window, &lo_g, &hi_g, &slot)) return;  // no rows at all
  const int tile0 = lo_g / kTile, tile1 = (hi_g + kTile - 1) / kTile;
  const int num_chunks = key_chunks(lo_g, hi_g, chunk_tiles);
  if (split >= num_chunks) return;  // (the same for the whole workgroup)
  const int* table = block_table + static_cast<size_t>(__builtin_amdgcn_readfirstlane(slot)) * table_stride;
  const int tb = tile0 + split * chunk_tiles;
  const int te = tb + chunk_tiles < tile1 ? tb + chunk_tiles : tile1;

  // this wave's R units and this lane's row of each: query token qi, query head g of the group
  const int qi = r / G, g = r % G;
  int rows[R], pos_r[R], lo_r[R], pos_first[R], pos_last[R], lo_first[R], lo_last[R], q_row[R];
  bool row_ok[R];
  bf16x8 qf[R][NDC];  // Q as B operands: lane (row r, grp) holds Q[row r][dc * 32 + grp * 8 .. + 8]
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const SeqMeta sm = units[u0 + wave * R + j];
    rows[j] = G * sm.q_len;  // <= 16
    row_ok[j] = r < rows[j];
    pos_r[j] = sm.pos0 + qi;
    lo_r[j] = (window > 0 && pos_r[j] - window + 1 > 0) ? pos_r[j] - window + 1 : 0;
    // over the unit's rows: positions [pos_first, pos_last], lower bounds [lo_first, lo_last]
    pos_first[j] = sm.pos0;
    pos_last[j] = sm.pos0 + sm.q_len - 1;
    lo_first[j] = (window > 0 && pos_first[j] - window + 1 > 0) ? pos_first[j] - window + 1 : 0;
    lo_last[j] = (window > 0 && pos_last[j] - window + 1 > 0) ? pos_last[j] - window + 1 : 0;
    q_row[j] = sm.q_start + qi;
    const bf16* qp = q + static_cast<size_t>(row_ok[j] ? q_row[j] : sm.q_start) * q_stride +
                     static_cast<size_t>(kh * G + (row_ok[j] ? g : 0)) * HD + grp * 8;
#pragma unroll
    for (int dc = 0; dc < NDC; ++dc)
      qf[j][dc] = (row_ok[j] && tb < te) ? *reinterpret_cast<const bf16x8*>(qp + dc * 32) : bf16x8{};
  }

  floatx4 acc[R][NDB];
  float m_run[R], l_run[R];  // per row, in units of log2; l_run is this lane group's share
#pragma unroll
  for (int j = 0; j < R; ++j) {
#pragma unroll
    for (int db = 0; db < NDB; ++db) acc[j][db] = floatx4{0.f, 0.f, 0.f, 0.f};
    m_run[j] = -INFINITY;
    l_run[j] = 0.f;
  }

  // scores in base-2 units: y = log2(e) * cap * tanh(s / cap) = c2 - 2 * c2 / (2^(s * c1) + 1), or log2(e) * s
  const float c1 = CAP ? 2.f * kLog2e / soft_cap : kLog2e;
  const float c2 = soft_cap * kLog2e;

  // How a tile of 32 keys lies in LDS.  The two score products of a tile do not take keys 0..15 and 16..31 but
  //     product t, row i of its A operand  <->  key 8 * (i / 4) + 4 * t + i % 4   of the tile,
  // so that a lane's eight scores (rows 4 * grp + v of both products) belong to the eight consecutive keys 8 * grp ..
  // 8 * grp + 7: the value operand of the second product is then one 16-byte piece of a value page per lane.  Both
  // operands lie in LDS in blocks of 64 lanes x 16 bytes in the order of the lanes that read them (no bank
  // conflicts); it is the load into LDS that picks, lane by lane, the matching 16 bytes of the pages:
  //   key block (t, dc), lane (kgrp, i):    sub-tile i / 8 of the tile, its key 8 * ((i / 4) % 2) + 4 * t + i % 4,
  //                                         dimensions 32 * dc + 8 * kgrp .. + 7
  //   value block db, lane (grp, r):        sub-tile grp / 2, keys 8 * (grp % 2) .. + 7 of dimension 16 * db + r
  // A wave loads blocks c = wave + 4 * i of the keys' 2 * NDC blocks and of the values' 2 * NDC blocks.
  uint32_t k_off[CPW], v_off[CPW], lds_off[CPW];  // in elements; what depends on the lane is computed once
  const int k_sub = (lane % 16) / 8, v_sub = lane / 32;  // the sub-tile (page) that this lane's pieces come from
#pragma unroll
  for (int i = 0; i < CPW; ++i) {
    const int c = wave + kWaves * i;
    const int t = c / NDC, dc = c % NDC, row = lane % 16;
    k_off[i] = dc * 512 + ((lane / 16) * 16 + 8 * ((row / 4) % 2) + 4 * t + row % 4) * 8;
    v_off[i] = (c * 16 + lane % 16) * page_size + ((lane / 16) % 2) * 8;
    lds_off[i] = __builtin_amdgcn_readfirstlane(c * 512);
  }
  // Where the two sub-tiles lie of the tile whose pages are looked up next: block blk[n] of the table, key off[n] of
  // its page; kept by stepping, without divisions.  All of it is the same for the whole wave: scalar registers.
  int blk[2], off[2];
#pragma unroll
  for (int n = 0; n < 2; ++n) {
    const int sk0 = tb * kTile + n * 16;
    blk[n] = __builtin_amdgcn_readfirstlane(sk0 / page_size);
    off[n] = __builtin_amdgcn_readfirstlane(sk0 % page_size);
  }
  const uint32_t page_stride = static_cast<uint32_t>(Kh) * page_size * HD;  // elements of a page, keys or values
  const bf16* const k_head = k_pages + static_cast<int64_t>(kh) * page_size * HD;
  const bf16* const v_head = v_pages + static_cast<int64_t>(kh) * page_size * HD;
  // sub-tiles (of 16 keys) with a page that this workgroup may read: [sub_lo, sub_hi)
  const int sub_lo = lo_g / 16, sub_hi = min((hi_g + 15) / 16, te * 2);
  // The loads of a tile are prepared in steps, so that no step waits for the one before it: the pages of its two
  // sub-tiles are looked up two tiles ahead (`look_up`, called for consecutive tiles: a sub-tile without a page,
  // beyond the keys or given back by a windowed layer, reads page 0, and its values are dropped when they are
  // used), this lane's addresses follow one tile ahead (`locate`), and the loads themselves are asked for one by
  // one among the products of the tile before (`ask`).
  struct Pages {
    uint32_t page[2], at[2];
  };
  auto look_up = [&](int tile) __attribute__((always_inline)) {
    Pages p;
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int sub = tile * 2 + n;
      p.page[n] = (sub >= sub_lo && sub < sub_hi) ? static_cast<uint32_t>(table[blk[n]]) : 0u;
      p.at[n] = static_cast<uint32_t>(off[n]);
      off[n] += kTile;
#pragma unroll
      for (int twice = 0; twice < 2; ++twice)
        if (off[n] >= page_size) {
          off[n] -= page_size;
          ++blk[n];
        }
    }
    return p;
  };
  const bf16* k_from;
  const bf16* v_from;
  auto locate = [&](const Pages& p) __attribute__((always_inline)) {
    const uint32_t page = k_sub ? p.page[1] : p.page[0], at_k = k_sub ? p.at[1] : p.at[0];
    k_from = k_head + static_cast<uint64_t>(page) * page_stride + (at_k >> 4) * (NDC * 512);
    const uint32_t page_v = v_sub ? p.page[1] : p.page[0], at_v = v_sub ? p.at[1] : p.at[0];
    v_from = v_head + static_cast<uint64_t>(page_v) * page_stride + at_v;
  };
  // load i (of CPW) of the keys and of the values of the located tile, into the buffer at byte address `to`
  auto ask = [&](int i, uint32_t to) __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    load_to_lds(k_from + k_off[i], to + lds_off[i] * 2);
    load_to_lds(v_from + v_off[i], to + (lds_off[i] + HALF) * 2);
    __builtin_amdgcn_sched_barrier(0);
  };

  Pages next;  // the pages of the tile after the one that is located
  // one tile from the buffer `stage`, for this wave's rows; meanwhile the located tile is asked for into the buffer
  // at byte address `to`
  auto compute = [&](int tile, const __bf16* stage, uint32_t to) __attribute__((always_inline)) {
    const int key0 = tile * kTile;
    bool any = false;
#pragma unroll
    for (int j = 0; j < R; ++j) any = any || (rows[j] > 0 && key0 <= pos_last[j] && key0 + kTile > lo_first[j]);
    if (tile >= te || !any) {  // no row of the wave sees a key of it
      next = look_up(tile + 2);
#pragma unroll
      for (int i = 0; i < CPW; ++i) ask(i, to);
      return;
    }
    const __bf16* k_s = stage;
    const __bf16* v_s = stage + HALF;
    // Operands come from LDS in batches; the reads of a batch are issued before the products of the batch before it,
    // which cover their latency.  After every second chunk of dimensions the next of the CPW loads is asked for:
    // asked for together, the waves queue up at the memory pipeline while the MFMA unit idles.
    constexpr int KB = NDC < 4 ? NDC : 4;  // dimension chunks per batch of key operands
    constexpr int KBATCHES = NDC / KB;
    floatx4 s[R][2];
#pragma unroll
    for (int j = 0; j < R; ++j) s[j][0] = s[j][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    bf16x8 kf[2][2][KB];
    auto read_keys = [&](int batch) __attribute__((always_inline)) {
#pragma unroll
      for (int b = 0; b < KB; ++b)
#pragma unroll
        for (int t = 0; t < 2; ++t)
          kf[batch % 2][t][b] = *reinterpret_cast<const bf16x8*>(k_s + ((t * NDC + batch * KB + b) * 64 + lane) * 8);
    };
    read_keys(0);
#pragma unroll
    for (int batch = 0; batch < KBATCHES; ++batch) {
      if (batch + 1 < KBATCHES) read_keys(batch + 1);
#pragma unroll
      for (int b = 0; b < KB; ++b) {
        const int dc = batch * KB + b;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < R; ++j)
            s[j][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[batch % 2][t][b], qf[j][dc], s[j][t], 0, 0, 0);
        if (dc % 2 == 1) ask(dc / 2, to);
      }
    }
    // All value operands are asked for here and arrive during the softmax arithmetic, in the registers that the key
    // operands have left: the reads of a workgroup's four waves take LDS 512 clocks, which the second product would
    // otherwise wait out (in batches of four blocks it was 3 to 4 % slower).
    constexpr int VB = NDB;  // output blocks per batch of value operands
    bf16x8 vf[2][VB];
    auto read_values = [&](int batch) __attribute__((always_inline)) {
#pragma unroll
      for (int b = 0; b < VB; ++b)
        vf[batch % 2][b] = *reinterpret_cast<const bf16x8*>(v_s + ((batch * VB + b) * 64 + lane) * 8);
    };
    read_values(0);
    // the pages of the tile after the next are looked up here: the table's entries arrive during the softmax
    // arithmetic, with the value operands (a wait for operands from LDS is a wait for scalar loads as well)
    next = look_up(tile + 2);
    __builtin_amdgcn_sched_barrier(0);
    bf16x8 pf[R];
    float alpha[R];
    bool rescale = false;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      // every row of the unit sees every key of the tile: no mask
      const bool whole = rows[j] == 16 && key0 + kTile - 1 <= pos_first[j] && key0 >= lo_last[j];
      float y[2][4];
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float x = s[j][t][v] * c1;
          if (CAP) x = c2 - 2.f * c2 * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x) + 1.f);
          y[t][v] = x;
        }
      if (!whole) {  // uniform over the wave
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int key = key0 + grp * 8 + t * 4 + v;
            y[t][v] = (row_ok[j] && key <= pos_r[j] && key >= lo_r[j]) ? y[t][v] : -INFINITY;
          }
      }
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) mx = fmaxf(mx, y[t][v]);
      mx = max_over_row_lanes(mx);
      const float m_new = fmaxf(m_run[j], mx);
      // a row that has seen no visible key yet keeps m = -inf; 2^(-inf - -inf) must not appear
      alpha[j] = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m_run[j] - m_new);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float e = __builtin_amdgcn_exp2f(y[t][v] - m_use);  // 2^-inf = 0
          psum += e;
          pf[j][t * 4 + v] = to_bf16_raw(e);
        }
      l_run[j] = l_run[j] * alpha[j] + psum;
      m_run[j] = m_new;
      rescale = rescale || alpha[j] != 1.f;
    }
    if (__builtin_amdgcn_ballot_w64(rescale) != 0) {  // rarely, once the maxima have settled
#pragma unroll
      for (int j = 0; j < R; ++j)
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[j][db][v] *= alpha[j];
    }
    // Lane (d = r, grp) of the value operand holds V^T[db * 16 + r][keys 8 * grp .. + 7 of the tile].  Values of
    // keys that no row may use (unwritten, given back, another request's) count as 0; their scores are masked
    // anyway.  That concerns the last tile of the keys and tiles at a window's lower edge.
    const bool fix = key0 + kTile > hi_g || key0 < lo_g;  // uniform
#pragma unroll
    for (int batch = 0; batch < NDB / VB; ++batch) {
      if (batch + 1 < NDB / VB) read_values(batch + 1);
      if (fix) {
#pragma unroll
        for (int b = 0; b < VB; ++b)
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int key = key0 + grp * 8 + e;
            if (key >= hi_g || key < lo_g) vf[batch % 2][b][e] = to_bf16_raw(0.f);
          }
      }
#pragma unroll
      for (int b = 0; b < VB; ++b)
#pragma unroll
        for (int j = 0; j < R; ++j)
          acc[j][batch * VB + b] =
              __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[batch % 2][b], pf[j], acc[j][batch * VB + b], 0, 0, 0);
    }
  };

  if (tb < te) {
    locate(look_up(tb));
#pragma unroll
    for (int i = 0; i < CPW; ++i) ask(i, lds0);
    next = look_up(tb + 1);
    // tile `tile` has been asked for into `cur`; `other` held tile - 1 and takes tile + 1
    auto step = [&](int tile, const __bf16* cur, uint32_t other) __attribute__((always_inline)) {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // this wave's chunks of `tile` have arrived
      bare_barrier();  // and everyone's; and every wave has finished tile - 1
      locate(next);
      compute(tile, cur, other);
    };
    const int te2 = tb + (te - tb + 1) / 2 * 2;
    for (int tile = tb; tile < te2; tile += 2) {
      step(tile, stage0, lds1);
      step(tile + 1, stage1, lds0);
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // the load asked for beyond the range
  }

  // acc[db][v] is O^T[d = db * 16 + 4 * grp + v][row r]
#pragma unroll
  for (int j = 0; j < R; ++j) {
    float l = l_run[j];
    l = sum_over_row_lanes(l);
    if (!row_ok[j]) continue;
    if (num_chunks == 1) {
      bf16* op = out + static_cast<size_t>(q_row[j]) * out_stride + static_cast<size_t>(kh * G + g) * HD;
      const float inv = 1.f / l;
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        const bf16x4 o4 = {to_bf16_raw(acc[j][db][0] * inv), to_bf16_raw(acc[j][db][1] * inv),
                           to_bf16_raw(acc[j][db][2] * inv), to_bf16_raw(acc[j][db][3] * inv)};
        *reinterpret_cast<bf16x4*>(op + db * 16 + 4 * grp) = o4;
      }
    } else {
      // the merge kernel works with natural logarithms
      const size_t row_words = HD + kRowExtra;
      const size_t unit = static_cast<size_t>(group * GROUP + wave * R + j) * Kh + kh;
      float* wp = workspace + ((unit * num_splits + split) * 16 + r) * row_words;
#pragma unroll
      for (int db = 0; db < NDB; ++db) *reinterpret_cast<floatx4*>(wp + db * 16 + 4 * grp) = acc[j][db];
      if (grp == 0) {
        wp[HD] = m_run[j] * (1.f / kLog2e);
        wp[HD + 1] = l;
      }
    }
  }
}

}  // namespace prefill

// R: units per wave.  2 halves the operand reads from LDS per row, but was 2.5 times slower: the compiler then keeps
// the accumulators of 32 rows in the registers that the arithmetic needs, a few loop invariants are spilled, and every
// reload of one waits for all outstanding memory loads, which are the next tile's keys and values.
constexpr int kPrefillRowTiles = 1;

int paged_attention_prefill_group() { return prefill::kWaves * kPrefillRowTiles; }

bool paged_attention_prefill_takes(int H, int Kh, int hd, int page_size, int max_q_len, int64_t q_stride, const void* q,
                                   int64_t out_stride, const void* out) {
  const int G = H / Kh;
  return (hd == 64 || hd == 128 || hd == 256) && page_size % 16 == 0 && G * max_q_len <= 16 && q_stride % 8 == 0 &&
         (reinterpret_cast<uintptr_t>(q) & 15u) == 0 && out_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 7u) == 0;
}

int paged_attention_prefill(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* units, int unit_begin, int unit_count,
                            void* out, int64_t out_stride, int H, int Kh, int hd, int page_size, int window,
                            float soft_cap, int max_kv_len, int max_q_len, int num_splits, void* workspace, size_t workspace_bytes,
                            hipStream_t stream) {
  constexpr int R = kPrefillRowTiles;
  constexpr int kGroup = prefill::kWaves * R;
  if (unit_count == 0) return 0;
  const int G = H / Kh;
  const int groups = unit_count / kGroup;
  int span = window > 0 && window < max_kv_len ? window + 16 * kGroup : max_kv_len;  // keys a workgroup reads at most
  if (span < 1) span = 1;
  const int max_tiles = (span + kTile - 1) / kTile + 1;
  // Ranges of `chunk` tiles, as many as a group's keys take.  Measured: best is one round of about two workgroups
  // per CU (every further range costs a set-up, and 16 KiB of partial results per unit and head written and read
  // again), with ranges of 16 tiles at least.  How many workgroups there will be is estimated from the tokens of
  // this launch: the groups of a fresh prompt see from a tile to all of it (half on average), a portion late in a
  // long prompt sees all of its history in every group.
  int chunk;
  if (num_splits > 0) {
    chunk = (max_tiles + num_splits - 1) / num_splits;
  } else {
    const int64_t tokens = static_cast<int64_t>(unit_count) * max_q_len;
    const int64_t avg_keys = span - (tokens < span ? tokens : span) / 2;
    const int64_t avg_tiles = avg_keys / kTile + 1;
    const int64_t pairs = static_cast<int64_t>(groups) * Kh;
    int64_t ranges = 512 * static_cast<int64_t>(max_tiles) / (pairs * avg_tiles);
    if (ranges > max_tiles / 16) ranges = max_tiles / 16;
    if (ranges < 1) ranges = 1;
    chunk = static_cast<int>((max_tiles + ranges - 1) / ranges);
  }
  if (chunk > max_tiles) chunk = max_tiles;
  int KS = (max_tiles + chunk - 1) / chunk;
  const size_t per_split = static_cast<size_t>(unit_count) * Kh * 16 * (hd + kRowExtra) * sizeof(float);
  while (KS > 1 && (KS > kMaxSplits || workspace == nullptr || per_split * KS > workspace_bytes)) {
    ++chunk;
    KS = (max_tiles + chunk - 1) / chunk;
  }
  const dim3 grid(Kh, KS, groups);
  const bf16* qp = static_cast<const bf16*>(q);
  const bf16* kp = static_cast<const bf16*>(k_pages);
  const bf16* vp = static_cast<const bf16*>(v_pages);
  const SeqMeta* um = reinterpret_cast<const SeqMeta*>(units);
  bf16* op = static_cast<bf16*>(out);
  float* ws = static_cast<float*>(workspace);
#define SA_LAUNCH(NDC)                                                                                              \
  do {                                                                                                              \
    if (soft_cap > 0.f)                                                                                             \
      prefill::paged_attention_prefill_kernel<NDC, R, true><<<grid, 256, 0, stream>>>(                              \
          qp, q_stride, kp, vp, block_table, table_stride, um, unit_begin, op, out_stride, Kh, G, page_size, window, \
          soft_cap, ws, chunk);                                                                                     \
    else                                                                                                            \
      prefill::paged_attention_prefill_kernel<NDC, R, false><<<grid, 256, 0, stream>>>(                             \
          qp, q_stride, kp, vp, block_table, table_stride, um, unit_begin, op, out_stride, Kh, G, page_size, window, \
          soft_cap, ws, chunk);                                                                                     \
  } while (0)
  if (hd == 64) SA_LAUNCH(2);
  else if (hd == 128) SA_LAUNCH(4);
  else if (hd == 256) SA_LAUNCH(8);
  else {
    set_error("paged_attention_prefill: head size %d is not 64, 128 or 256", hd);
    return 1;
  }
#undef SA_LAUNCH
  if (check_launch("paged_attention_prefill")) return 1;
  if (KS > 1)
    return attention_merge_ranges(ws, KS, hd, um, unit_begin, unit_count, max_q_len, op, out_stride, Kh, G, stream, chunk,
                                  kGroup, window);
  return 0;
}

}  // namespace sa
