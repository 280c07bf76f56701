// What the two MFMA attention kernels (few query rows with the keys cut over workgroups; blocks of 64 query rows
// with keys and values shared through LDS) have in common.
#pragma once
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int kTile = 32;         // keys per MFMA tile
constexpr int kMaxSplits = 256;
constexpr int kRowExtra = 4;   // key ranges per request at most

// A unit of work: `q_len` consecutive tokens of the request in block-table row `slot`; the first is row `q_start`
// of the step and stands at position `pos0`.
struct SeqMeta {
  int slot, q_start, q_len, pos0;
};

__device__ inline __bf16 to_bf16_raw(float f) { return static_cast<__bf16>(f); }

// A value of the lanes l, l ^ 16, l ^ 32 and l ^ 48 combined (the four lanes that share a row of an MFMA result),
// in every one of them, with gfx950's swaps of 16- and 32-lane rows between two registers: one instruction each
// on the vector unit, where a shuffle goes through the LDS crossbar and waits behind the operand reads queued there.
// v_permlane16_swap exchanges rows 1 and 3 of its first operand with rows 0 and 2 of its second, v_permlane32_swap
// the upper half of the first with the lower half of the second: from two copies of x come [x0 x0 x2 x2] and
// [x1 x1 x3 x3], then the halves.
template <typename Op>
__device__ __forceinline__ float over_row_lanes(float x, Op op) {
  const unsigned u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned v = __float_as_uint(op(__uint_as_float(a[0]), __uint_as_float(a[1])));
  const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return op(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float max_over_row_lanes(float x) {
  return over_row_lanes(x, [](float a, float b) { return fmaxf(a, b); });
}
__device__ __forceinline__ float sum_over_row_lanes(float x) {
  return over_row_lanes(x, [](float a, float b) { return a + b; });
}

// Partial results of key ranges lie in the workspace as [unit * Kh + kh][range][16 rows][hd + kRowExtra] floats:
// the unnormalised output, then the maximum and the sum of the row (and two unused words: rows stay 16-byte
// aligned).  Adds them up, range by range in order, into `out`.  max_q_len: the most tokens in a unit.
// chunk_tiles == 0: every unit has all num_ranges ranges.  chunk_tiles > 0: units come in groups of `group`, a
// group's keys (what some row of it sees, with `window`) are cut into ranges of chunk_tiles tiles of kTile keys,
// as many as it takes (num_ranges at most); a group with one range has written `out` itself and is skipped.
int attention_merge_ranges(const float* workspace, int num_ranges, int hd, const SeqMeta* units, int unit_begin,
                           int unit_count, int max_q_len, bf16* out, int64_t out_stride, int Kh, int G,
                           hipStream_t stream, int chunk_tiles = 0, int group = 1, int window = 0);

// The keys [lo, hi) that some row of the units [first, first + group) sees, and their request's slot.  False: no
// rows.
__device__ inline bool group_keys(const SeqMeta* units, int first, int group, int window, int* lo, int* hi, int* slot) {
  int lo_g = 0x7fffffff, hi_g = 0;
  for (int w = 0; w < group; ++w) {
    const SeqMeta m = units[first + w];
    if (m.q_len > 0) {
      const int lo_w = (window > 0 && m.pos0 - window + 1 > 0) ? m.pos0 - window + 1 : 0;
      lo_g = lo_w < lo_g ? lo_w : lo_g;
      hi_g = m.pos0 + m.q_len > hi_g ? m.pos0 + m.q_len : hi_g;
      *slot = m.slot;
    }
  }
  *lo = lo_g;
  *hi = hi_g;
  return hi_g != 0;
}

// How many ranges of chunk_tiles tiles of kTile keys the keys [lo, hi) are cut into.
__device__ inline int key_chunks(int lo, int hi, int chunk_tiles) {
  const int tiles = (hi + kTile - 1) / kTile - lo / kTile;
  return (tiles + chunk_tiles - 1) / chunk_tiles;
}

}  // namespace sa
