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

// Partial results of key ranges lie in the workspace as [unit * Kh + kh][range][16 rows][hd + kRowExtra] floats:
// the unnormalised output, then the maximum and the sum of the row (and two unused words: rows stay 16-byte
// aligned).  Adds them up, range by range in order, into `out`.
// max_q_len: the most tokens in a unit.
int attention_merge_ranges(const float* workspace, int num_ranges, int hd, const SeqMeta* units, int unit_begin,
                           int unit_count, int max_q_len, bf16* out, int64_t out_stride, int Kh, int G,
                           hipStream_t stream);

}  // namespace sa
