// Shared helpers of the gfx950 kernels: element types, conversions, wave
// reductions and the error channel of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "activations.h"

namespace sa {

// Element type codes used across the C interface.
enum DType : int { kF32 = 0, kBF16 = 1 };

constexpr int kWave = 64;  // CDNA wavefront width

struct bf16 {
  uint16_t bits;
};

__host__ __device__ inline float to_float(bf16 x) {
  union { uint32_t u; float f; } c;
  c.u = static_cast<uint32_t>(x.bits) << 16;
  return c.f;
}
__host__ __device__ inline float to_float(float x) { return x; }

// Round to nearest even; NaN stays NaN.  On the device this is gfx950's own conversion instruction.
__host__ __device__ inline bf16 float_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_bit_cast(bf16, static_cast<__bf16>(f));
#endif
  union { uint32_t u; float f; } c;
  c.f = f;
  uint32_t u = c.u;
  bf16 r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = static_cast<uint16_t>((u >> 16) | 0x0040u);
    return r;
  }
  u += 0x7fffu + ((u >> 16) & 1u);
  r.bits = static_cast<uint16_t>(u >> 16);
  return r;
}

template <typename T> __host__ __device__ inline T from_float(float f);
template <> __host__ __device__ inline float from_float<float>(float f) { return f; }
template <> __host__ __device__ inline bf16 from_float<bf16>(float f) { return float_to_bf16(f); }

// Loads and stores through a runtime element type (uniform over a launch).
__device__ inline float load_f(const void* p, int dtype, size_t i) {
  return dtype == kF32 ? static_cast<const float*>(p)[i] : to_float(static_cast<const bf16*>(p)[i]);
}
__device__ inline void store_f(void* p, int dtype, size_t i, float v) {
  if (dtype == kF32) static_cast<float*>(p)[i] = v;
  else static_cast<bf16*>(p)[i] = float_to_bf16(v);
}

// A value of all 64 lanes of a wave combined, in every lane (all lanes active): within rows of 16 lanes by data-parallel
// primitives on the vector unit (quad exchanges, then the mirrored half row and the mirrored row: every lane of a quad,
// then of a half row, holds the same partial result, so the mirror image brings the other half's), across rows by
// gfx950's row swaps.  Eight instructions where six shuffles through the LDS crossbar took 500 to 700 clocks.
template <int CTRL>
__device__ __forceinline__ float lane_exchange(float v) {  // a DPP control: the value of another lane of the row
  const int bits = __float_as_int(v);
  return __int_as_float(__builtin_amdgcn_update_dpp(bits, bits, CTRL, 0xF, 0xF, false));
}
template <typename Op>
__device__ __forceinline__ float wave_combine(float v, Op op) {
  v = op(v, lane_exchange<0xB1>(v));   // quad_perm [1, 0, 3, 2]
  v = op(v, lane_exchange<0x4E>(v));   // quad_perm [2, 3, 0, 1]
  v = op(v, lane_exchange<0x141>(v));  // row_half_mirror
  v = op(v, lane_exchange<0x140>(v));  // row_mirror
  const unsigned u = __float_as_uint(v);
  const auto rows = __builtin_amdgcn_permlane16_swap(u, u, false, false);   // [r0 r0 r2 r2], [r1 r1 r3 r3]
  const unsigned w = __float_as_uint(op(__uint_as_float(rows[0]), __uint_as_float(rows[1])));
  const auto halves = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return op(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
}
__device__ inline float wave_sum(float v) {
  return wave_combine(v, [](float a, float b) { return a + b; });
}
__device__ inline float wave_max(float v) {
  return wave_combine(v, [](float a, float b) { return fmaxf(a, b); });
}

// Sum over a block of up to 1024 threads; every thread gets the result.  The
// order of additions depends only on the block size, never on the data.
__device__ inline float block_sum(float v, float* scratch /* >= 16 floats */) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

// Layout of a page of keys [page_size keys][hd]: row-major, or, when the sizes allow it, in 16-key x 32-dimension
// blocks of MFMA operand order (as weight tiles are): [page_size / 16][hd / 32][lane 64][8] with
// lane = (d % 32) / 8 * 16 + key % 16, so that a wave reads a block of 16 keys as contiguous KiB.
__host__ __device__ inline bool keys_tiled(int page_size, int hd) { return page_size % 16 == 0 && hd % 32 == 0; }
__host__ __device__ inline size_t key_index(bool tiled, int page_size, int hd, int key_in_page, int d) {
  if (!tiled) return static_cast<size_t>(key_in_page) * hd + d;
  return ((static_cast<size_t>(key_in_page / 16) * (hd / 32) + d / 32) * 64 + ((d % 32) / 8) * 16 + key_in_page % 16) * 8 +
         d % 8;
}

// Error channel: entry points return 0 on success, non-zero after set_error().
void set_error(const char* fmt, ...);
int check_launch(const char* what);

}  // namespace sa

#define SA_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      sa::set_error(__VA_ARGS__);        \
      return 1;                          \
    }                                    \
  } while (0)
