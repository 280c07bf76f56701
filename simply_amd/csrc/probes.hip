// Two measurements of the machine itself, by which the kernels' rates are judged: how fast all CUs together read
// from HBM (contiguously, and in 8 KiB pieces in a given order, as the pages of a cache lie), and how many
// v_mfma_f32_16x16x32_bf16 they retire with operands of a given content (the clock that the GPU holds under the
// matrix units' load depends on the bits that toggle: zeros run near the published rate, random values do not).
// Neither result is used; both kernels exist for their time.
#include "api.h"
#include "common.h"

namespace sa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int kPiece = 8192;  // bytes

// A wave reads pieces wave, wave + waves, ... (two at a time: sixteen loads of 1 KiB in flight).
__global__ __launch_bounds__(512) void hbm_read_kernel(const floatx4* __restrict__ in, const int* __restrict__ order,
                                                       int64_t pieces, float* __restrict__ sink) {
  const int lane = threadIdx.x % kWave;
  const int64_t waves = static_cast<int64_t>(gridDim.x) * (blockDim.x / kWave);
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  floatx4 sum = {0.f, 0.f, 0.f, 0.f};
  for (int64_t p = wave; p < pieces; p += 2 * waves) {
    floatx4 v[16];
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const int64_t at = p + g * waves < pieces ? p + g * waves : p;
      const int64_t piece = order != nullptr ? order[at] : at;
#pragma unroll
      for (int u = 0; u < 8; ++u) v[g * 8 + u] = in[piece * (kPiece / 16) + u * kWave + lane];
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) sum += v[u];
  }
  if (sum[0] + sum[1] + sum[2] + sum[3] == 12345.678f) sink[threadIdx.x] = sum[0];  // (keeps the loads)
}

// Eight waves a workgroup, two per SIMD, sixteen independent accumulators each.
__global__ __launch_bounds__(512) void mfma_rate_kernel(const bf16x8* __restrict__ operands, int iters,
                                                        float* __restrict__ sink) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[(threadIdx.x + 64 * i + blockIdx.x) % 1024];
    b[i] = operands[(threadIdx.x * 3 + 7 * i + blockIdx.x) % 1024];
  }
  floatx4 acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i % 4], b[i / 4], acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  if (s == 12345.678f) sink[threadIdx.x] = s;
}

}  // namespace sa

extern "C" {

int sa_probe_hbm_read(const void* buffer, int64_t bytes, const int* order, void* sink, hipStream_t stream) {
  SA_REQUIRE(buffer != nullptr && sink != nullptr && bytes >= sa::kPiece && bytes % sa::kPiece == 0,
             "probe_hbm_read: a buffer of whole 8 KiB pieces and a sink of 512 floats");
  SA_REQUIRE((reinterpret_cast<uintptr_t>(buffer) & 15u) == 0, "probe_hbm_read: the buffer must be 16-byte aligned");
  sa::hbm_read_kernel<<<256, 512, 0, stream>>>(static_cast<const sa::floatx4*>(buffer), order, bytes / sa::kPiece,
                                               static_cast<float*>(sink));
  return sa::check_launch("probe_hbm_read");
}

int sa_probe_mfma(const void* operands, int iters, int workgroups, void* sink, hipStream_t stream) {
  SA_REQUIRE(operands != nullptr && sink != nullptr && iters >= 1 && workgroups >= 1 && workgroups <= 65536,
             "probe_mfma: 16 KiB of operands, a sink of 512 floats, at least one iteration and workgroup");
  sa::mfma_rate_kernel<<<workgroups, 512, 0, stream>>>(static_cast<const sa::bf16x8*>(operands), iters,
                                                       static_cast<float*>(sink));
  return sa::check_launch("probe_mfma");
}

}  // extern "C"
