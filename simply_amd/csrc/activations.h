// Activations of the gated product's epilogue, C = act(A.Wg^T) * (A.Wu^T) (simply/model_lib.py:714-727, where
// `act` is looked up by name: gelu :94-96, squared_relu :99-101, silu :104).  An activation is a code that travels
// in the epilogue argument of the entry points (epilogue = 1 + 16 * code) and reaches the kernels as a launch
// argument; a kernel calls gated_activation(code, x), whose branch is uniform over the launch.  Another
// activation is another code, a function here and a case in the two switches: no kernel changes.
#pragma once
#include <hip/hip_runtime.h>

namespace sa {

enum Activation : int { kActGeluTanh = 0, kActSilu = 1, kActSquaredRelu = 2, kNumActivations = 3 };

constexpr int kEpilogueNone = 0, kEpilogueGated = 1, kEpilogueSoftCap = 2;
// The epilogue argument of an entry point: its kind in the low four bits, the gated kind's activation above them.
__host__ __device__ inline int epilogue_kind(int epilogue) { return epilogue & 15; }
__host__ __device__ inline int epilogue_activation(int epilogue) { return epilogue >> 4; }

// tanh-approximated GELU for the bfloat16 kernels: tanh(u) = 1 - 2 / (exp(2 u) + 1) with the hardware's exponential and
// reciprocal (relative error about 1e-6, far below a bfloat16 step); exact at both ends.  simply/model_lib.py:94-96.
__device__ inline float gelu_tanh_fast(float x) {
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  const float t = 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * u) + 1.f);
  return 0.5f * x * (1.f + t);
}
// x * sigmoid(x) with the hardware's exponential and reciprocal; exact at both ends (exp(-x) = inf gives x * 0).
__device__ inline float silu_fast(float x) { return x * __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
__device__ inline float squared_relu(float x) { return x > 0.f ? x * x : 0.f; }

// For the bfloat16 kernels.
__device__ inline float gated_activation(int act, float x) {
  switch (act) {
    case kActSilu: return silu_fast(x);
    case kActSquaredRelu: return squared_relu(x);
    default: return gelu_tanh_fast(x);
  }
}

// For the 32-bit path: the library's tanhf and expf, no approximations.
__device__ inline float gated_activation_exact(int act, float x) {
  switch (act) {
    case kActSilu: return x / (1.f + expf(-x));
    case kActSquaredRelu: return squared_relu(x);
    default: return 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
  }
}

}  // namespace sa
