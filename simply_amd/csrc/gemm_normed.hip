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
constexpr int kUnroll = 4;
constexpr int kMaxGroups = 256;  // one workgroup per compute unit; each takes the same number of tiles, or one fewer

__device__ inline float gelu_tanh_f(float x) {
  const float k = 0.7978845608028654f;
  return 0.5f * x * (1.f + tanhf(k * (x + 0.044715f * x * x * x)));
}
__device__ inline bf16x8 load_frag(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }

// NCH: 256-element pieces of a row (K <= 256 * NCH)
template <int EPI, int NCH>
__global__ __launch_bounds__(kWaves* kWave) void gemm_normed_kernel(
    const bf16* __restrict__ y, const float* __restrict__ h_in, float* __restrict__ h_out,
    const void* __restrict__ w_post, int w_post_dtype, float eps_post, float plus_post,
    const void* __restrict__ w_next, int w_next_dtype, float eps_next, float plus_next, const bf16* __restrict__ W,
    void* __restrict__ C, int c_dtype, int64_t ldc, int M, int N, int K, int chunks, int act_rows, float cap) {
  constexpr int NP = EPI == 1 ? 2 : 1;
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
  const int ntiles = (N + 15) / 16;
  const int c0 = static_cast<int>(static_cast<int64_t>(chunks) * wave / kWaves);
  const int c1 = static_cast<int>(static_cast<int64_t>(chunks) * (wave + 1) / kWaves);
  const size_t tile_elems = static_cast<size_t>(chunks) * 512;
  const bf16* wrow = W + (EPI == 1 ? 2 : 1) * static_cast<size_t>(blockIdx.x) * tile_elems + lane * 8;
  const bf16* w2row = wrow + tile_elems;
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
      if (EPI == 1) a2[set][u] = ok ? load_frag(w2row + static_cast<size_t>(c + u) * 512) : zero;
    }
  };
  auto mul_set = [&](int set, int c) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      // beyond the wave's range the W fragment is zero; the activations read there are finite (zero padded rows)
      const int k = (c + u < c1 ? c + u : c0) * 32;
      const bf16x8 b = a_ok ? load_frag(arow + k) : zero;
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[set][u], b, acc[0], 0, 0, 0);
      if (EPI == 1) acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[set][u], b, acc[1], 0, 0, 0);
    }
  };
  load_set(0, c0);

  // ---- the two norms, one wave per row.  A lane holds 4 consecutive elements of each 256-element piece of the
  // row; all loads of a row are issued before the first use, so a row costs one trip to L2.
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  const bool add = y != nullptr, post = add && w_post != nullptr;
  for (int m = wave; m < act_rows; m += kWaves) {
    bf16* dst = act + static_cast<size_t>(m) * pitch;
    if (m >= M) {
      for (int d = lane; d < pitch; d += kWave) dst[d] = float_to_bf16(0.f);
      continue;
    }
    const size_t rb = static_cast<size_t>(m) * K;
    float4 hv[NCH];
    bf16x4 yv[NCH], wpv[NCH], wnv[NCH];
    const bf16* wp16 = static_cast<const bf16*>(w_post);
    const bf16* wn16 = static_cast<const bf16*>(w_next);
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int d = c * 256 + lane * 4;
      hv[c] = d < K ? *reinterpret_cast<const float4*>(h_in + rb + d) : float4{0.f, 0.f, 0.f, 0.f};
      yv[c] = (add && d < K) ? *reinterpret_cast<const bf16x4*>(y + rb + d) : bf16x4{};
      wpv[c] = (post && d < K) ? *reinterpret_cast<const bf16x4*>(wp16 + d) : bf16x4{};
      wnv[c] = d < K ? *reinterpret_cast<const bf16x4*>(wn16 + d) : bf16x4{};
    }
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
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = static_cast<float>(yv[c][e]);
          h[e] += post ? v * rr * (static_cast<float>(wpv[c][e]) + plus_post) : v;
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
#pragma unroll
      for (int e = 0; e < 4; ++e)
        dst[d + e] = float_to_bf16(h[e] * r2 * (static_cast<float>(wnv[c][e]) + plus_next));
    }
    for (int d = K + lane; d < pitch; d += kWave) dst[d] = float_to_bf16(0.f);
  }
  __syncthreads();

  for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
#pragma unroll
    for (int p = 0; p < NP; ++p) acc[p] = floatx4{0.f, 0.f, 0.f, 0.f};
    const bool more = tile + static_cast<int>(gridDim.x) < ntiles;
    const size_t step = (EPI == 1 ? 2 : 1) * static_cast<size_t>(gridDim.x) * tile_elems;
    for (int c = c0; c < c1; c += 2 * kUnroll) {
      load_set(1, c + kUnroll);
      mul_set(0, c);
      if (c + 2 * kUnroll < c1) {
        load_set(0, c + 2 * kUnroll);
      } else if (more) {  // the next tile's first fragments
        wrow += step;
        w2row += step;
        load_set(0, c0);
        wrow -= step;
        w2row -= step;
      }
      mul_set(1, c + kUnroll);
    }
    wrow += step;
    w2row += step;

    // ---- lane holds D[n = 4 * kq + v][m = r]; the waves' tiles are added up through LDS, in wave order
    __syncthreads();  // the previous tile's sums have been read
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[(wave * NP + p) * (16 * 17) + (4 * kq + v) * 17 + r] = acc[p][v];
    __syncthreads();
    if (tid < 256) {
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
        if (EPI == 1) v = gelu_tanh_f(to_float(float_to_bf16(v))) * to_float(float_to_bf16(sum[NP - 1]));
        else if (EPI == 2) v = cap * tanhf(v / cap);
        store_f(C, c_dtype, static_cast<size_t>(ml) * ldc + n, v);
      }
    }
  }
}

template <int EPI, int NCH>
static int launch(const bf16* y, const float* h_in, float* h_out, const void* w_post, int w_post_dtype, float eps_post,
                  float plus_post, const void* w_next, int w_next_dtype, float eps_next, float plus_next, const bf16* W,
                  void* C, int c_dtype, int64_t ldc, int M, int N, int K, float cap, hipStream_t stream) {
  const int act_rows = M <= 8 ? 8 : 16;
  const size_t lds = static_cast<size_t>(act_rows) * (K + 8) * sizeof(bf16) +
                     static_cast<size_t>(kWaves) * (EPI == 1 ? 2 : 1) * 16 * 17 * sizeof(float);
  auto kernel = gemm_normed_kernel<EPI, NCH>;
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
  const int ntiles = (N + 15) / 16;
  const int grid = (ntiles + (ntiles + kMaxGroups - 1) / kMaxGroups - 1) / ((ntiles + kMaxGroups - 1) / kMaxGroups);
  kernel<<<grid, kWaves * kWave, lds, stream>>>(y, h_in, h_out, w_post, w_post_dtype, eps_post, plus_post, w_next,
                                                         w_next_dtype, eps_next, plus_next, W, C, c_dtype, ldc, M, N, K,
                                                         (K + 31) / 32, act_rows, cap);
  return check_launch("gemm_normed");
}

}  // namespace normed
}  // namespace sa

using namespace sa;

extern "C" int sa_gemm_normed_takes(int M, int N, int K) {
  const size_t lds = static_cast<size_t>(M <= 8 ? 8 : 16) * (K + 8) * 2 + 8 * 2 * 16 * 17 * 4;
  return M >= 1 && M <= 16 && K % 32 == 0 && K <= 256 * 10 && lds <= 160 * 1024;
}

extern "C" int sa_gemm_normed(const void* y, const float* h_in, float* h_out, const void* w_post, int w_post_dtype,
                              float eps_post, int plus_one_post, const void* w_next, int w_next_dtype, float eps_next,
                              int plus_one_next, const void* W, void* C, int c_dtype, int64_t ldc, int M, int N, int K,
                              int epilogue, float cap, hipStream_t stream) {
  SA_REQUIRE(sa_gemm_normed_takes(M, N, K),
             "gemm_normed takes 1..16 rows and a width that is a multiple of 32, at most 2560, and fits in LDS; got M=%d K=%d", M, K);
  SA_REQUIRE(N > 0 && ldc >= N && w_next != nullptr && h_in != nullptr && W != nullptr, "gemm_normed: bad arguments");
  SA_REQUIRE(w_next_dtype == kBF16 && (w_post == nullptr || w_post_dtype == kBF16),
             "gemm_normed: the norm weights must be bfloat16");
  SA_REQUIRE(y == nullptr || (h_out != nullptr && h_out != h_in),
             "gemm_normed: with y the updated residual goes to a buffer other than the input");
  SA_REQUIRE(epilogue >= 0 && epilogue <= 2 && (epilogue != 2 || cap > 0.f), "gemm_normed: bad epilogue");
  const bf16* yb = static_cast<const bf16*>(y);
  const bf16* w = static_cast<const bf16*>(W);
  const float pp = plus_one_post ? 1.f : 0.f, pn = plus_one_next ? 1.f : 0.f;
#define SA_NORMED(EPI, NCH)                                                                                      \
  return normed::launch<EPI, NCH>(yb, h_in, h_out, w_post, w_post_dtype, eps_post, pp, w_next, w_next_dtype, eps_next, \
                                  pn, w, C, c_dtype, ldc, M, N, K, cap, stream)
  if (epilogue == 0) SA_NORMED(0, 10);
  if (epilogue == 1) SA_NORMED(1, 10);
  SA_NORMED(2, 10);
#undef SA_NORMED
}
