// Row-wise kernels: embedding lookup, RMSNorm (alone and fused with the residual
// sum and the next norm), rotary encoding fused with the cache write, row gather.
// All statistics, angles and the residual sum are in 32-bit whatever the
// activation type is.
#include <type_traits>

#include "api.h"
#include "common.h"

namespace sa {

// ------------------------------------------------------------------ embedding
// out[t, :] = float(table[tokens[t], :]) * scale.   simply/utils/module.py:450-481
// `packed`: the table is tiled like a matrix-product weight, [V / 16][ceil(D / 32)][kq 4][row 16][8].
__global__ void embed_kernel(const void* __restrict__ table, int table_dtype, const int* __restrict__ tokens,
                             float* __restrict__ out, int D, int V, float scale, int packed) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);  // the host has already refused ids outside the table
  const size_t base = static_cast<size_t>(tok) * D;
  const int chunks = (D + 31) / 32;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const size_t i = packed ? ((static_cast<size_t>(tok / 16) * chunks + d / 32) * 64 + ((d % 32) / 8) * 16 + tok % 16) * 8 + d % 8
                            : base + d;
    out[static_cast<size_t>(t) * D + d] = load_f(table, table_dtype, i) * scale;
  }
}

// ------------------------------------------------------------------ RMSNorm
// y = x * rsqrt(mean(x^2) + eps) * (w + plus_one).   simply/model_lib.py:154-178
__global__ void rmsnorm_kernel(const void* __restrict__ x, int x_dtype, int64_t x_stride,
                               const void* __restrict__ w, int w_dtype, void* __restrict__ out, int out_dtype,
                               int64_t out_stride, int D, float eps, float plus_one) {
  __shared__ float scratch[16];
  const size_t xb = static_cast<size_t>(blockIdx.x) * x_stride, ob = static_cast<size_t>(blockIdx.x) * out_stride;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = load_f(x, x_dtype, xb + d);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = rsqrtf(ss / static_cast<float>(D) + eps);
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = load_f(x, x_dtype, xb + d) * r;
    store_f(out, out_dtype, ob + d, v * (load_f(w, w_dtype, d) + plus_one));
  }
}

// residual[t, :] += norm(y[t, :]; w_post);  then, if w_next: out[t, :] = norm(residual[t, :]; w_next).
// The residual stream is 32-bit.  simply/model_lib.py:2681-2683 and :2690.
// Rows of up to kRowRegs * blockDim elements are held in registers: every input is read once and all loads are
// issued before the first reduction, so that the kernel pays the memory latency once (it runs a hundred times
// per decode step on a handful of rows).
constexpr int kRowRegs = 5;  // (1024 threads hold 5120: the width of the 27B shape is 4608)
__global__ void add_rmsnorm_kernel(const void* __restrict__ y, int y_dtype, const void* __restrict__ w_post,
                                   int w_post_dtype, float eps_post, float plus_one_post, float* __restrict__ residual,
                                   const void* __restrict__ w_next, int w_next_dtype, float eps_next,
                                   float plus_one_next, void* __restrict__ out, int out_dtype, int D,
                                   const int* __restrict__ index) {
  // index: block b works on row index[b] of y and of the residual, which it only reads, and writes row b of out
  // (the rows whose logits are wanted, at a model's end: the other rows' sums are of no use to anyone)
  __shared__ float scratch[16];
  const size_t rb = static_cast<size_t>(index != nullptr ? index[blockIdx.x] : static_cast<int>(blockIdx.x)) * D;
  const size_t ob = static_cast<size_t>(blockIdx.x) * D;
  const bool keep = index == nullptr;  // the residual stream is updated
  if (D <= kRowRegs * static_cast<int>(blockDim.x)) {
    float yv[kRowRegs], hv[kRowRegs], wp[kRowRegs], wn[kRowRegs];
#pragma unroll
    for (int j = 0; j < kRowRegs; ++j) {
      const int d = threadIdx.x + j * blockDim.x;
      const bool ok = d < D;
      yv[j] = ok ? load_f(y, y_dtype, rb + d) : 0.f;
      hv[j] = ok ? residual[rb + d] : 0.f;
      wp[j] = (ok && w_post != nullptr) ? load_f(w_post, w_post_dtype, d) + plus_one_post : 1.f;
      wn[j] = (ok && w_next != nullptr) ? load_f(w_next, w_next_dtype, d) + plus_one_next : 1.f;
    }
    float r = 1.f;
    if (w_post != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < kRowRegs; ++j) ss += yv[j] * yv[j];
      ss = block_sum(ss, scratch);
      r = rsqrtf(ss / static_cast<float>(D) + eps_post);
    }
    float ss2 = 0.f;
#pragma unroll
    for (int j = 0; j < kRowRegs; ++j) {
      const int d = threadIdx.x + j * blockDim.x;
      const float v = w_post != nullptr ? yv[j] * r * wp[j] : yv[j];
      hv[j] += v;
      if (d < D) {
        if (keep) residual[rb + d] = hv[j];
        ss2 += hv[j] * hv[j];
      }
    }
    if (w_next == nullptr) return;
    ss2 = block_sum(ss2, scratch);
    const float r2 = rsqrtf(ss2 / static_cast<float>(D) + eps_next);
#pragma unroll
    for (int j = 0; j < kRowRegs; ++j) {
      const int d = threadIdx.x + j * blockDim.x;
      if (d < D) store_f(out, out_dtype, ob + d, hv[j] * r2 * wn[j]);
    }
    return;
  }
  float ss = 0.f;
  if (w_post != nullptr) {
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      const float v = load_f(y, y_dtype, rb + d);
      ss += v * v;
    }
    ss = block_sum(ss, scratch);
  }
  const float r = w_post != nullptr ? rsqrtf(ss / static_cast<float>(D) + eps_post) : 1.f;
  float ss2 = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float v = load_f(y, y_dtype, rb + d);
    if (w_post != nullptr) v = v * r * (load_f(w_post, w_post_dtype, d) + plus_one_post);
    const float h = residual[rb + d] + v;
    if (keep) residual[rb + d] = h;  // re-read below by the same thread only
    ss2 += h * h;
  }
  if (w_next == nullptr) return;
  ss2 = block_sum(ss2, scratch);
  const float r2 = rsqrtf(ss2 / static_cast<float>(D) + eps_next);
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float h = residual[rb + d];
    if (!keep) {  // the sum was not stored: made once more
      float v = load_f(y, y_dtype, rb + d);
      if (w_post != nullptr) v = v * r * (load_f(w_post, w_post_dtype, d) + plus_one_post);
      h += v;
    }
    store_f(out, out_dtype, ob + d, h * r2 * (load_f(w_next, w_next_dtype, d) + plus_one_next));
  }
}

// The same for many rows (portions of prompts), a row to a workgroup of four waves: every lane holds NP pieces of
// four elements, all loads of a row are asked for before the first use, the two sums go through LDS.  A row is a
// chain of load, sum, store, sum, store; with a row spread over four waves there are four times the waves to
// overlap these chains than with a wave to a row: 2,048 rows of 2,304 elements (56 MB read and written) take 14 us
// where a wave to a row took 20, 512 rows 6.6 against 9.0, 8,192 rows 52 against 77.  D % 4 == 0, D <= 1024 NP,
// 16-byte aligned.
// PLANES (with YT = bf16, one row to a workgroup): y is not read but made, as the sum of that many float planes
// [T][D] at y_planes in their order, rounded to bfloat16: what the sum kernel of a product with K cut over
// workgroups would have written, without that kernel and its round trip through memory.
template <typename YT, typename OT, int NP, bool PLANES = false>
__global__ __launch_bounds__(256) void add_rmsnorm_split_kernel(
    const YT* __restrict__ y, const void* __restrict__ w_post, int w_post_dtype, float eps_post, float plus_one_post,
    float* __restrict__ residual, const void* __restrict__ w_next, int w_next_dtype, float eps_next, float plus_one_next,
    OT* __restrict__ out, int T, int D, int rows_per_group, const float* __restrict__ y_planes, int planes) {
  __shared__ float scratch[32];
  const int tid = threadIdx.x;
  using RawY = typename std::conditional<sizeof(YT) == 4, float4, uint2>::type;
  auto scales = [&](const void* w, int dtype, float plus, int d) __attribute__((always_inline)) {
    if (dtype == kBF16) {
      const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const bf16*>(w) + d);
      return float4{__uint_as_float(raw.x << 16) + plus, __uint_as_float(raw.x & 0xffff0000u) + plus,
                    __uint_as_float(raw.y << 16) + plus, __uint_as_float(raw.y & 0xffff0000u) + plus};
    }
    const float4 raw = *reinterpret_cast<const float4*>(static_cast<const float*>(w) + d);
    return float4{raw.x + plus, raw.y + plus, raw.z + plus, raw.w + plus};
  };
  float4 wp[NP], wn[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int d = (p * 256 + tid) * 4;
    wp[p] = wn[p] = float4{1.f, 1.f, 1.f, 1.f};
    if (d < D && w_post != nullptr) wp[p] = scales(w_post, w_post_dtype, plus_one_post, d);
    if (d < D && w_next != nullptr) wn[p] = scales(w_next, w_next_dtype, plus_one_next, d);
  }
  struct Row {
    float4 h[NP];
    RawY y[NP];
  };
  auto load = [&](int row, Row& b) __attribute__((always_inline)) {
    const size_t rb = static_cast<size_t>(row) * D;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int d = (p * 256 + tid) * 4;
      b.h[p] = float4{0.f, 0.f, 0.f, 0.f};
      b.y[p] = RawY{};
      if (d < D) {
        b.h[p] = *reinterpret_cast<const float4*>(residual + rb + d);
        if constexpr (!PLANES) b.y[p] = *reinterpret_cast<const RawY*>(y + rb + d);
      }
    }
    if constexpr (PLANES) {
      {
        const size_t plane = static_cast<size_t>(T) * D;
        float4 sum[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) sum[p] = float4{0.f, 0.f, 0.f, 0.f};
        for (int z0 = 0; z0 < planes; z0 += 4) {
          float4 part[4][NP];
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int p = 0; p < NP; ++p) {
              const int d = (p * 256 + tid) * 4;
              part[j][p] = (z0 + j < planes && d < D)
                               ? *reinterpret_cast<const float4*>(y_planes + (z0 + j) * plane + rb + d)
                               : float4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int p = 0; p < NP; ++p) {
              sum[p].x += part[j][p].x; sum[p].y += part[j][p].y; sum[p].z += part[j][p].z; sum[p].w += part[j][p].w;
            }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
          b.y[p].x = static_cast<uint32_t>(float_to_bf16(sum[p].x).bits) | (static_cast<uint32_t>(float_to_bf16(sum[p].y).bits) << 16);
          b.y[p].y = static_cast<uint32_t>(float_to_bf16(sum[p].z).bits) | (static_cast<uint32_t>(float_to_bf16(sum[p].w).bits) << 16);
        }
      }
    }
  };
  auto process = [&](int row, Row& b, float* red) __attribute__((always_inline)) {
    const size_t rb = static_cast<size_t>(row) * D;
    float4 yv[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      if constexpr (sizeof(YT) == 4) yv[p] = b.y[p];
      else yv[p] = float4{__uint_as_float(b.y[p].x << 16), __uint_as_float(b.y[p].x & 0xffff0000u),
                          __uint_as_float(b.y[p].y << 16), __uint_as_float(b.y[p].y & 0xffff0000u)};
    }
    float r = 1.f;
    if (w_post != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int p = 0; p < NP; ++p) ss += yv[p].x * yv[p].x + yv[p].y * yv[p].y + yv[p].z * yv[p].z + yv[p].w * yv[p].w;
      r = rsqrtf(block_sum(ss, red) / static_cast<float>(D) + eps_post);
    }
    float ss2 = 0.f;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int d = (p * 256 + tid) * 4;
      float4& h = b.h[p];
      if (w_post != nullptr) {
        h.x += yv[p].x * r * wp[p].x;
        h.y += yv[p].y * r * wp[p].y;
        h.z += yv[p].z * r * wp[p].z;
        h.w += yv[p].w * r * wp[p].w;
      } else {
        h.x += yv[p].x;
        h.y += yv[p].y;
        h.z += yv[p].z;
        h.w += yv[p].w;
      }
      ss2 += h.x * h.x + h.y * h.y + h.z * h.z + h.w * h.w;
      if (d < D) *reinterpret_cast<float4*>(residual + rb + d) = h;
    }
    if (w_next == nullptr) return;
    const float r2 = rsqrtf(block_sum(ss2, red + 8) / static_cast<float>(D) + eps_next);
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int d = (p * 256 + tid) * 4;
      if (d >= D) continue;
      const float4 h = b.h[p];
      const float o[4] = {h.x * r2 * wn[p].x, h.y * r2 * wn[p].y, h.z * r2 * wn[p].z, h.w * r2 * wn[p].w};
      if constexpr (sizeof(OT) == 4) {
        *reinterpret_cast<float4*>(out + rb + d) = float4{o[0], o[1], o[2], o[3]};
      } else {
        uint2 packed;
        packed.x = static_cast<uint32_t>(float_to_bf16(o[0]).bits) | (static_cast<uint32_t>(float_to_bf16(o[1]).bits) << 16);
        packed.y = static_cast<uint32_t>(float_to_bf16(o[2]).bits) | (static_cast<uint32_t>(float_to_bf16(o[3]).bits) << 16);
        *reinterpret_cast<uint2*>(out + rb + d) = packed;
      }
    }
  };
  // the group's rows in turn; the next row is asked for before the one at hand is worked on
  const int row0 = blockIdx.x * rows_per_group;
  const int nrows = T - row0 < rows_per_group ? T - row0 : rows_per_group;
  Row a, b;
  load(row0, a);
  for (int i = 0; i < nrows; i += 2) {
    if (i + 1 < nrows) load(row0 + i + 1, b);
    process(row0 + i, a, scratch);
    if (i + 1 < nrows) {
      if (i + 2 < nrows) load(row0 + i + 2, a);
      process(row0 + i + 1, b, scratch + 16);
    }
  }
}

// ------------------------------------------------------------------ rotary + cache write
// One block per (token, head) of a fused [T, (H + 2K) * hd] projection.
//   q heads: rotate, divide by query_scale, write back in place.
//   k heads: rotate, write into the key pages at slot_mapping[t] (pages in the layout of key_index()).
//   v heads: copy into the value pages (stored transposed: [page, head, hd, page_size]).
// Angles: pos / timescale[i] / scale_factor, pairs (i, i + hd/2).  simply/utils/position_encoding.py:83-110;
// the query scale comes after the rotation (simply/model_lib.py:2010-2019).
template <typename T>
__global__ void rope_cache_write_kernel(T* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions,
                                        const float* __restrict__ timescale /* [hd/2] or null = no rotation */,
                                        float inv_scale_factor, float q_div, const int64_t* __restrict__ slot_mapping,
                                        T* __restrict__ k_pages, T* __restrict__ v_pages, int H, int K, int hd,
                                        int page_size, const float* __restrict__ planes = nullptr, int count = 0,
                                        size_t plane_words = 0) {
  const int t = blockIdx.x, head = blockIdx.y;
  const int half = hd / 2;
  T* src = qkv + static_cast<size_t>(t) * row_stride + static_cast<size_t>(head) * hd;
  // planes: the projection has not been added up yet; its element is the sum of `count` planes [tokens][(H + 2K) hd]
  // in their order, rounded to T as the product's sum kernel would have left it in qkv
  const float* part = planes == nullptr ? nullptr
                                        : planes + (static_cast<size_t>(t) * (H + 2 * K) + head) * hd;
  auto at = [&](int i) __attribute__((always_inline)) {
    if (part == nullptr) return to_float(src[i]);
    float sum = 0.f;
    for (int z = 0; z < count; ++z) sum += part[z * plane_words + i];
    return to_float(from_float<T>(sum));
  };
  const float pos = static_cast<float>(positions[t]);
  if (head < H + K) {
    const bool is_q = head < H;
    T* dst = src;
    bool to_pages = false;
    int koff = 0;
    if (!is_q) {
      if (k_pages == nullptr) return;
      const int64_t slot = slot_mapping[t];
      if (slot < 0) return;
      const int64_t page = slot / page_size;
      koff = static_cast<int>(slot % page_size);
      dst = k_pages + (page * K + (head - H)) * page_size * hd;
      to_pages = true;
    }
    const bool tiled = to_pages && keys_tiled(page_size, hd);
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      const float x1 = at(i), x2 = at(i + half);
      float o1 = x1, o2 = x2;
      if (timescale != nullptr) {
        const float angle = pos / timescale[i] * inv_scale_factor;
        float s, c;
        sincosf(angle, &s, &c);
        o1 = x1 * c - x2 * s;
        o2 = x2 * c + x1 * s;
      }
      if (is_q) {
        o1 = o1 / q_div;
        o2 = o2 / q_div;
      }
      if (to_pages) {
        dst[key_index(tiled, page_size, hd, koff, i)] = from_float<T>(o1);
        dst[key_index(tiled, page_size, hd, koff, i + half)] = from_float<T>(o2);
      } else {
        dst[i] = from_float<T>(o1);
        dst[i + half] = from_float<T>(o2);
      }
    }
  } else {
    if (v_pages == nullptr) return;
    const int64_t slot = slot_mapping[t];
    if (slot < 0) return;
    const int64_t page = slot / page_size, off = slot % page_size;
    // value pages are [page, head, hd, page_size]: the keys of a page are contiguous for each dimension
    T* dst = v_pages + (page * K + (head - H - K)) * page_size * hd + off;
    for (int i = threadIdx.x; i < hd; i += blockDim.x) dst[static_cast<size_t>(i) * page_size] = from_float<T>(at(i));
  }
}

// The same for many tokens: one block per token, which works out the sines and cosines of the token's angles once
// for all heads (hd / 2 <= kMaxHalf).
constexpr int kMaxHalf = 512;
template <typename T>
__global__ __launch_bounds__(256) void rope_cache_write_rows_kernel(
    T* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions, const float* __restrict__ timescale,
    float inv_scale_factor, float q_div, const int64_t* __restrict__ slot_mapping, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int H, int K, int hd, int page_size) {
  __shared__ float sn[kMaxHalf], cs[kMaxHalf];
  const int t = blockIdx.x, half = hd / 2;
  const float pos = static_cast<float>(positions[t]);
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float s = 0.f, c = 1.f;
    if (timescale != nullptr) sincosf(pos / timescale[i] * inv_scale_factor, &s, &c);
    sn[i] = s;
    cs[i] = c;
  }
  __syncthreads();
  T* row = qkv + static_cast<size_t>(t) * row_stride;
  const int64_t slot = slot_mapping != nullptr ? slot_mapping[t] : -1;
  const bool write = k_pages != nullptr && slot >= 0;
  const int64_t page = write ? slot / page_size : 0;
  const int koff = write ? static_cast<int>(slot % page_size) : 0;
  const bool tiled = keys_tiled(page_size, hd);
  for (int idx = threadIdx.x; idx < (H + K) * half; idx += blockDim.x) {
    const int head = idx / half, i = idx % half;
    T* src = row + static_cast<size_t>(head) * hd;
    const float x1 = to_float(src[i]), x2 = to_float(src[i + half]);
    const float o1 = x1 * cs[i] - x2 * sn[i], o2 = x2 * cs[i] + x1 * sn[i];
    if (head < H) {
      src[i] = from_float<T>(o1 / q_div);
      src[i + half] = from_float<T>(o2 / q_div);
    } else if (write) {
      T* dst = k_pages + (page * K + (head - H)) * page_size * hd;
      dst[key_index(tiled, page_size, hd, koff, i)] = from_float<T>(o1);
      dst[key_index(tiled, page_size, hd, koff, i + half)] = from_float<T>(o2);
    }
  }
  if (!write) return;
  // value pages are [page, head, hd, page_size]: the keys of a page are contiguous for each dimension
  const T* vsrc = row + static_cast<size_t>(H + K) * hd;
  T* vdst = v_pages + page * K * page_size * hd + koff;
  for (int idx = threadIdx.x; idx < K * hd; idx += blockDim.x) vdst[static_cast<size_t>(idx) * page_size] = vsrc[idx];
}

// The same for many tokens in bfloat16 with 16-byte accesses (hd a multiple of 16, 16-byte aligned rows and pages).
// The first rot_blocks blocks rotate the q and k heads of kRotTokens tokens each: sines and cosines once per token
// in LDS, then eight dimensions (and the eight that pair with them) per thread and step; keys go into the pages as
// 16-byte pieces (eight neighbouring dimensions of a key are neighbours in both page layouts).  The other blocks
// copy the v heads of kValTokens tokens each into the transposed value pages: a thread holds eight dimensions of
// all 16 tokens and, when their slots are one run inside a page that starts at a multiple of eight (a prompt's
// portion that starts at a page's edge), writes each dimension's 16 keys as two 16-byte pieces instead of 16
// scattered 2-byte ones.
constexpr int kRotTokens = 8, kValTokens = 16, kWideMaxHalf = 256;
// two floats rounded to bfloat16 (to nearest even, one instruction for both), the first in the low half
__device__ inline uint32_t pack_bf16(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  const bf16x2 p = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(uint32_t, p);
}
__global__ __launch_bounds__(256) void rope_cache_write_wide_kernel(
    bf16* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions, const float* __restrict__ timescale,
    float inv_scale_factor, float q_div, const int64_t* __restrict__ slot_mapping, bf16* __restrict__ k_pages,
    bf16* __restrict__ v_pages, int T, int H, int K, int hd, int page_size, int rot_blocks) {
  __shared__ float sn[kRotTokens * kWideMaxHalf], cs[kRotTokens * kWideMaxHalf];
  const int tid = threadIdx.x, half = hd / 2;
  if (static_cast<int>(blockIdx.x) < rot_blocks) {
    const int t0 = blockIdx.x * kRotTokens;
    const int nt = T - t0 < kRotTokens ? T - t0 : kRotTokens;
    const int groups = half / 8, per_token = (H + K) * groups;
    const bool tiled = keys_tiled(page_size, hd);
    // Six items a thread at a time (all that a thread has at the usual sizes), their loads asked for together: one
    // after the other they are six trips to memory in a row; and the first six before the sines and cosines are
    // computed, which takes as long as the loads are under way.  The query scale is a multiplication by the
    // reciprocal: a division per rotated value was a third of the arithmetic, which is most of a block's time
    // (timestamps: 8.9 of 10.6 us before, 6 of 7.7 after).
    constexpr int kBatch = 6;
    const float q_mul = 1.f / q_div;
    const int total = nt * per_token;
    struct Batch {
      uint4 av[kBatch], bv[kBatch];
      bf16* to1[kBatch];
      bf16* to2[kBatch];
      int jj[kBatch], ii[kBatch];
      float scale[kBatch];
      bool ok[kBatch];
    };
    auto ask = [&](int first, Batch& b) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int item = first + u * static_cast<int>(blockDim.x);
        b.ok[u] = item < total;
        const int it = b.ok[u] ? item : 0;
        const int j = it / per_token, head = (it % per_token) / groups, i = (it % groups) * 8;
        bf16* src = qkv + static_cast<size_t>(t0 + j) * row_stride + static_cast<size_t>(head) * hd + i;
        b.jj[u] = j;
        b.ii[u] = i;
        b.scale[u] = head < H ? q_mul : 1.f;
        b.to1[u] = src;
        b.to2[u] = src + half;
        if (head >= H) {
          const int64_t slot = k_pages != nullptr ? slot_mapping[t0 + j] : -1;
          if (slot < 0) {
            b.ok[u] = false;
          } else {
            const int koff = static_cast<int>(slot % page_size);
            bf16* page = k_pages + ((slot / page_size) * K + (head - H)) * page_size * hd;
            b.to1[u] = page + key_index(tiled, page_size, hd, koff, i);
            b.to2[u] = page + key_index(tiled, page_size, hd, koff, i + half);
          }
        }
        b.av[u] = *reinterpret_cast<const uint4*>(src);
        b.bv[u] = *reinterpret_cast<const uint4*>(src + half);
      }
    };
    auto rotate = [&](const Batch& b) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        if (!b.ok[u]) continue;
        const uint32_t aw[4] = {b.av[u].x, b.av[u].y, b.av[u].z, b.av[u].w}, bw[4] = {b.bv[u].x, b.bv[u].y, b.bv[u].z, b.bv[u].w};
        uint32_t o1[4], o2[4];
        const float* sj = sn + b.jj[u] * half + b.ii[u];
        const float* cj = cs + b.jj[u] * half + b.ii[u];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          float r1[2], r2[2];
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const float x1 = __uint_as_float(e ? aw[w] & 0xffff0000u : aw[w] << 16);
            const float x2 = __uint_as_float(e ? bw[w] & 0xffff0000u : bw[w] << 16);
            const float s = sj[2 * w + e], c = cj[2 * w + e];
            r1[e] = (x1 * c - x2 * s) * b.scale[u];
            r2[e] = (x2 * c + x1 * s) * b.scale[u];
          }
          o1[w] = pack_bf16(r1[0], r1[1]);
          o2[w] = pack_bf16(r2[0], r2[1]);
        }
        *reinterpret_cast<uint4*>(b.to1[u]) = uint4{o1[0], o1[1], o1[2], o1[3]};
        *reinterpret_cast<uint4*>(b.to2[u]) = uint4{o2[0], o2[1], o2[2], o2[3]};
      }
    };
    Batch batch;
    ask(tid, batch);
    for (int idx = tid; idx < nt * half; idx += blockDim.x) {
      float s = 0.f, c = 1.f;
      if (timescale != nullptr)
        sincosf(static_cast<float>(positions[t0 + idx / half]) / timescale[idx % half] * inv_scale_factor, &s, &c);
      sn[idx] = s;
      cs[idx] = c;
    }
    __syncthreads();
    rotate(batch);
    for (int first = tid + static_cast<int>(blockDim.x) * kBatch; first < total; first += blockDim.x * kBatch) {
      ask(first, batch);
      rotate(batch);
    }
    return;
  }
  if (v_pages == nullptr) return;
  const int t0 = (blockIdx.x - rot_blocks) * kValTokens;
  const int nt = T - t0 < kValTokens ? T - t0 : kValTokens;
  const int64_t slot0 = slot_mapping[t0];
  bool run = nt == kValTokens && slot0 >= 0 && slot0 % 8 == 0 && slot0 % page_size + kValTokens <= page_size;
  if (tid < nt && slot_mapping[t0 + tid] != slot0 + tid) run = false;
  run = __syncthreads_and(run);
  const int groups = hd / 8;
  for (int item = tid; item < K * groups; item += blockDim.x) {
    const int head = item / groups, d0 = (item % groups) * 8;
    const bf16* src = qkv + static_cast<size_t>(t0) * row_stride + static_cast<size_t>(H + K + head) * hd + d0;
    uint32_t x[kValTokens][4];
#pragma unroll
    for (int j = 0; j < kValTokens; ++j) {
      const uint4 v = j < nt ? *reinterpret_cast<const uint4*>(src + static_cast<size_t>(j) * row_stride) : uint4{0, 0, 0, 0};
      x[j][0] = v.x, x[j][1] = v.y, x[j][2] = v.z, x[j][3] = v.w;
    }
    if (run) {
      bf16* dst = v_pages + (((slot0 / page_size) * K + head) * hd + d0) * page_size + slot0 % page_size;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        uint32_t o[kValTokens / 2];
#pragma unroll
        for (int w = 0; w < kValTokens / 2; ++w) {
          const uint32_t lo = x[2 * w][e / 2], hi = x[2 * w + 1][e / 2];
          o[w] = e % 2 ? (lo >> 16) | (hi & 0xffff0000u) : (lo & 0xffffu) | (hi << 16);
        }
        uint4* to = reinterpret_cast<uint4*>(dst + static_cast<size_t>(e) * page_size);
        to[0] = uint4{o[0], o[1], o[2], o[3]};
        to[1] = uint4{o[4], o[5], o[6], o[7]};
      }
    } else {
#pragma unroll
      for (int j = 0; j < kValTokens; ++j) {
        if (j >= nt) continue;
        const int64_t slot = slot_mapping[t0 + j];
        if (slot < 0) continue;
        uint16_t* dst = reinterpret_cast<uint16_t*>(v_pages) + (((slot / page_size) * K + head) * hd + d0) * page_size +
                        slot % page_size;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          dst[static_cast<size_t>(e) * page_size] = static_cast<uint16_t>(e % 2 ? x[j][e / 2] >> 16 : x[j][e / 2] & 0xffffu);
      }
    }
  }
}

// Rotation alone, in place, on [T, n_heads, hd] rows of stride row_stride.
template <typename T>
__global__ void rope_kernel(T* __restrict__ x, int64_t row_stride, const int* __restrict__ positions,
                            const float* __restrict__ timescale, float inv_scale_factor, float div, int hd) {
  const int t = blockIdx.x, head = blockIdx.y, half = hd / 2;
  T* p = x + static_cast<size_t>(t) * row_stride + static_cast<size_t>(head) * hd;
  const float pos = static_cast<float>(positions[t]);
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float x1 = to_float(p[i]), x2 = to_float(p[i + half]);
    const float angle = pos / timescale[i] * inv_scale_factor;
    float s, c;
    sincosf(angle, &s, &c);
    p[i] = from_float<T>((x1 * c - x2 * s) / div);
    p[i + half] = from_float<T>((x2 * c + x1 * s) / div);
  }
}

// out[r, :] = x[index[r], :]
__global__ void gather_rows_kernel(const void* __restrict__ x, int x_dtype, const int* __restrict__ index,
                                   void* __restrict__ out, int out_dtype, int D) {
  const size_t src = static_cast<size_t>(index[blockIdx.x]) * D, dst = static_cast<size_t>(blockIdx.x) * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) store_f(out, out_dtype, dst + d, load_f(x, x_dtype, src + d));
}

// p[i] = value for i < n (32-bit words); stands in for a memset inside captured graphs.
__global__ void fill_u32_kernel(uint32_t* __restrict__ p, uint32_t value, int64_t n) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    p[i] = value;
}

// ------------------------------------------------------------------ decoding several steps without the host
// After a decode step and its sampling: records what was drawn as step *step_counter of this run, makes the drawn
// tokens the next step's input, and moves every request on by one position (its token's position, its
// descriptor's first position, its draw counter).  One block; B <= 1024.
__global__ void decode_advance_kernel(int B, int* __restrict__ step_counter, const int* __restrict__ sampled_tokens,
                                      const float* __restrict__ sampled_logprobs, int* __restrict__ tokens_in,
                                      int* __restrict__ positions, int* __restrict__ seq_meta,
                                      int* __restrict__ draw_counters, int* __restrict__ out_tokens,
                                      float* __restrict__ out_logprobs, int max_steps) {
  const int b = threadIdx.x;
  const int k = *step_counter;
  __syncthreads();
  if (b < B) {
    if (k < max_steps) {
      out_tokens[static_cast<size_t>(k) * B + b] = sampled_tokens[b];
      out_logprobs[static_cast<size_t>(k) * B + b] = sampled_logprobs[b];
    }
    tokens_in[b] = sampled_tokens[b];
    positions[b] += 1;
    seq_meta[4 * b + 3] += 1;
    draw_counters[b] += 1;
  }
  if (b == 0) *step_counter = k + 1;
}

// The same, and where the next token's keys go in up to kMaxSlotGroups cache groups (what decode_slots_kernel
// computes, for every group, from the positions just moved on): one launch between two decode steps instead of one
// and one per group.
constexpr int kMaxSlotGroups = 4;
struct SlotGroups {
  const int* table[kMaxSlotGroups];
  int table_stride[kMaxSlotGroups];
  int64_t* slot_mapping[kMaxSlotGroups];
  int count, page_size;
};
__global__ void decode_advance_slots_kernel(int B, int* __restrict__ step_counter, const int* __restrict__ sampled_tokens,
                                            const float* __restrict__ sampled_logprobs, int* __restrict__ tokens_in,
                                            int* __restrict__ positions, int* __restrict__ seq_meta,
                                            int* __restrict__ draw_counters, int* __restrict__ out_tokens,
                                            float* __restrict__ out_logprobs, int max_steps,
                                            const int* __restrict__ token_seq, SlotGroups groups) {
  const int b = threadIdx.x;
  const int k = *step_counter;
  __syncthreads();
  if (b < B) {
    if (k < max_steps) {
      out_tokens[static_cast<size_t>(k) * B + b] = sampled_tokens[b];
      out_logprobs[static_cast<size_t>(k) * B + b] = sampled_logprobs[b];
    }
    tokens_in[b] = sampled_tokens[b];
    const int pos = positions[b] + 1;
    positions[b] = pos;
    seq_meta[4 * b + 3] += 1;
    draw_counters[b] += 1;
    const int row = token_seq[b];
    for (int g = 0; g < groups.count; ++g) {
      const int page = groups.table[g][static_cast<size_t>(row) * groups.table_stride[g] + pos / groups.page_size];
      groups.slot_mapping[g][b] = static_cast<int64_t>(page) * groups.page_size + pos % groups.page_size;
    }
  }
  if (b == 0) *step_counter = k + 1;
}

// slot_mapping[b] = where the key of token b goes: page (from its request's block-table row) * page_size + offset
__global__ void decode_slots_kernel(int B, const int* __restrict__ positions, const int* __restrict__ token_seq,
                                    const int* __restrict__ block_table, int table_stride, int page_size,
                                    int64_t* __restrict__ slot_mapping) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int pos = positions[b];
  const int page = block_table[static_cast<size_t>(token_seq[b]) * table_stride + pos / page_size];
  slot_mapping[b] = static_cast<int64_t>(page) * page_size + pos % page_size;
}

static int row_threads(int D) {
  int t = 64;
  while (t < 1024 && t * 4 < D) t *= 2;
  return t;
}

}  // namespace sa

using namespace sa;

extern "C" int sa_embed(const void* table, int table_dtype, const int* tokens, float* out, int T, int D, int V,
                        float scale, int packed, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(table_dtype == kF32 || table_dtype == kBF16, "embed: unknown table dtype %d", table_dtype);
  SA_REQUIRE(T > 0 && D > 0 && V > 0, "embed: bad sizes T=%d D=%d V=%d", T, D, V);
  embed_kernel<<<T, row_threads(D), 0, stream>>>(table, table_dtype, tokens, out, D, V, scale, packed);
  return check_launch("embed");
}

extern "C" int sa_rmsnorm(const void* x, int x_dtype, int64_t x_stride, const void* w, int w_dtype, void* out,
                          int out_dtype, int64_t out_stride, int T, int D, float eps, int plus_one,
                          hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && D > 0, "rmsnorm: bad sizes T=%d D=%d", T, D);
  SA_REQUIRE(x_stride >= D && out_stride >= D, "rmsnorm: row strides %lld, %lld are below the width %d",
             (long long)x_stride, (long long)out_stride, D);
  rmsnorm_kernel<<<T, row_threads(D), 0, stream>>>(x, x_dtype, x_stride, w, w_dtype, out, out_dtype, out_stride, D,
                                                   eps, plus_one ? 1.f : 0.f);
  return check_launch("rmsnorm");
}

extern "C" int sa_add_rmsnorm(const void* y, int y_dtype, const void* w_post, int w_post_dtype, float eps_post,
                              int plus_one_post, float* residual, const void* w_next, int w_next_dtype,
                              float eps_next, int plus_one_next, void* out, int out_dtype, int T, int D,
                              hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(T > 0 && D > 0, "add_rmsnorm: bad sizes T=%d D=%d", T, D);
  SA_REQUIRE(w_next == nullptr || out != nullptr, "add_rmsnorm: a next norm needs an output");
  // many rows: a workgroup of four waves per row (or two rows)
  const auto aligned16 = [](const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  const int o_dtype = out != nullptr ? out_dtype : y_dtype;
  if (T >= 64 && D % 4 == 0 && D <= 5120 && aligned16(y) && aligned16(residual) && aligned16(out) &&
      aligned16(w_post) && aligned16(w_next)) {
    const float pp = plus_one_post ? 1.f : 0.f, pn = plus_one_next ? 1.f : 0.f;
    // two rows to a workgroup, the second asked for before the first is worked on, once there are rows enough
    // (2,048 rows: 14.3 us against 16.8 with one; 512 rows: 8.2 against 6.6)
    const int rpg = T >= 2048 ? 2 : 1;
#define SA_SPLIT(YT, OT, NP)                                                                                       \
  add_rmsnorm_split_kernel<YT, OT, NP><<<(T + rpg - 1) / rpg, 256, 0, stream>>>(                                   \
      static_cast<const YT*>(y), w_post, w_post_dtype, eps_post, pp, residual, w_next, w_next_dtype, eps_next, pn, \
      static_cast<OT*>(out), T, D, rpg, nullptr, 0)
#define SA_SPLIT_N(YT, OT)            \
  do {                                \
    if (D <= 2048) SA_SPLIT(YT, OT, 2); \
    else if (D <= 3072) SA_SPLIT(YT, OT, 3); \
    else if (D <= 4096) SA_SPLIT(YT, OT, 4); \
    else SA_SPLIT(YT, OT, 5);         \
  } while (0)
    if (y_dtype == kBF16 && o_dtype == kBF16) SA_SPLIT_N(bf16, bf16);
    else if (y_dtype == kBF16) SA_SPLIT_N(bf16, float);
    else if (o_dtype == kBF16) SA_SPLIT_N(float, bf16);
    else SA_SPLIT_N(float, float);
#undef SA_SPLIT_N
#undef SA_SPLIT
    return check_launch("add_rmsnorm");
  }
  add_rmsnorm_kernel<<<T, row_threads(D), 0, stream>>>(y, y_dtype, w_post, w_post_dtype, eps_post,
                                                       plus_one_post ? 1.f : 0.f, residual, w_next, w_next_dtype,
                                                       eps_next, plus_one_next ? 1.f : 0.f, out, out_dtype, D, nullptr);
  return check_launch("add_rmsnorm");
}

extern "C" int sa_add_rmsnorm_rows(const void* y, int y_dtype, const void* w_post, int w_post_dtype, float eps_post,
                                   int plus_one_post, const float* residual, const void* w_next, int w_next_dtype,
                                   float eps_next, int plus_one_next, void* out, int out_dtype, const int* index, int R,
                                   int D, hipStream_t stream) {
  if (R == 0) return 0;
  SA_REQUIRE(R > 0 && D > 0 && index != nullptr && w_next != nullptr && out != nullptr && y != nullptr &&
                 residual != nullptr,
             "add_rmsnorm_rows: bad arguments (R=%d D=%d)", R, D);
  add_rmsnorm_kernel<<<R, row_threads(D), 0, stream>>>(y, y_dtype, w_post, w_post_dtype, eps_post,
                                                       plus_one_post ? 1.f : 0.f, const_cast<float*>(residual), w_next,
                                                       w_next_dtype, eps_next, plus_one_next ? 1.f : 0.f, out,
                                                       out_dtype, D, index);
  return check_launch("add_rmsnorm_rows");
}

extern "C" int sa_add_rmsnorm_planes(const float* y_planes, int planes, const void* w_post, int w_post_dtype,
                                     float eps_post, int plus_one_post, float* residual, const void* w_next,
                                     int w_next_dtype, float eps_next, int plus_one_next, void* out, int out_dtype,
                                     int T, int D, hipStream_t stream) {
  if (T == 0) return 0;
  const auto aligned16 = [](const void* p) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  SA_REQUIRE(T > 0 && D > 0 && planes >= 1 && y_planes != nullptr, "add_rmsnorm_planes: bad sizes T=%d D=%d planes=%d",
             T, D, planes);
  SA_REQUIRE(D % 4 == 0 && D <= 5120 && aligned16(y_planes) && aligned16(residual) && aligned16(out) &&
                 aligned16(w_post) && aligned16(w_next),
             "add_rmsnorm_planes: rows of a multiple of 4 and at most 5120 elements, 16-byte aligned; got D=%d", D);
  SA_REQUIRE(w_next == nullptr || out != nullptr, "add_rmsnorm_planes: a next norm needs an output");
  SA_REQUIRE(out == nullptr || out_dtype == kBF16 || out_dtype == kF32, "add_rmsnorm_planes: unknown output type");
  const float pp = plus_one_post ? 1.f : 0.f, pn = plus_one_next ? 1.f : 0.f;
#define SA_PLANES(OT, NP)                                                                                         \
  add_rmsnorm_split_kernel<bf16, OT, NP, true><<<T, 256, 0, stream>>>(nullptr, w_post, w_post_dtype, eps_post, pp,       \
                                                                residual, w_next, w_next_dtype, eps_next, pn,      \
                                                                static_cast<OT*>(out), T, D, 1, y_planes, planes)
#define SA_PLANES_N(OT)              \
  do {                               \
    if (D <= 2048) SA_PLANES(OT, 2); \
    else if (D <= 3072) SA_PLANES(OT, 3); \
    else if (D <= 4096) SA_PLANES(OT, 4); \
    else SA_PLANES(OT, 5);           \
  } while (0)
  if (out != nullptr && out_dtype == kF32) SA_PLANES_N(float);
  else SA_PLANES_N(bf16);
#undef SA_PLANES_N
#undef SA_PLANES
  return check_launch("add_rmsnorm_planes");
}

extern "C" int sa_rope_cache_write(void* qkv, int dtype, int64_t row_stride, const int* positions,
                                   const float* timescale, float scale_factor, float q_div,
                                   const int64_t* slot_mapping, void* k_pages, void* v_pages, int T, int H, int K,
                                   int hd, int page_size, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(hd > 0 && hd % 2 == 0, "rope_cache_write: head size %d must be even", hd);
  SA_REQUIRE(H >= 0 && K >= 0 && H + 2 * K > 0, "rope_cache_write: bad head counts H=%d K=%d", H, K);
  SA_REQUIRE(row_stride >= static_cast<int64_t>(H + 2 * K) * hd, "rope_cache_write: row stride %lld is too small",
             (long long)row_stride);
  SA_REQUIRE(page_size > 0 && scale_factor > 0.f && q_div > 0.f, "rope_cache_write: bad page size, scale factor or query scale");
  SA_REQUIRE((k_pages == nullptr) == (v_pages == nullptr) && (k_pages == nullptr || slot_mapping != nullptr),
             "rope_cache_write: key pages, value pages and slots come together");
  auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (T >= 256 && dtype == kBF16 && hd % 16 == 0 && hd / 2 <= kWideMaxHalf && row_stride % 8 == 0 && aligned16(qkv) &&
      aligned16(k_pages) && aligned16(v_pages)) {
    const int rot_blocks = (T + kRotTokens - 1) / kRotTokens;
    const int val_blocks = v_pages != nullptr && K > 0 ? (T + kValTokens - 1) / kValTokens : 0;
    rope_cache_write_wide_kernel<<<rot_blocks + val_blocks, 256, 0, stream>>>(
        static_cast<bf16*>(qkv), row_stride, positions, timescale, 1.f / scale_factor, q_div, slot_mapping,
        static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), T, H, K, hd, page_size, rot_blocks);
    return check_launch("rope_cache_write");
  }
  if (T >= 256 && hd / 2 <= kMaxHalf) {  // many tokens (a block for every compute unit): a block per token
    if (dtype == kF32)
      rope_cache_write_rows_kernel<float><<<T, 256, 0, stream>>>(static_cast<float*>(qkv), row_stride, positions,
                                                                 timescale, 1.f / scale_factor, q_div, slot_mapping,
                                                                 static_cast<float*>(k_pages),
                                                                 static_cast<float*>(v_pages), H, K, hd, page_size);
    else if (dtype == kBF16)
      rope_cache_write_rows_kernel<bf16><<<T, 256, 0, stream>>>(static_cast<bf16*>(qkv), row_stride, positions,
                                                                timescale, 1.f / scale_factor, q_div, slot_mapping,
                                                                static_cast<bf16*>(k_pages),
                                                                static_cast<bf16*>(v_pages), H, K, hd, page_size);
    else
      SA_REQUIRE(false, "rope_cache_write: unknown dtype %d", dtype);
    return check_launch("rope_cache_write");
  }
  const dim3 grid(T, H + 2 * K);
  const int threads = hd / 2 >= 128 ? 128 : 64;
  if (dtype == kF32)
    rope_cache_write_kernel<float><<<grid, threads, 0, stream>>>(static_cast<float*>(qkv), row_stride, positions,
                                                                 timescale, 1.f / scale_factor, q_div, slot_mapping,
                                                                 static_cast<float*>(k_pages),
                                                                 static_cast<float*>(v_pages), H, K, hd, page_size);
  else if (dtype == kBF16)
    rope_cache_write_kernel<bf16><<<grid, threads, 0, stream>>>(static_cast<bf16*>(qkv), row_stride, positions,
                                                                timescale, 1.f / scale_factor, q_div, slot_mapping,
                                                                static_cast<bf16*>(k_pages),
                                                                static_cast<bf16*>(v_pages), H, K, hd, page_size);
  else
    SA_REQUIRE(false, "rope_cache_write: unknown dtype %d", dtype);
  return check_launch("rope_cache_write");
}

extern "C" int sa_rope_cache_write_planes(const float* planes, int count, void* qkv, int64_t row_stride,
                                          const int* positions, const float* timescale, float scale_factor,
                                          float q_div, const int64_t* slot_mapping, void* k_pages, void* v_pages,
                                          int T, int H, int K, int hd, int page_size, hipStream_t stream) {
  if (T == 0) return 0;
  SA_REQUIRE(planes != nullptr && count >= 1, "rope_cache_write_planes: no planes");
  SA_REQUIRE(hd > 0 && hd % 2 == 0, "rope_cache_write: head size %d must be even", hd);
  SA_REQUIRE(H >= 0 && K >= 0 && H + 2 * K > 0, "rope_cache_write: bad head counts H=%d K=%d", H, K);
  SA_REQUIRE(row_stride >= static_cast<int64_t>(H + 2 * K) * hd, "rope_cache_write: row stride %lld is too small",
             (long long)row_stride);
  SA_REQUIRE(page_size > 0 && scale_factor > 0.f && q_div > 0.f, "rope_cache_write: bad page size, scale factor or query scale");
  SA_REQUIRE((k_pages == nullptr) == (v_pages == nullptr) && (k_pages == nullptr || slot_mapping != nullptr),
             "rope_cache_write: key pages, value pages and slots come together");
  const dim3 grid(T, H + 2 * K);
  const int threads = hd / 2 >= 128 ? 128 : 64;
  rope_cache_write_kernel<bf16><<<grid, threads, 0, stream>>>(
      static_cast<bf16*>(qkv), row_stride, positions, timescale, 1.f / scale_factor, q_div, slot_mapping,
      static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), H, K, hd, page_size, planes, count,
      static_cast<size_t>(T) * (H + 2 * K) * hd);
  return check_launch("rope_cache_write_planes");
}

extern "C" int sa_rope(void* x, int dtype, int64_t row_stride, const int* positions, const float* timescale,
                       float scale_factor, float div, int T, int n_heads, int hd, hipStream_t stream) {
  if (T == 0 || n_heads == 0) return 0;
  SA_REQUIRE(hd > 0 && hd % 2 == 0, "rope: head size %d must be even", hd);
  SA_REQUIRE(timescale != nullptr && scale_factor > 0.f && div > 0.f, "rope: no timescales, or a bad scale");
  const dim3 grid(T, n_heads);
  const int threads = hd / 2 >= 128 ? 128 : 64;
  if (dtype == kF32)
    rope_kernel<float><<<grid, threads, 0, stream>>>(static_cast<float*>(x), row_stride, positions, timescale,
                                                     1.f / scale_factor, div, hd);
  else if (dtype == kBF16)
    rope_kernel<bf16><<<grid, threads, 0, stream>>>(static_cast<bf16*>(x), row_stride, positions, timescale,
                                                    1.f / scale_factor, div, hd);
  else
    SA_REQUIRE(false, "rope: unknown dtype %d", dtype);
  return check_launch("rope");
}

extern "C" int sa_gather_rows(const void* x, int x_dtype, const int* index, void* out, int out_dtype, int R, int D,
                              hipStream_t stream) {
  if (R == 0) return 0;
  gather_rows_kernel<<<R, row_threads(D), 0, stream>>>(x, x_dtype, index, out, out_dtype, D);
  return check_launch("gather_rows");
}

extern "C" int sa_fill_u32(void* p, uint32_t value, int64_t n, hipStream_t stream) {
  if (n == 0) return 0;
  const int64_t blocks = (n + 255) / 256;
  fill_u32_kernel<<<static_cast<int>(blocks > 4096 ? 4096 : blocks), 256, 0, stream>>>(static_cast<uint32_t*>(p),
                                                                                      value, n);
  return check_launch("fill_u32");
}

extern "C" int sa_decode_advance(int B, int* step_counter, const int* sampled_tokens, const float* sampled_logprobs,
                                 int* tokens_in, int* positions, int* seq_meta, int* draw_counters, int* out_tokens,
                                 float* out_logprobs, int max_steps, hipStream_t stream) {
  if (B == 0) return 0;
  SA_REQUIRE(B > 0 && B <= 1024 && max_steps > 0, "decode_advance: 1..1024 requests and a positive number of steps");
  int threads = 64;
  while (threads < B) threads *= 2;
  decode_advance_kernel<<<1, threads, 0, stream>>>(B, step_counter, sampled_tokens, sampled_logprobs, tokens_in,
                                                   positions, seq_meta, draw_counters, out_tokens, out_logprobs,
                                                   max_steps);
  return check_launch("decode_advance");
}

extern "C" int sa_decode_advance_slots(int B, int* step_counter, const int* sampled_tokens, const float* sampled_logprobs,
                                       int* tokens_in, int* positions, int* seq_meta, int* draw_counters, int* out_tokens,
                                       float* out_logprobs, int max_steps, const int* token_seq, int num_groups,
                                       const int* const* block_tables, const int* table_strides,
                                       int64_t* const* slot_mappings, int page_size, hipStream_t stream) {
  if (B == 0) return 0;
  SA_REQUIRE(B > 0 && B <= 1024 && max_steps > 0, "decode_advance: 1..1024 requests and a positive number of steps");
  SA_REQUIRE(num_groups >= 0 && num_groups <= kMaxSlotGroups && page_size > 0 && (num_groups == 0 || token_seq != nullptr),
             "decode_advance_slots: 0..%d cache groups, a positive page size", kMaxSlotGroups);
  SlotGroups groups{};
  groups.count = num_groups;
  groups.page_size = page_size;
  for (int g = 0; g < num_groups; ++g) {
    SA_REQUIRE(block_tables[g] != nullptr && slot_mappings[g] != nullptr && table_strides[g] > 0,
               "decode_advance_slots: group %d lacks a table or a slot mapping", g);
    groups.table[g] = block_tables[g];
    groups.table_stride[g] = table_strides[g];
    groups.slot_mapping[g] = slot_mappings[g];
  }
  int threads = 64;
  while (threads < B) threads *= 2;
  decode_advance_slots_kernel<<<1, threads, 0, stream>>>(B, step_counter, sampled_tokens, sampled_logprobs, tokens_in,
                                                         positions, seq_meta, draw_counters, out_tokens, out_logprobs,
                                                         max_steps, token_seq, groups);
  return check_launch("decode_advance_slots");
}

extern "C" int sa_decode_slots(int B, const int* positions, const int* token_seq, const int* block_table,
                               int table_stride, int page_size, int64_t* slot_mapping, hipStream_t stream) {
  if (B == 0) return 0;
  SA_REQUIRE(B > 0 && table_stride > 0 && page_size > 0, "decode_slots: bad sizes");
  decode_slots_kernel<<<(B + 63) / 64, 64, 0, stream>>>(B, positions, token_seq, block_table, table_stride, page_size,
                                                        slot_mapping);
  return check_launch("decode_slots");
}
