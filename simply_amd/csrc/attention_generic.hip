// Paged attention for every size and both element types: one workgroup per
// (query token, key/value head), all arithmetic in 32-bit on the vector ALU.
//
// A query at absolute position p of its request sees the keys [lo, p] with
// lo = max(0, p - window + 1) for a windowed layer and 0 otherwise; the keys of
// this step have been written to the pages before the launch.  Keys are taken
// in chunks of 64 aligned to absolute positions, in increasing order, with a
// running maximum, sum and output (online softmax).  The order of every sum is
// fixed by p alone, so the result for a token does not depend on how the tokens
// were cut into steps, on what else is in the batch, or on which pages hold the
// keys.
//
// Scores -> cap -> mask -> softmax -> values as in simply/model_lib.py:611-638
// and simply/kernels/ragged_paged_attention.py:222-249; query head h reads
// key/value head h / G (simply/kernels/ragged_paged_attention.py:214-215).
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kChunk = 64;     // keys per chunk
constexpr int kThreads = 256;  // 4 waves
constexpr int kMaxDimsPerThread = 2;  // head sizes up to 512

template <typename T>
__global__ __launch_bounds__(kThreads) void paged_attention_generic_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_seq,
    const int* __restrict__ positions, T* __restrict__ out, int64_t out_stride, int Kh, int G, int hd, int page_size,
    int window, float soft_cap) {
  extern __shared__ float smem[];
  float* q_s = smem;                      // [G][hd]
  float* s_s = q_s + G * hd;              // [G][kChunk] scores, then probabilities
  float* m_s = s_s + G * kChunk;          // [G] running maximum
  float* l_s = m_s + G;                   // [G] running sum
  float* a_s = l_s + G;                   // [G] rescale factor of this chunk
  int* page_s = reinterpret_cast<int*>(a_s + G);  // [kChunk] page of each key of the chunk

  const int t = blockIdx.x, kh = blockIdx.y, tid = threadIdx.x;
  const bool tiled = keys_tiled(page_size, hd);
  const int seq = token_seq[t];
  const int pos = positions[t];
  const int hi = pos + 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + static_cast<size_t>(seq) * table_stride;

  for (int i = tid; i < G * hd; i += kThreads) {
    const int g = i / hd, d = i % hd;
    q_s[i] = to_float(q[static_cast<size_t>(t) * q_stride + static_cast<size_t>(kh * G + g) * hd + d]);
  }
  for (int g = tid; g < G; g += kThreads) {
    m_s[g] = -INFINITY;
    l_s[g] = 0.f;
  }
  float acc[kMaxDimsPerThread][8];  // [dim slot][g within a tile of 8 heads]; G > 8 loops over head tiles
  // Heads are processed in tiles of 8 so that the accumulators stay in registers.
  for (int g0 = 0; g0 < G; g0 += 8) {
    const int gn = G - g0 < 8 ? G - g0 : 8;
#pragma unroll
    for (int s = 0; s < kMaxDimsPerThread; ++s)
#pragma unroll
      for (int g = 0; g < 8; ++g) acc[s][g] = 0.f;
    __syncthreads();

    for (int c0 = (lo / kChunk) * kChunk; c0 < hi; c0 += kChunk) {
      const int jlo = lo > c0 ? lo - c0 : 0;
      const int jhi = hi - c0 < kChunk ? hi - c0 : kChunk;
      if (tid < kChunk) {
        const int key = c0 + tid;
        page_s[tid] = (tid >= jlo && tid < jhi) ? table[key / page_size] : -1;
      }
      __syncthreads();
      // ---- scores: 4 threads per key, each over a quarter of the head size (interleaved)
      {
        const int j = tid / 4, part = tid % 4;
        const bool valid = j >= jlo && j < jhi;
        float dot[8];
#pragma unroll
        for (int g = 0; g < 8; ++g) dot[g] = 0.f;
        if (valid) {
          const int key = c0 + j;
          const T* kp = k_pages + (static_cast<size_t>(page_s[j]) * Kh + kh) * page_size * hd;
          const int kin = key % page_size;
          for (int d = part; d < hd; d += 4) {
            const float kv = to_float(kp[key_index(tiled, page_size, hd, kin, d)]);
#pragma unroll
            for (int g = 0; g < 8; ++g)
              if (g < gn) dot[g] = fmaf(q_s[(g0 + g) * hd + d], kv, dot[g]);
          }
        }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
          if (g < gn) {
            float s = dot[g];
            s += __shfl_xor(s, 1, kWave);
            s += __shfl_xor(s, 2, kWave);
            if (part == 0) {
              if (soft_cap > 0.f) s = soft_cap * tanhf(s / soft_cap);
              s_s[(g0 + g) * kChunk + j] = valid ? s : -INFINITY;
            }
          }
        }
      }
      __syncthreads();
      // ---- softmax update: wave w takes heads w, w + 4, ...
      {
        const int wave = tid / kWave, lane = tid % kWave;
        for (int g = wave; g < gn; g += kThreads / kWave) {
          const float s = s_s[(g0 + g) * kChunk + lane];
          const float m_old = m_s[g0 + g];
          const float m_new = fmaxf(m_old, wave_max(s));
          const float p = (lane >= jlo && lane < jhi) ? expf(s - m_new) : 0.f;
          const float sum = wave_sum(p);
          s_s[(g0 + g) * kChunk + lane] = p;
          if (lane == 0) {
            const float alpha = expf(m_old - m_new);  // 0 for the first chunk (m_old = -inf)
            a_s[g0 + g] = alpha;
            l_s[g0 + g] = l_s[g0 + g] * alpha + sum;
            m_s[g0 + g] = m_new;
          }
        }
      }
      __syncthreads();
      // ---- values: thread d accumulates output dimension d for every head of the tile
#pragma unroll
      for (int s = 0; s < kMaxDimsPerThread; ++s) {
        const int d = tid + s * kThreads;
        if (d < hd) {
#pragma unroll
          for (int g = 0; g < 8; ++g)
            if (g < gn) acc[s][g] *= a_s[g0 + g];
          for (int j = jlo; j < jhi; ++j) {
            const int key = c0 + j;
            const float v = to_float(
                v_pages[((static_cast<size_t>(page_s[j]) * Kh + kh) * hd + d) * page_size + key % page_size]);
#pragma unroll
            for (int g = 0; g < 8; ++g)
              if (g < gn) acc[s][g] = fmaf(s_s[(g0 + g) * kChunk + j], v, acc[s][g]);
          }
        }
      }
      __syncthreads();
    }
#pragma unroll
    for (int s = 0; s < kMaxDimsPerThread; ++s) {
      const int d = tid + s * kThreads;
      if (d < hd) {
#pragma unroll
        for (int g = 0; g < 8; ++g)
          if (g < gn)
            out[static_cast<size_t>(t) * out_stride + static_cast<size_t>(kh * G + g0 + g) * hd + d] =
                from_float<T>(acc[s][g] / l_s[g0 + g]);
      }
    }
  }
}

int paged_attention_generic(const void* q, int dtype, int64_t q_stride, const void* k_pages, const void* v_pages,
                            const int* block_table, int table_stride, const int* token_seq, const int* positions,
                            void* out, int64_t out_stride, int T, int H, int Kh, int hd, int page_size, int window,
                            float soft_cap, hipStream_t stream) {
  const int G = H / Kh;
  if (hd > kThreads * kMaxDimsPerThread) {
    set_error("paged_attention: head size %d is above the largest supported (%d)", hd, kThreads * kMaxDimsPerThread);
    return 1;
  }
  const size_t smem = sizeof(float) * (static_cast<size_t>(G) * hd + static_cast<size_t>(G) * kChunk + 3 * G) +
                      sizeof(int) * kChunk;
  if (smem > 64 * 1024) {
    set_error("paged_attention: %d query heads per key head at head size %d need %zu bytes of LDS (limit 65536)", G,
              hd, smem);
    return 1;
  }
  const dim3 grid(T, Kh);
  if (dtype == kF32)
    paged_attention_generic_kernel<float><<<grid, kThreads, smem, stream>>>(
        static_cast<const float*>(q), q_stride, static_cast<const float*>(k_pages),
        static_cast<const float*>(v_pages), block_table, table_stride, token_seq, positions, static_cast<float*>(out),
        out_stride, Kh, G, hd, page_size, window, soft_cap);
  else
    paged_attention_generic_kernel<bf16><<<grid, kThreads, smem, stream>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<const bf16*>(k_pages), static_cast<const bf16*>(v_pages),
        block_table, table_stride, token_seq, positions, static_cast<bf16*>(out), out_stride, Kh, G, hd, page_size,
        window, soft_cap);
  return check_launch("paged_attention_generic");
}

}  // namespace sa
