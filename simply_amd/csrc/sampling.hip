// Sampling from rows of 32-bit logits: greedy, temperature, top-k and top-p, one
// workgroup per row.
//
// simply/utils/sampling_lib.py:472-537: temperature == 0 or top_k == 1 is argmax
// with log-probability 0; otherwise the logits are divided by the temperature,
// masked by top-k and/or top-p (kept entries: simply/utils/sampling_lib.py:427-469)
// and a token is drawn from the categorical distribution, which
// jax.random.categorical does with the Gumbel-max trick; the log-probability is
// log_softmax(masked scaled logits)[token] (simply/utils/distributions.py:98-121).
//
// Random numbers are counter-based (Philox4x32-10) and keyed by the row's own
// seed and draw counter, so a request's tokens do not depend on which other
// requests share the batch.
#include "api.h"
#include "common.h"

namespace sa {

constexpr int kSampleThreads = 1024;
// what the rows of a call may ask for (sa_sample's modes): a draw at all, top-k, top-p
constexpr int kSampleDrawn = 1, kSampleTopK = 2, kSampleTopP = 4;

struct Philox4 {
  uint32_t v[4];
};

__host__ __device__ inline Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                 uint32_t k1) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = static_cast<uint64_t>(M0) * c0, p1 = static_cast<uint64_t>(M1) * c2;
    const uint32_t hi0 = static_cast<uint32_t>(p0 >> 32), lo0 = static_cast<uint32_t>(p0);
    const uint32_t hi1 = static_cast<uint32_t>(p1 >> 32), lo1 = static_cast<uint32_t>(p1);
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += W0; k1 += W1;
  }
  Philox4 o;
  o.v[0] = c0; o.v[1] = c1; o.v[2] = c2; o.v[3] = c3;
  return o;
}

// Gumbel noise for the four vocabulary entries 4 b .. 4 b + 3 (one generator block).
__device__ inline void gumbel_noise4(uint64_t seed, uint32_t counter, uint32_t block, float out[4]) {
  const Philox4 r = philox4x32_10(block, counter, 0u, 0u, static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32));
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float u = (static_cast<float>(r.v[j] >> 8) + 0.5f) * (1.0f / 16777216.0f);
    out[j] = -logf(-logf(u));
  }
}

// Maps a float to an unsigned key with the same order.
__device__ inline uint32_t ordered_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ inline float key_to_float(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

struct ArgMax {
  float v;
  int i;
};
__device__ inline ArgMax better(ArgMax a, ArgMax b) {
  // larger value wins, the lower index on ties (jnp.argmax returns the first maximum)
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}
__device__ inline ArgMax block_argmax(ArgMax a, ArgMax* scratch) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    ArgMax b;
    b.v = __shfl_xor(a.v, o, kWave);
    b.i = __shfl_xor(a.i, o, kWave);
    a = better(a, b);
  }
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, nw = blockDim.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = a;
  __syncthreads();
  ArgMax r = scratch[0];
  for (int w = 1; w < nw; ++w) r = better(r, scratch[w]);
  return r;
}
__device__ inline float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, nw = blockDim.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < nw; ++w) r = fmaxf(r, scratch[w]);
  return r;
}

// Finds, among the entries x (scaled logits) of one row that are >= `floor_key`, the
// key of the boundary entry, by radix selection from the most significant byte down:
//   by_mass == 0: the `target_count`-th largest entry;
//   by_mass == 1: the entry at which the mass exp(x - max) summed from the top first
//                 reaches `target_mass` (so the mass strictly above it is below it).
// Masses are accumulated as 64-bit fixed point so that the result does not depend on
// the order in which threads add.  Returns the key; all threads get it.
__device__ uint32_t radix_select(const float* __restrict__ row, int V, float inv_t, float max_scaled, int by_mass,
                                 uint64_t target, uint32_t floor_key, unsigned long long* hist /* [256] LDS */,
                                 uint32_t* shared_out /* [2] LDS */, unsigned long long* shared_above /* [1] LDS */) {
  uint32_t prefix = 0, prefix_mask = 0;
  unsigned long long above = 0;  // count or mass of entries whose key is above the current prefix range
  for (int shift = 24; shift >= 0; shift -= 8) {
    for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0ull;
    __syncthreads();
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float x = row[i] * inv_t;
      const uint32_t key = ordered_key(x);
      if (key < floor_key || (key & prefix_mask) != prefix) continue;
      unsigned long long w = 1ull;
      if (by_mass) w = static_cast<unsigned long long>(expf(x - max_scaled) * 4294967296.0f);
      atomicAdd(&hist[(key >> shift) & 0xffu], w);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned long long run = above;
      int chosen = 0;
      for (int b = 255; b >= 0; --b) {
        if (run + hist[b] >= target) {
          chosen = b;
          break;
        }
        run += hist[b];
        if (b == 0) chosen = 0;  // target beyond the total: take everything
      }
      shared_out[0] = static_cast<uint32_t>(chosen);
      *shared_above = run;
    }
    __syncthreads();
    prefix |= shared_out[0] << shift;
    prefix_mask |= 0xffu << shift;
    above = *shared_above;
    __syncthreads();
  }
  return prefix;
}

// The rows' largest entries, for kArgChunks equal parts of each row: one workgroup per (row, part), so that a row
// of a large vocabulary is read by many compute units instead of one.  sample_kernel picks among the parts.
constexpr int kArgChunks = 32, kArgThreads = 256;

// What the selection of a row's top-k and top-p boundaries in parts keeps per row, in 64-bit words: the histograms
// of the four passes by count and of the four by mass (added up over the parts with atomics, complete when the
// kernel that adds them has ended), the mass of the entries that top-k leaves, and the selection's state after
// 1 .. 4 choices (prefix of the key, count or mass above it) for both.
constexpr int kSelCount = 0, kSelMass = 4 * 256, kSelTotal = 8 * 256, kSelCountState = kSelTotal + 2,
              kSelMassState = kSelCountState + 10, kSelWords = kSelMassState + 10;
__device__ inline bool is_greedy(float temp, int k) { return temp == 0.f || k == 1; }
__device__ inline bool uses_top_k(float temp, int k) { return !is_greedy(temp, k) && k > 0; }
__device__ inline bool uses_top_p(float temp, int k, float p) { return !is_greedy(temp, k) && p < 1.f; }

// sel: null, or the rows' selection words, which are cleared here.
__global__ __launch_bounds__(kArgThreads) void argmax_parts_kernel(const float* __restrict__ logits, int64_t row_stride,
                                                                  int V, ArgMax* __restrict__ parts,
                                                                  unsigned long long* __restrict__ sel) {
  __shared__ ArgMax am_scratch[kArgThreads / kWave];
  const int r = blockIdx.x, c = blockIdx.y;
  if (sel != nullptr)
    for (int i = c * kArgThreads + threadIdx.x; i < kSelWords; i += kArgChunks * kArgThreads)
      sel[static_cast<size_t>(r) * kSelWords + i] = 0ull;
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const int len = ((V + kArgChunks - 1) / kArgChunks + 3) / 4 * 4;
  const int lo = c * len < V ? c * len : V, hi = lo + len < V ? lo + len : V;
  ArgMax a{-INFINITY, 0x7fffffff};
  if ((reinterpret_cast<uintptr_t>(row + lo) & 15u) == 0) {
    const float4* row4 = reinterpret_cast<const float4*>(row + lo);
    const int quads = (hi - lo) / 4;
    for (int b = threadIdx.x; b < quads; b += blockDim.x) {
      const float4 x = row4[b];
      const int i = lo + 4 * b;
      a = better(a, ArgMax{x.x, i});
      a = better(a, ArgMax{x.y, i + 1});
      a = better(a, ArgMax{x.z, i + 2});
      a = better(a, ArgMax{x.w, i + 3});
    }
    for (int i = lo + 4 * quads + threadIdx.x; i < hi; i += blockDim.x) a = better(a, ArgMax{row[i], i});
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) a = better(a, ArgMax{row[i], i});
  }
  a = block_argmax(a, am_scratch);
  if (threadIdx.x == 0) parts[static_cast<size_t>(r) * kArgChunks + c] = a;
}

// One choice of the selection (256 threads): from the complete histogram of a pass (bins of the key's next byte)
// and what lies above the prefix chosen so far, the bin in which the target is reached, going down from the top
// bin, and what lies above that bin (everything, with bin 0, if the target is beyond the total): what thread 0
// of radix_select does in a loop, as a suffix sum over the bins.
struct SelPos {
  uint32_t prefix;
  unsigned long long above;
};
__device__ inline SelPos choose_bin(const unsigned long long* __restrict__ hist, SelPos at, int pass,
                                    unsigned long long target, unsigned long long* scan /* [256] LDS */,
                                    int* chosen_s /* LDS */) {
  const int b = threadIdx.x;
  scan[b] = hist[b];
  if (b == 0) *chosen_s = -1;
  __syncthreads();
  for (int o = 1; o < 256; o <<= 1) {
    const unsigned long long v = b + o < 256 ? scan[b + o] : 0ull;
    __syncthreads();
    scan[b] += v;
    __syncthreads();
  }
  if (at.above + scan[b] >= target) atomicMax(chosen_s, b);  // true for every bin from the chosen one down
  __syncthreads();
  const int chosen = *chosen_s;
  SelPos out;
  out.prefix = at.prefix | (static_cast<uint32_t>(chosen < 0 ? 0 : chosen) << (24 - 8 * pass));
  out.above = at.above + (chosen < 0 ? scan[0] : chosen + 1 < 256 ? scan[chosen + 1] : 0ull);
  __syncthreads();
  return out;
}
// The state after `n` choices (1 .. 4): what an earlier kernel has stored after n - 1, and the choice from the
// histogram of pass n - 1.  Part 0 of the row stores it for the kernels that follow.
__device__ inline SelPos advance(unsigned long long* __restrict__ S, int hist_base, int state_base, int n,
                                 unsigned long long target, unsigned long long* scan, int* chosen_s) {
  SelPos at{0u, 0ull};
  if (n > 1) {
    at.prefix = static_cast<uint32_t>(S[state_base + 2 * (n - 1)]);
    at.above = S[state_base + 2 * (n - 1) + 1];
  }
  const SelPos out = choose_bin(S + hist_base + (n - 1) * 256, at, n - 1, target, scan, chosen_s);
  if (blockIdx.y == 0 && threadIdx.x == 0) {
    S[state_base + 2 * n] = out.prefix;
    S[state_base + 2 * n + 1] = out.above;
  }
  return out;
}
__device__ inline unsigned long long mass_of(float x, float mx) {
  return static_cast<unsigned long long>(expf(x - mx) * 4294967296.0f);
}

// Pass `pass` (0 .. 3) of a selection, one workgroup per (row, part): the histogram of the next byte of the keys of
// the part's entries whose key continues the prefix chosen so far, added to the row's.  by_mass 0: top-k (entries
// count 1); 1: top-p (entries count their mass, among those that top-k leaves).
__global__ __launch_bounds__(kArgThreads) void select_pass_kernel(const float* __restrict__ logits, int64_t row_stride,
                                                                 int V, const float* __restrict__ temperature,
                                                                 const int* __restrict__ top_k,
                                                                 const float* __restrict__ top_p,
                                                                 const ArgMax* __restrict__ parts,
                                                                 unsigned long long* __restrict__ sel, int pass,
                                                                 int by_mass) {
  __shared__ unsigned long long hist[256], scan[256];
  __shared__ int chosen_s;
  const int r = blockIdx.x, c = blockIdx.y;
  const float temp = temperature[r];
  const int k = top_k[r];
  const float p = top_p[r];
  if (by_mass ? !uses_top_p(temp, k, p) : !uses_top_k(temp, k)) return;
  unsigned long long* S = sel + static_cast<size_t>(r) * kSelWords;
  const float inv_t = 1.f / temp;
  float mx = -INFINITY;
  for (int j = 0; j < kArgChunks; ++j) mx = fmaxf(mx, parts[static_cast<size_t>(r) * kArgChunks + j].v * inv_t);
  uint32_t floor_key = 0u;
  unsigned long long target;
  if (by_mass) {
    if (uses_top_k(temp, k)) floor_key = static_cast<uint32_t>(S[kSelCountState + 2 * 4]);  // (the mass kernel's)
    target = static_cast<unsigned long long>(static_cast<double>(p) * static_cast<double>(S[kSelTotal]));
    if (target < 1ull) target = 1ull;
  } else {
    target = static_cast<unsigned long long>(k < V ? k : V);
  }
  SelPos at{0u, 0ull};
  if (pass > 0) at = advance(S, by_mass ? kSelMass : kSelCount, by_mass ? kSelMassState : kSelCountState, pass, target, scan, &chosen_s);
  const uint32_t mask = pass == 0 ? 0u : 0xffffffffu << (32 - 8 * pass);
  const int shift = 24 - 8 * pass;
  hist[threadIdx.x] = 0ull;
  __syncthreads();
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const int len = ((V + kArgChunks - 1) / kArgChunks + 3) / 4 * 4;
  const int lo = c * len < V ? c * len : V, hi = lo + len < V ? lo + len : V;
  for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    const float x = row[i] * inv_t;
    const uint32_t key = ordered_key(x);
    if (key < floor_key || (key & mask) != at.prefix) continue;
    atomicAdd(&hist[(key >> shift) & 0xffu], by_mass ? mass_of(x, mx) : 1ull);
  }
  __syncthreads();
  const unsigned long long mine = hist[threadIdx.x];
  if (mine != 0ull) atomicAdd(&S[(by_mass ? kSelMass : kSelCount) + pass * 256 + threadIdx.x], mine);
}

// Between the two selections, for the rows with top-p: the mass of the entries that top-k leaves (all, without
// top-k), added up over the parts.
__global__ __launch_bounds__(kArgThreads) void select_mass_kernel(const float* __restrict__ logits, int64_t row_stride,
                                                                 int V, const float* __restrict__ temperature,
                                                                 const int* __restrict__ top_k,
                                                                 const float* __restrict__ top_p,
                                                                 const ArgMax* __restrict__ parts,
                                                                 unsigned long long* __restrict__ sel) {
  __shared__ unsigned long long scan[256];
  __shared__ int chosen_s;
  const int r = blockIdx.x, c = blockIdx.y;
  const float temp = temperature[r];
  const int k = top_k[r];
  if (!uses_top_p(temp, k, top_p[r])) return;
  unsigned long long* S = sel + static_cast<size_t>(r) * kSelWords;
  const float inv_t = 1.f / temp;
  float mx = -INFINITY;
  for (int j = 0; j < kArgChunks; ++j) mx = fmaxf(mx, parts[static_cast<size_t>(r) * kArgChunks + j].v * inv_t);
  uint32_t floor_key = 0u;
  if (uses_top_k(temp, k))
    floor_key = advance(S, kSelCount, kSelCountState, 4, static_cast<unsigned long long>(k < V ? k : V), scan, &chosen_s).prefix;
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const int len = ((V + kArgChunks - 1) / kArgChunks + 3) / 4 * 4;
  const int lo = c * len < V ? c * len : V, hi = lo + len < V ? lo + len : V;
  unsigned long long local = 0ull;
  for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    const float x = row[i] * inv_t;
    if (ordered_key(x) >= floor_key) local += mass_of(x, mx);
  }
  scan[threadIdx.x] = local;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (static_cast<int>(threadIdx.x) < o) scan[threadIdx.x] += scan[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0 && scan[0] != 0ull) atomicAdd(&S[kSelTotal], scan[0]);
}

// For the rows that are sampled (a temperature), again one workgroup per (row, part): among the part's entries that
// top-k and top-p leave (sel null: only rows without them are served), the largest with its noise added and the
// part's share of the softmax sum.  The noise of an entry depends on the request's seed, its draw counter and the
// entry's number alone, so the parts draw what one workgroup would.
struct DrawPart {
  ArgMax best;
  float sum, unused;
};
// Whether a row is drawn in parts: its top-k and top-p, if it has them, must have been selected in parts (`selected`: the
// modes whose selection kernels have run).
__device__ inline bool drawn_in_parts(float temp, int k, float p, int selected) {
  return !is_greedy(temp, k) && (!uses_top_k(temp, k) || (selected & kSampleTopK)) &&
         (!uses_top_p(temp, k, p) || (selected & kSampleTopP));
}

__global__ __launch_bounds__(kArgThreads) void draw_parts_kernel(const float* __restrict__ logits, int64_t row_stride,
                                                                int V, const float* __restrict__ temperature,
                                                                const int* __restrict__ top_k,
                                                                const float* __restrict__ top_p,
                                                                const uint64_t* __restrict__ seed,
                                                                const int* __restrict__ counter,
                                                                const ArgMax* __restrict__ parts,
                                                                DrawPart* __restrict__ draws,
                                                                unsigned long long* __restrict__ sel, int selected) {
  __shared__ ArgMax am_scratch[kArgThreads / kWave];
  __shared__ float f_scratch[kArgThreads / kWave];
  __shared__ unsigned long long scan[256];
  __shared__ int chosen_s;
  const int r = blockIdx.x, c = blockIdx.y;
  const float temp = temperature[r];
  const int k = top_k[r];
  const float p = top_p[r];
  if (!drawn_in_parts(temp, k, p, selected)) return;
  const float inv_t = 1.f / temp;
  float mx = -INFINITY;
  for (int j = 0; j < kArgChunks; ++j) mx = fmaxf(mx, parts[static_cast<size_t>(r) * kArgChunks + j].v * inv_t);
  // entries whose key is >= floor_key stay
  uint32_t floor_key = 0u;
  if (selected != 0) {
    unsigned long long* S = sel + static_cast<size_t>(r) * kSelWords;
    if (uses_top_k(temp, k))
      floor_key = uses_top_p(temp, k, p)
                      ? static_cast<uint32_t>(S[kSelCountState + 2 * 4])  // (the mass kernel has stored it)
                      : advance(S, kSelCount, kSelCountState, 4, static_cast<unsigned long long>(k < V ? k : V), scan,
                                &chosen_s).prefix;
    if (uses_top_p(temp, k, p)) {
      unsigned long long target = static_cast<unsigned long long>(static_cast<double>(p) * static_cast<double>(S[kSelTotal]));
      if (target < 1ull) target = 1ull;
      const uint32_t p_key = advance(S, kSelMass, kSelMassState, 4, target, scan, &chosen_s).prefix;
      floor_key = p_key > floor_key ? p_key : floor_key;
    }
  }
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const int len = ((V + kArgChunks - 1) / kArgChunks + 3) / 4 * 4;
  const int lo = c * len < V ? c * len : V, hi = lo + len < V ? lo + len : V;
  const uint64_t sd = seed[r];
  const uint32_t ctr = static_cast<uint32_t>(counter[r]);
  ArgMax a{-INFINITY, 0x7fffffff};
  float sum = 0.f;
  // one generator block gives the noise of four consecutive entries (lo is a multiple of four)
  for (int b = lo / 4 + threadIdx.x; 4 * b < hi; b += blockDim.x) {
    float g[4];
    gumbel_noise4(sd, ctr, static_cast<uint32_t>(b), g);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = 4 * b + j;
      if (i >= hi) break;
      const float x = row[i] * inv_t;
      if (ordered_key(x) < floor_key) continue;
      sum += expf(x - mx);
      a = better(a, ArgMax{x + g[j], i});
    }
  }
  a = block_argmax(a, am_scratch);
  sum = block_sum(sum, f_scratch);
  if (threadIdx.x == 0) draws[static_cast<size_t>(r) * kArgChunks + c] = DrawPart{a, sum, 0.f};
}

// parts: what argmax_parts_kernel has left for the rows, or null (they read their rows themselves); draws: what
// draw_parts_kernel has left for the sampled rows (selected: the modes, top-k and top-p, that were selected in parts).
// SCORE: nothing is drawn; tokens holds a given token per row, and logprobs receives its log-probability under the
// row's temperature, top-k and top-p: 0 or kMasked for greedy rows (simply/utils/sampling_lib.py:550-558), kMasked
// for a token that the masks leave out (simply/utils/distributions.py:104-121).
constexpr float kMasked = -0.5f * 3.402823466e38f;  // simply/utils/common.py:543-551 for float32
template <bool SCORE>
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, int64_t row_stride, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const uint64_t* __restrict__ seed,
    const int* __restrict__ counter, int* __restrict__ tokens, float* __restrict__ logprobs,
    const ArgMax* __restrict__ parts, const DrawPart* __restrict__ draws, int selected) {
  __shared__ ArgMax am_scratch[kSampleThreads / kWave];
  __shared__ float f_scratch[kSampleThreads / kWave];
  __shared__ unsigned long long hist[256];
  __shared__ uint32_t sel_out[2];
  __shared__ unsigned long long sel_above;
  const int r = blockIdx.x;
  const float* row = logits + static_cast<size_t>(r) * row_stride;
  const float temp = temperature[r];
  const int k = top_k[r];
  const float p = top_p[r];

  // rows are read four entries at a time where their address allows it (every row does if the stride is a
  // multiple of four); the few entries before and after the aligned part are read singly
  const int head = static_cast<int>((4 - (reinterpret_cast<uintptr_t>(row) / 4) % 4) % 4) < V
                       ? static_cast<int>((4 - (reinterpret_cast<uintptr_t>(row) / 4) % 4) % 4) : V;
  const int quads = (V - head) / 4;
  const float4* row4 = reinterpret_cast<const float4*>(row + head);
  const int tail0 = head + 4 * quads;

  if (temp == 0.f || k == 1) {
    ArgMax a{-INFINITY, 0x7fffffff};
    if (parts != nullptr) {
      if (threadIdx.x < kArgChunks) a = parts[static_cast<size_t>(r) * kArgChunks + threadIdx.x];
      a = block_argmax(a, am_scratch);
      if (threadIdx.x == 0) {
        if (SCORE) {
          logprobs[r] = tokens[r] == a.i ? 0.f : kMasked;
        } else {
          tokens[r] = a.i;
          logprobs[r] = 0.f;
        }
      }
      return;
    }
    for (int i = threadIdx.x; i < head; i += blockDim.x) a = better(a, ArgMax{row[i], i});
    for (int b = threadIdx.x; b < quads; b += blockDim.x) {
      const float4 x = row4[b];
      const int i = head + 4 * b;
      a = better(a, ArgMax{x.x, i});
      a = better(a, ArgMax{x.y, i + 1});
      a = better(a, ArgMax{x.z, i + 2});
      a = better(a, ArgMax{x.w, i + 3});
    }
    for (int i = tail0 + threadIdx.x; i < V; i += blockDim.x) a = better(a, ArgMax{row[i], i});
    a = block_argmax(a, am_scratch);
    if (threadIdx.x == 0) {
      if (SCORE) {
        logprobs[r] = tokens[r] == a.i ? 0.f : kMasked;
      } else {
        tokens[r] = a.i;
        logprobs[r] = 0.f;
      }
    }
    return;
  }

  const float inv_t = 1.f / temp;
  if (!SCORE && draws != nullptr && drawn_in_parts(temp, k, p, selected)) {
    float mx = -INFINITY, sum = 0.f;
    ArgMax a{-INFINITY, 0x7fffffff};
    if (threadIdx.x < kArgChunks) {
      const DrawPart d = draws[static_cast<size_t>(r) * kArgChunks + threadIdx.x];
      a = d.best;
      sum = d.sum;
      mx = parts[static_cast<size_t>(r) * kArgChunks + threadIdx.x].v * inv_t;
    }
    a = block_argmax(a, am_scratch);
    mx = block_max(mx, f_scratch);
    sum = block_sum(sum, f_scratch);
    if (threadIdx.x == 0) {
      tokens[r] = a.i;
      logprobs[r] = row[a.i] * inv_t - mx - logf(sum);
    }
    return;
  }
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < head; i += blockDim.x) mx = fmaxf(mx, row[i] * inv_t);
  for (int b = threadIdx.x; b < quads; b += blockDim.x) {
    const float4 x = row4[b];
    mx = fmaxf(fmaxf(mx, x.x * inv_t), fmaxf(fmaxf(x.y * inv_t, x.z * inv_t), x.w * inv_t));
  }
  for (int i = tail0 + threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, row[i] * inv_t);
  mx = block_max(mx, f_scratch);

  // Entries whose key is >= floor_key stay (the mask of the reference, as a threshold).
  uint32_t floor_key = 0u;
  if (k > 0) {
    const uint64_t kk = static_cast<uint64_t>(k < V ? k : V);
    floor_key = radix_select(row, V, inv_t, mx, 0, kk, 0u, hist, sel_out, &sel_above);
  }
  if (p < 1.f) {
    // total mass of the entries that are still in (after top-k, whose softmax is renormalised over them)
    __syncthreads();
    if (threadIdx.x == 0) hist[0] = 0ull;
    __syncthreads();
    unsigned long long local = 0ull;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float x = row[i] * inv_t;
      if (ordered_key(x) >= floor_key) local += static_cast<unsigned long long>(expf(x - mx) * 4294967296.0f);
    }
    atomicAdd(&hist[0], local);
    __syncthreads();
    const unsigned long long total = hist[0];
    __syncthreads();
    // keep while the mass before an entry is < p * total: the boundary entry is the first at which the
    // running mass reaches p * total (it is kept, simply/utils/sampling_lib.py:434-441)
    unsigned long long target = static_cast<unsigned long long>(static_cast<double>(p) * static_cast<double>(total));
    if (target < 1ull) target = 1ull;
    const uint32_t p_key = radix_select(row, V, inv_t, mx, 1, target, floor_key, hist, sel_out, &sel_above);
    floor_key = p_key > floor_key ? p_key : floor_key;
  }

  if (SCORE) {
    float sum = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float x = row[i] * inv_t;
      if (ordered_key(x) >= floor_key) sum += expf(x - mx);
    }
    sum = block_sum(sum, f_scratch);
    if (threadIdx.x == 0) {
      const int given = tokens[r];
      const float x = (given >= 0 && given < V) ? row[given] * inv_t : -INFINITY;
      logprobs[r] = (given >= 0 && given < V && ordered_key(x) >= floor_key) ? x - mx - logf(sum) : kMasked;
    }
    return;
  }
  if (SCORE) {
    float sum = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float x = row[i] * inv_t;
      if (ordered_key(x) >= floor_key) sum += expf(x - mx);
    }
    sum = block_sum(sum, f_scratch);
    if (threadIdx.x == 0) {
      const int given = tokens[r];
      const float x = (given >= 0 && given < V) ? row[given] * inv_t : -INFINITY;
      logprobs[r] = (given >= 0 && given < V && ordered_key(x) >= floor_key) ? x - mx - logf(sum) : kMasked;
    }
    return;
  }
  const uint64_t sd = seed[r];
  const uint32_t ctr = static_cast<uint32_t>(counter[r]);
  ArgMax a{-INFINITY, 0x7fffffff};
  float sum = 0.f;
  // one generator block gives the noise of four consecutive entries
  for (int b = threadIdx.x; 4 * b < V; b += blockDim.x) {
    float g[4];
    gumbel_noise4(sd, ctr, static_cast<uint32_t>(b), g);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = 4 * b + j;
      if (i >= V) break;
      const float x = row[i] * inv_t;
      if (ordered_key(x) < floor_key) continue;
      sum += expf(x - mx);
      a = better(a, ArgMax{x + g[j], i});
    }
  }
  a = block_argmax(a, am_scratch);
  sum = block_sum(sum, f_scratch);
  if (threadIdx.x == 0) {
    tokens[r] = a.i;
    logprobs[r] = row[a.i] * inv_t - mx - logf(sum);
  }
}

}  // namespace sa

using namespace sa;

extern "C" int sa_sample(const float* logits, int64_t row_stride, int R, int V, const float* temperature,
                         const int* top_k, const float* top_p, const uint64_t* seed, const int* counter, int* tokens,
                         float* logprobs, int modes, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  if (R == 0) return 0;
  SA_REQUIRE(R > 0 && V > 0 && row_stride >= V, "sample: bad sizes R=%d V=%d stride=%lld", R, V,
             (long long)row_stride);
  // Large vocabularies: the rows are worked on in kArgChunks parts by as many workgroups, in several kernels (a
  // row of 256,000 logits in one workgroup took 40 us for the argmax, 150 us for a draw, 350-600 us with top-k
  // and top-p).  modes says what the rows may ask for, so that kernels nobody needs are not launched.
  ArgMax* parts = nullptr;
  DrawPart* draws = nullptr;
  unsigned long long* sel = nullptr;
  const bool any_drawn = (modes & (kSampleDrawn | kSampleTopK | kSampleTopP)) != 0;
  const bool any_selection = (modes & (kSampleTopK | kSampleTopP)) != 0;
  int selected = 0;  // the selections that run in parts
  const int64_t need = static_cast<int64_t>(R) * (kArgChunks * static_cast<int64_t>(sizeof(ArgMax) + sizeof(DrawPart)) +
                                                  kSelWords * static_cast<int64_t>(sizeof(unsigned long long)));
  if (V >= 16384 && workspace != nullptr && workspace_bytes >= need) {
    draws = static_cast<DrawPart*>(workspace);
    parts = reinterpret_cast<ArgMax*>(draws + static_cast<size_t>(R) * kArgChunks);
    if (any_selection) {
      sel = reinterpret_cast<unsigned long long*>(parts + static_cast<size_t>(R) * kArgChunks);
      selected = modes & (kSampleTopK | kSampleTopP);
    }
    const dim3 grid(R, kArgChunks);
    argmax_parts_kernel<<<grid, kArgThreads, 0, stream>>>(logits, row_stride, V, parts, sel);
    if (modes & kSampleTopK)
      for (int pass = 0; pass < 4; ++pass)
        select_pass_kernel<<<grid, kArgThreads, 0, stream>>>(logits, row_stride, V, temperature, top_k, top_p, parts,
                                                             sel, pass, 0);
    if (modes & kSampleTopP) {
      select_mass_kernel<<<grid, kArgThreads, 0, stream>>>(logits, row_stride, V, temperature, top_k, top_p, parts, sel);
      for (int pass = 0; pass < 4; ++pass)
        select_pass_kernel<<<grid, kArgThreads, 0, stream>>>(logits, row_stride, V, temperature, top_k, top_p, parts,
                                                             sel, pass, 1);
    }
    if (any_drawn)
      draw_parts_kernel<<<grid, kArgThreads, 0, stream>>>(logits, row_stride, V, temperature, top_k, top_p, seed,
                                                          counter, parts, draws, sel, selected);
    else
      draws = nullptr;
    if (check_launch("sample (parts)")) return 1;
  }
  sample_kernel<false><<<R, kSampleThreads, 0, stream>>>(logits, row_stride, V, temperature, top_k, top_p, seed, counter,
                                                         tokens, logprobs, parts, draws, selected);
  return check_launch("sample");
}

extern "C" int sa_score(const float* logits, int64_t row_stride, int R, int V, const float* temperature,
                        const int* top_k, const float* top_p, const int* tokens, float* scores, hipStream_t stream) {
  if (R == 0) return 0;
  SA_REQUIRE(R > 0 && V > 0 && row_stride >= V, "score: bad sizes R=%d V=%d stride=%lld", R, V, (long long)row_stride);
  sample_kernel<true><<<R, kSampleThreads, 0, stream>>>(logits, row_stride, V, temperature, top_k, top_p, nullptr, nullptr,
                                                        const_cast<int*>(tokens), scores, nullptr, nullptr, 0);
  return check_launch("score");
}

// Host-side copy of the generator, for tests of the kernel's random stream.
extern "C" void sa_philox4x32_10(const uint32_t* counter4, const uint32_t* key2, uint32_t* out4) {
  const Philox4 r = philox4x32_10(counter4[0], counter4[1], counter4[2], counter4[3], key2[0], key2[1]);
  for (int i = 0; i < 4; ++i) out4[i] = r.v[i];
}
