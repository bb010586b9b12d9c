// Sampling from float32 logits [R, V]: one block per row.
//
//   argmax        first maximal index (servelab/engine/sampler.py:23-24).
//   sample        temperature 0 => argmax; else a draw from
//                 softmax(logits / max(T, 1e-6)) (sampler.py:29,45), restricted
//                 to the top_k largest when top_k > 0 (sampler.py:30-35, top_p
//                 then ignored as there), else to the sorted prefix whose
//                 cumulative probability stays <= top_p, first entry always kept
//                 (sampler.py:36-44).
// The draw is Gumbel-max: argmax_i (logit_i / T + g_i), g_i = -log(-log(u_i)),
// which is an exact sample of the softmax and needs no normalisation.  u_i is a
// counter-based hash of (seed, draw, i): a request's stream depends only on its
// seed and how many tokens it has drawn, not on the batch it is in.  The
// reference draws from a host generator instead (sampler.py:11-13).
#include "common.h"

struct Best { float v; int i; };

__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ Best block_best(Best b, Best* scratch) {
#pragma unroll
  for (int o = SL_WAVE / 2; o > 0; o >>= 1) {
    Best other;
    other.v = __shfl_xor(b.v, o, SL_WAVE);
    other.i = __shfl_xor(b.i, o, SL_WAVE);
    b = better(b, other);
  }
  const int wave = threadIdx.x / SL_WAVE, lane = threadIdx.x % SL_WAVE;
  const int nwaves = blockDim.x / SL_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = b;
  __syncthreads();
  Best r = scratch[0];
  for (int i = 1; i < nwaves; ++i) r = better(r, scratch[i]);
  return r;
}

__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t draw, uint32_t i) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * (draw * 0x100000001B3ull + i + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return ((float)(z >> 40) + 0.5f) * (1.0f / 16777216.0f);     // in (0, 1)
}

// e^x for x <= 0 by the hardware's 2^x: the top-p search below evaluates it for
// every logit in each of its 32 passes, where the accurate expf was most of
// the kernel's time; the weights only decide where the cut falls.
__device__ __forceinline__ float weight_of(float x) {
  return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
}

// -ln(-ln u) for u in (0, 1) by the hardware's log2 (the draw evaluates it once
// per kept logit; the accurate logf pair was most of a plain draw's time)
__device__ __forceinline__ float gumbel_of(float u) {
  const float ln2 = 0.6931471805599453f;
  return -ln2 * __builtin_amdgcn_logf(-ln2 * __builtin_amdgcn_logf(u));
}

// order-preserving map float -> uint32
__device__ __forceinline__ uint32_t key_of(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float float_of(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// f(value, index) for every logit of a row, four at a time with 16-byte loads
// where the row allows it.  One workgroup walks a whole row, so the time of a
// pass is the time of its loads.
template <class F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ x, int V, F f) {
  struct __attribute__((aligned(16))) f4 { float v[4]; };
  int done = 0;
  if (((uintptr_t)x % 16) == 0) {
    const int V4 = V / 4;
    for (int q = threadIdx.x; q < V4; q += blockDim.x) {
      const f4 v = ((const f4*)x)[q];
#pragma unroll
      for (int j = 0; j < 4; ++j) f(v.v[j], 4 * q + j);
    }
    done = V4 * 4;
  }
  for (int i = done + threadIdx.x; i < V; i += blockDim.x) f(x[i], i);
}

// Sums of WAYS values over the block, in a fixed order.
template <int WAYS>
__device__ __forceinline__ void block_sums(float (&v)[WAYS], float (*scratch)[WAYS]) {
  const int wave = threadIdx.x / SL_WAVE, lane = threadIdx.x % SL_WAVE;
  const int nwaves = (blockDim.x + SL_WAVE - 1) / SL_WAVE;
#pragma unroll
  for (int j = 0; j < WAYS; ++j) v[j] = wave_sum(v[j]);
  __syncthreads();
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < WAYS; ++j) scratch[wave][j] = v[j];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < WAYS; ++j) {
    float t = 0.f;
    for (int i = 0; i < nwaves; ++i) t += scratch[i][j];
    v[j] = t;
  }
}

// The cut of top-k and of top-p is found by a search over the ordered bit
// patterns of the logits.  Each pass over the row tests WAYS thresholds at
// once, which narrows the range to an eighth: about 11 passes instead of 32.
constexpr int WAYS = 7;

__global__ __launch_bounds__(1024) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ draws, int* __restrict__ out) {
  __shared__ Best sb[16];
  __shared__ float sf[16];
  __shared__ float sw[16][WAYS];
  const int r = blockIdx.x;
  const float* x = logits + (size_t)r * V;
  const float T = temperature != nullptr ? temperature[r] : 0.f;

  Best b = {-INFINITY, 0x7fffffff};
  for_each_logit(x, V, [&](float v, int i) { b = better(b, Best{v, i}); });
  b = block_best(b, sb);
  if (T == 0.f) {
    if (threadIdx.x == 0) out[r] = b.i;
    return;
  }
  const float invT = 1.f / fmaxf(T, 1e-6f);
  const float xmax = b.v;
  // threshold: entries with logit >= cut stay in the draw
  float cut = -INFINITY;
  const int k = top_k != nullptr ? top_k[r] : -1;
  const float pmass = top_p != nullptr ? top_p[r] : 1.f;
  if (k > 0 && k < V) {
    // largest cut with count(x >= cut) >= k: the count falls as the cut rises
    uint32_t lo = key_of(-INFINITY), hi = key_of(xmax);
    while (lo < hi) {
      const uint64_t span = hi - lo;
      float c[WAYS], cnt[WAYS];
#pragma unroll
      for (int j = 0; j < WAYS; ++j) {
        c[j] = float_of(lo + (uint32_t)((span * (j + 1) + WAYS) / (WAYS + 1)));   // rounded up: above lo
        cnt[j] = 0.f;
      }
      for_each_logit(x, V, [&](float v, int) {
#pragma unroll
        for (int j = 0; j < WAYS; ++j) cnt[j] += v >= c[j] ? 1.f : 0.f;
      });
      block_sums<WAYS>(cnt, sw);
      uint32_t new_lo = lo, new_hi = hi;
      bool capped = false;
#pragma unroll
      for (int j = 0; j < WAYS; ++j) {
        const uint32_t t = key_of(c[j]);
        if (cnt[j] >= (float)k) new_lo = t;
        else if (!capped) { new_hi = t - 1; capped = true; }
      }
      lo = new_lo;
      hi = new_hi;
    }
    cut = float_of(lo);
  } else if (k <= 0 && pmass < 1.f) {
    float z = 0.f;
    for_each_logit(x, V, [&](float v, int) { z += weight_of((v - xmax) * invT); });
    z = block_sum(z, sf);
    const float target = pmass * z;
    // smallest cut whose mass sum(p_i : x_i >= cut) stays <= top_p: the mass
    // falls as the cut rises; the maximum always stays
    uint32_t lo = key_of(-INFINITY), hi = key_of(xmax);
    while (lo < hi) {
      const uint64_t span = hi - lo;
      float c[WAYS], mass[WAYS];
#pragma unroll
      for (int j = 0; j < WAYS; ++j) {
        c[j] = float_of(lo + (uint32_t)(span * (j + 1) / (WAYS + 1)));            // rounded down: below hi
        mass[j] = 0.f;
      }
      for_each_logit(x, V, [&](float v, int) {
        const float w = weight_of((v - xmax) * invT);
#pragma unroll
        for (int j = 0; j < WAYS; ++j) mass[j] += v >= c[j] ? w : 0.f;
      });
      block_sums<WAYS>(mass, sw);
      uint32_t new_lo = lo, new_hi = hi;
      bool found = false;
#pragma unroll
      for (int j = 0; j < WAYS; ++j) {
        const uint32_t t = key_of(c[j]);
        if (!found) {
          if (mass[j] <= target) { new_hi = t; found = true; }
          else new_lo = t + 1;
        }
      }
      lo = new_lo;
      hi = new_hi;
    }
    cut = float_of(lo);
  }
  const uint64_t seed = (uint64_t)seeds[r], draw = (uint64_t)draws[r];
  Best g = {-INFINITY, 0x7fffffff};
  for_each_logit(x, V, [&](float v, int i) {
    if (v >= cut) {
      const float u = uniform01(seed, draw, (uint32_t)i);
      g = better(g, Best{v * invT + gumbel_of(u), i});      // the same value as in the two-stage draw
    }
  });
  g = block_best(g, sb);
  if (threadIdx.x == 0) out[r] = g.i;
}

// Greedy rows of a wide vocabulary: CHUNKS workgroups per row each find the
// best of a slice, a second small kernel picks among them (ties: first index).
// With temperatures the same two stages draw from the whole softmax: the
// winner of logit_i / T + g_i needs neither the maximum nor a cut, so the row
// is split like a greedy one (rows with temperature 0 stay greedy).
__global__ __launch_bounds__(256) void argmax_partial_kernel(
    const float* __restrict__ logits, int V, int chunks, Best* __restrict__ part,
    const float* __restrict__ temperature, const int64_t* __restrict__ seeds,
    const int64_t* __restrict__ draws) {
  __shared__ Best sb[16];
  const int r = blockIdx.y, c = blockIdx.x;
  const float* x = logits + (size_t)r * V;
  const int per = (V + chunks - 1) / chunks;
  const int lo = c * per, hi = lo + per < V ? lo + per : V;
  const float T = temperature != nullptr ? temperature[r] : 0.f;
  Best b = {-INFINITY, 0x7fffffff};
  if (T == 0.f) {
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) b = better(b, Best{x[i], i});
  } else {
    const float invT = 1.f / fmaxf(T, 1e-6f);
    const uint64_t seed = (uint64_t)seeds[r], draw = (uint64_t)draws[r];
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x)
      b = better(b, Best{x[i] * invT + gumbel_of(uniform01(seed, draw, (uint32_t)i)), i});
  }
  b = block_best(b, sb);
  if (threadIdx.x == 0) part[(size_t)r * chunks + c] = b;
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const Best* __restrict__ part, int chunks,
                                                          int* __restrict__ out) {
  __shared__ Best sb[16];
  const int r = blockIdx.x;
  Best b = {-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < chunks; i += blockDim.x) b = better(b, part[(size_t)r * chunks + i]);
  b = block_best(b, sb);
  if (threadIdx.x == 0) out[r] = b.i;
}

// part: chunks * R pairs of (float, int) = 8 * chunks * R bytes of scratch.
extern "C" const char* sl_argmax(const float* logits, int R, int V, int chunks, void* part,
                                 int* out, hipStream_t stream) {
  SL_CHECK(R >= 0 && V > 0, "argmax: sizes must be positive");
  SL_CHECK(chunks >= 1 && chunks <= 1024 && part != nullptr, "argmax: 1..1024 chunks and scratch");
  SL_CHECK(R <= 65535, "argmax: more than 65535 rows");
  if (R == 0) return nullptr;
  argmax_partial_kernel<<<dim3(chunks, R), 256, 0, stream>>>(logits, V, chunks, (Best*)part, nullptr,
                                                           nullptr, nullptr);
  const char* e = sl_launch_status();
  if (e) return e;
  argmax_final_kernel<<<R, 64, 0, stream>>>((const Best*)part, chunks, out);
  return sl_launch_status();
}

// top_k == nullptr and top_p == nullptr: every row draws from its whole
// softmax (or is greedy), in two stages over `chunks` slices of a row; `part`
// as for sl_argmax.  Otherwise one workgroup per row finds the row's cut first.
extern "C" const char* sl_sample(const float* logits, int R, int V, const float* temperature,
                                 const int* top_k, const float* top_p, const int64_t* seeds,
                                 const int64_t* draws, int chunks, void* part, int* out,
                                 hipStream_t stream) {
  SL_CHECK(R >= 0 && V > 0, "sample: sizes must be positive");
  SL_CHECK(temperature == nullptr || (seeds != nullptr && draws != nullptr),
           "sample: a temperature needs seeds and draw counters");
  SL_CHECK((top_k == nullptr) == (top_p == nullptr), "sample: top_k and top_p go together");
  if (R == 0) return nullptr;
  if (top_k == nullptr) {
    SL_CHECK(chunks >= 1 && chunks <= 1024 && part != nullptr, "sample: 1..1024 chunks and scratch");
    SL_CHECK(R <= 65535, "sample: more than 65535 rows");
    argmax_partial_kernel<<<dim3(chunks, R), 256, 0, stream>>>(logits, V, chunks, (Best*)part,
                                                             temperature, seeds, draws);
    const char* e = sl_launch_status();
    if (e) return e;
    argmax_final_kernel<<<R, 64, 0, stream>>>((const Best*)part, chunks, out);
    return sl_launch_status();
  }
  sample_kernel<<<R, 1024, 0, stream>>>(logits, V, temperature, top_k, top_p, seeds, draws, out);
  return sl_launch_status();
}
