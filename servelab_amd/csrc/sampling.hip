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

// order-preserving map float -> uint32
__device__ __forceinline__ uint32_t key_of(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float float_of(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

__global__ __launch_bounds__(1024) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p,
    const int64_t* __restrict__ seeds, const int64_t* __restrict__ draws, int* __restrict__ out) {
  __shared__ Best sb[16];
  __shared__ float sf[16];
  const int r = blockIdx.x;
  const float* x = logits + (size_t)r * V;
  const float T = temperature != nullptr ? temperature[r] : 0.f;

  Best b = {-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < V; i += blockDim.x) b = better(b, Best{x[i], i});
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
    // largest cut with count(x >= cut) >= k, by bisection on the ordered bits
    uint32_t lo = key_of(-INFINITY), hi = key_of(xmax);
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      const float c = float_of(mid);
      float cnt = 0.f;
      for (int i = threadIdx.x; i < V; i += blockDim.x) cnt += x[i] >= c ? 1.f : 0.f;
      cnt = block_sum(cnt, sf);
      if (cnt >= (float)k) lo = mid; else hi = mid - 1;
    }
    cut = float_of(lo);
  } else if (k <= 0 && pmass < 1.f) {
    float z = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) z += expf((x[i] - xmax) * invT);
    z = block_sum(z, sf);
    // smallest cut whose mass sum(p_i : x_i >= cut) stays <= top_p; the maximum always stays
    uint32_t lo = key_of(-INFINITY), hi = key_of(xmax);
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      const float c = float_of(mid);
      float mass = 0.f;
      for (int i = threadIdx.x; i < V; i += blockDim.x)
        mass += x[i] >= c ? expf((x[i] - xmax) * invT) : 0.f;
      mass = block_sum(mass, sf);
      if (mass <= pmass * z) hi = mid; else lo = mid + 1;
    }
    cut = float_of(lo);
  }
  const uint64_t seed = (uint64_t)seeds[r], draw = (uint64_t)draws[r];
  Best g = {-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    if (x[i] >= cut) {
      const float u = uniform01(seed, draw, (uint32_t)i);
      g = better(g, Best{(x[i] - xmax) * invT - logf(-logf(u)), i});
    }
  }
  g = block_best(g, sb);
  if (threadIdx.x == 0) out[r] = g.i;
}

// Greedy rows of a wide vocabulary: CHUNKS workgroups per row each find the
// best of a slice, a second small kernel picks among them (ties: first index).
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits, int V,
                                                             int chunks, Best* __restrict__ part) {
  __shared__ Best sb[16];
  const int r = blockIdx.y, c = blockIdx.x;
  const float* x = logits + (size_t)r * V;
  const int per = (V + chunks - 1) / chunks;
  const int lo = c * per, hi = lo + per < V ? lo + per : V;
  Best b = {-INFINITY, 0x7fffffff};
  for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) b = better(b, Best{x[i], i});
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
  argmax_partial_kernel<<<dim3(chunks, R), 256, 0, stream>>>(logits, V, chunks, (Best*)part);
  const char* e = sl_launch_status();
  if (e) return e;
  argmax_final_kernel<<<R, 64, 0, stream>>>((const Best*)part, chunks, out);
  return sl_launch_status();
}

extern "C" const char* sl_sample(const float* logits, int R, int V, const float* temperature,
                                 const int* top_k, const float* top_p, const int64_t* seeds,
                                 const int64_t* draws, int* out, hipStream_t stream) {
  SL_CHECK(R >= 0 && V > 0, "sample: sizes must be positive");
  SL_CHECK(temperature == nullptr || (seeds != nullptr && draws != nullptr),
           "sample: a temperature needs seeds and draw counters");
  if (R == 0) return nullptr;
  sample_kernel<<<R, 1024, 0, stream>>>(logits, V, temperature, top_k, top_p, seeds, draws, out);
  return sl_launch_status();
}
