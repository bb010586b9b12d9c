// Sampling from float32 logits [R, V].
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
#include "sampling_api.h"
#include <mutex>

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
  // 23 bits: k + 0.5 is then exact in float32, so u stays inside (0, 1).  (With 24 bits the largest
  // k + 0.5 rounds up to 2^24, u becomes 1 and its Gumbel value infinite: once in 2^24 logits a
  // token would be drawn whatever its logit.)
  return ((float)(z >> 41) + 0.5f) * (1.0f / 8388608.0f);
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

// ---------------------------------------------------------------------------
// Cuts of a wide vocabulary, on many workgroups.  One workgroup per row (the
// kernel above) re-reads its row for every pass of the search through one CU;
// at 152,064 logits that is most of a millisecond for a handful of rows.  Here
// a row is split into `chunks` slices, one workgroup each, and the cut is
// found digit by digit, as in a radix sort: round d counts, for each of the 256
// values of the d-th byte of the ordered bit pattern, the logits that carry it
// (among those that match the bytes already decided) and the mass of their
// weights.  The next launch adds the slices' tables up, walks them from the
// top and decides that byte: the byte in which the k-th largest logit lies
// (top-k), or in which the cumulative mass passes top_p times the whole
// (top-p).  After four rounds the cut's bit pattern is known exactly.  Masses
// are integers (weight * 2^32), so the sums do not depend on the order in which
// workgroups and lanes add, and a seed draws the same token every time.
// ---------------------------------------------------------------------------
constexpr int DIGITS = 256;
constexpr int CUT_ROUNDS = 4;
constexpr int CUT_THREADS = 256;          // = DIGITS: thread d decides about digit d
constexpr int CUT_MAX_CHUNKS = 64;

struct CutState {                          // what the rounds so far know of a row's cut
  uint64_t mass_above;                     // mass of the logits above every pattern that begins with `prefix`
  uint64_t target;                         // top-p: top_p * the row's whole mass (known once the first digit is counted)
  uint32_t prefix;                         // the leading bytes of the cut's pattern
  uint32_t count_above;
  float xmax;
  int mode;                                // 0: no cut (or greedy), 1: top-k, 2: top-p
  int k;
  int pad;
};

__device__ __forceinline__ int cut_mode(int V, float T, int k, float p) {
  if (T == 0.f) return 0;
  if (k > 0 && k < V) return 1;
  if (k <= 0 && p < 1.f) return 2;
  return 0;
}

// The slice [lo, hi) of a row, four logits at a time where it is 16-byte aligned.
template <class F>
__device__ __forceinline__ void for_each_in_slice(const float* __restrict__ x, int lo, int hi, F f) {
  struct __attribute__((aligned(16))) f4 { float v[4]; };
  int done = lo;
  if (((uintptr_t)(x + lo) % 16) == 0) {
    const int n4 = (hi - lo) / 4;
    const f4* q = (const f4*)(x + lo);
    for (int i = threadIdx.x; i < n4; i += blockDim.x) {
      const f4 v = q[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) f(v.v[j], lo + 4 * i + j);
    }
    done = lo + 4 * n4;
  }
  for (int i = done + threadIdx.x; i < hi; i += blockDim.x) f(x[i], i);
}

// Adds up the slices' tables of the round that has just run and decides its
// digit.  Every workgroup of the next launch does this for itself (the tables
// of a row are a few tens of KB in L2); all threads return the new state.
__device__ CutState cut_advance(CutState st, int round, float top_p, int chunks,
                                const uint32_t* __restrict__ hc, const uint64_t* __restrict__ hm) {
  __shared__ uint32_t sn[DIGITS];
  __shared__ uint64_t sm[DIGITS];
  __shared__ CutState chosen;
  const int d = threadIdx.x;
  uint32_t n = 0;
  uint64_t m = 0;
  for (int c = 0; c < chunks; ++c) {
    n += hc[(size_t)c * DIGITS + d];
    m += hm[(size_t)c * DIGITS + d];
  }
  __syncthreads();                         // the arrays may still be read by an earlier call
  sn[d] = n;
  sm[d] = m;
  if (d == 0) {
    chosen = st;
    chosen.mode = 0;                       // nothing crosses: the row keeps everything
  }
  __syncthreads();
  // inclusive sums from the top digit down to d
  for (int step = 1; step < DIGITS; step *= 2) {
    uint32_t an = 0;
    uint64_t am = 0;
    if (d + step < DIGITS) {
      an = sn[d + step];
      am = sm[d + step];
    }
    __syncthreads();
    sn[d] += an;
    sm[d] += am;
    __syncthreads();
  }
  const uint32_t above_n = sn[d] - n;
  const uint64_t above_m = sm[d] - m;
  if (round == 0 && st.mode == 2)          // sm[0]: the whole row
    st.target = (uint64_t)((double)top_p * (double)sm[0]);
  bool mine;
  if (st.mode == 1) {
    const uint32_t need = (uint32_t)st.k - st.count_above;
    mine = above_n < need && need <= above_n + n;
  } else {
    const uint64_t before = st.mass_above + above_m;
    mine = before <= st.target && before + m > st.target;
  }
  if (mine) {
    CutState r = st;
    r.prefix = (st.prefix << 8) | (uint32_t)d;
    r.count_above = st.count_above + above_n;
    r.mass_above = st.mass_above + above_m;
    chosen = r;
  }
  __syncthreads();
  return chosen;
}

__device__ __forceinline__ uint64_t fixed_weight(float v, float xmax, float invT) {
  return (uint64_t)(weight_of((v - xmax) * invT) * 4294967296.f);
}

// Round ROUND: decide the digit of the round before (if any), then count this
// round's digit over the slice.  hc/hm: [2][R][chunks][DIGITS], the rounds
// alternate between the two halves; states: [CUT_ROUNDS][R].
template <int ROUND>
__global__ __launch_bounds__(CUT_THREADS) void cut_round_kernel(
    const float* __restrict__ logits, int V, int R, int chunks,
    const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const Best* __restrict__ maxes,
    CutState* __restrict__ states, uint32_t* __restrict__ hc, uint64_t* __restrict__ hm) {
  __shared__ uint32_t cnt[DIGITS];
  __shared__ unsigned long long mass[DIGITS];
  const int r = blockIdx.y, c = blockIdx.x, t = threadIdx.x;
  const float T = temperature[r];
  const size_t tables = (size_t)R * chunks * DIGITS;
  CutState st;
  if (ROUND == 0) {
    st.mode = cut_mode(V, T, top_k[r], top_p[r]);
    float xmax = -INFINITY;
    for (int i = 0; i < chunks; ++i) xmax = fmaxf(xmax, maxes[(size_t)r * chunks + i].v);
    st.xmax = xmax;
    st.prefix = 0;
    st.count_above = 0;
    st.mass_above = 0;
    st.target = 0;
    st.k = top_k[r];
    st.pad = 0;
  } else {
    st = states[(size_t)(ROUND - 1) * R + r];
    if (st.mode != 0) {
      const size_t prev = ((ROUND - 1) % 2) * tables + (size_t)r * chunks * DIGITS;
      st = cut_advance(st, ROUND - 1, top_p[r], chunks, hc + prev, hm + prev);
    }
  }
  if (c == 0 && t == 0) states[(size_t)ROUND * R + r] = st;
  if (st.mode == 0) return;

  cnt[t] = 0;
  mass[t] = 0;
  __syncthreads();
  const float invT = 1.f / fmaxf(T, 1e-6f);
  const int per = ((V + chunks - 1) / chunks + 3) & ~3;
  const int lo = c * per < V ? c * per : V, hi = lo + per < V ? lo + per : V;
  const bool weigh = st.mode == 2;
  // neighbours mostly share a digit in the first rounds: a thread adds up a
  // run of equal digits before it goes to the table
  int run_digit = -1;
  uint32_t run_n = 0;
  uint64_t run_m = 0;
  auto flush = [&]() {
    if (run_n) {
      atomicAdd(&cnt[run_digit], run_n);
      if (weigh) atomicAdd(&mass[run_digit], (unsigned long long)run_m);
    }
  };
  for_each_in_slice(logits + (size_t)r * V, lo, hi, [&](float v, int) {
    const uint32_t key = key_of(v);
    if (ROUND > 0 && (key >> (32 - 8 * ROUND)) != st.prefix) return;
    const int digit = (int)((key >> (24 - 8 * ROUND)) & 255u);
    if (digit != run_digit) {
      flush();
      run_digit = digit;
      run_n = 0;
      run_m = 0;
    }
    run_n += 1;
    if (weigh) run_m += fixed_weight(v, st.xmax, invT);
  });
  flush();
  __syncthreads();
  const size_t mine = (ROUND % 2) * tables + ((size_t)r * chunks + c) * DIGITS;
  hc[mine + t] = cnt[t];
  hm[mine + t] = mass[t];
}

// Greedy rows of a wide vocabulary: CHUNKS workgroups per row each find the
// best of a slice, a second small kernel picks among them (ties: first index).
// With temperatures the same two stages draw from the whole softmax: the
// winner of logit_i / T + g_i needs neither the maximum nor a cut, so the row
// is split like a greedy one (rows with temperature 0 stay greedy).  After the
// rounds above (`states` given) a row draws among the logits its cut keeps.
__global__ __launch_bounds__(CUT_THREADS) void argmax_partial_kernel(
    const float* __restrict__ logits, int V, int R, int chunks, Best* __restrict__ part,
    const float* __restrict__ temperature, const int64_t* __restrict__ seeds,
    const int64_t* __restrict__ draws, const float* __restrict__ top_p,
    const CutState* __restrict__ states, const uint32_t* __restrict__ hc,
    const uint64_t* __restrict__ hm) {
  __shared__ Best sb[16];
  const int r = blockIdx.y, c = blockIdx.x;
  const float* x = logits + (size_t)r * V;
  const int per = ((V + chunks - 1) / chunks + 3) & ~3;
  const int lo = c * per < V ? c * per : V, hi = lo + per < V ? lo + per : V;
  const float T = temperature != nullptr ? temperature[r] : 0.f;
  Best b = {-INFINITY, 0x7fffffff};
  if (T == 0.f) {
    for_each_in_slice(x, lo, hi, [&](float v, int i) { b = better(b, Best{v, i}); });
  } else {
    uint32_t lowest = 0;                   // patterns from here on stay in the draw
    if (states != nullptr) {
      CutState st = states[(size_t)(CUT_ROUNDS - 1) * R + r];
      if (st.mode != 0) {
        const size_t last = ((CUT_ROUNDS - 1) % 2) * ((size_t)R * chunks * DIGITS) +
                            (size_t)r * chunks * DIGITS;
        st = cut_advance(st, CUT_ROUNDS - 1, top_p[r], chunks, hc + last, hm + last);
      }
      // top-k keeps the k-th largest and its equals; top-p keeps what lies
      // above the logit at which the mass passes the target, and the maximum
      // in any case (servelab/engine/sampler.py:30-44)
      if (st.mode == 1 || (st.mode == 2 && st.count_above == 0)) lowest = st.prefix;
      else if (st.mode == 2) lowest = st.prefix + 1;
    }
    const float invT = 1.f / fmaxf(T, 1e-6f);
    const uint64_t seed = (uint64_t)seeds[r], draw = (uint64_t)draws[r];
    for_each_in_slice(x, lo, hi, [&](float v, int i) {
      if (key_of(v) >= lowest)
        b = better(b, Best{v * invT + gumbel_of(uniform01(seed, draw, (uint32_t)i)), i});
    });
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

static size_t align_up(size_t n) { return (n + 255) & ~(size_t)255; }

// Bytes of scratch for a call with these sizes: the slices' bests, and for
// cuts found on many workgroups also the rows' maxima, states and tables.
extern "C" size_t sl_sample_workspace(int R, int chunks, int cuts) {
  const size_t bests = align_up((size_t)R * chunks * sizeof(Best));
  if (!cuts) return bests;
  return 2 * bests + align_up((size_t)CUT_ROUNDS * R * sizeof(CutState)) +
         align_up(2 * (size_t)R * chunks * DIGITS * sizeof(uint64_t)) +
         align_up(2 * (size_t)R * chunks * DIGITS * sizeof(uint32_t));
}

extern "C" const char* sl_argmax(const float* logits, int R, int V, int chunks, void* work,
                                 int* out, hipStream_t stream) {
  SL_CHECK(R >= 0 && V > 0, "argmax: sizes must be positive");
  SL_CHECK(chunks >= 1 && chunks <= 1024 && work != nullptr, "argmax: 1..1024 chunks and scratch");
  SL_CHECK(R <= 65535, "argmax: more than 65535 rows");
  if (R == 0) return nullptr;
  argmax_partial_kernel<<<dim3(chunks, R), CUT_THREADS, 0, stream>>>(
      logits, V, R, chunks, (Best*)work, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
  const char* e = sl_launch_status();
  if (e) return e;
  argmax_final_kernel<<<R, 64, 0, stream>>>((const Best*)work, chunks, out);
  return sl_launch_status();
}

// top_k == nullptr and top_p == nullptr: every row draws from its whole
// softmax (or is greedy), in two stages over `chunks` slices of a row.
// Otherwise the rows' cuts are found first: with chunks >= 2 by the rounds
// over slices, else by one workgroup per row.  `work`: sl_sample_workspace bytes.
extern "C" const char* sl_sample(const float* logits, int R, int V, const float* temperature,
                                 const int* top_k, const float* top_p, const int64_t* seeds,
                                 const int64_t* draws, int chunks, void* work, int* out,
                                 hipStream_t stream) {
  SL_CHECK(R >= 0 && V > 0, "sample: sizes must be positive");
  SL_CHECK(temperature == nullptr || (seeds != nullptr && draws != nullptr),
           "sample: a temperature needs seeds and draw counters");
  SL_CHECK((top_k == nullptr) == (top_p == nullptr), "sample: top_k and top_p go together");
  if (R == 0) return nullptr;
  if (top_k != nullptr && chunks < 2) {
    sample_kernel<<<R, 1024, 0, stream>>>(logits, V, temperature, top_k, top_p, seeds, draws, out);
    return sl_launch_status();
  }
  SL_CHECK(chunks >= 1 && chunks <= 1024 && work != nullptr, "sample: 1..1024 chunks and scratch");
  SL_CHECK(R <= 65535, "sample: more than 65535 rows");
  Best* bests = (Best*)work;
  if (top_k == nullptr) {
    argmax_partial_kernel<<<dim3(chunks, R), CUT_THREADS, 0, stream>>>(
        logits, V, R, chunks, bests, temperature, seeds, draws, nullptr, nullptr, nullptr, nullptr);
  } else {
    SL_CHECK(temperature != nullptr, "sample: cuts need temperatures");
    SL_CHECK(chunks <= CUT_MAX_CHUNKS, "sample: at most 64 slices a row when cuts are searched");
    char* at = (char*)work + align_up((size_t)R * chunks * sizeof(Best));
    Best* maxes = (Best*)at;
    at += align_up((size_t)R * chunks * sizeof(Best));
    CutState* states = (CutState*)at;
    at += align_up((size_t)CUT_ROUNDS * R * sizeof(CutState));
    uint64_t* hm = (uint64_t*)at;
    at += align_up(2 * (size_t)R * chunks * DIGITS * sizeof(uint64_t));
    uint32_t* hc = (uint32_t*)at;
    const dim3 grid(chunks, R);
    argmax_partial_kernel<<<grid, CUT_THREADS, 0, stream>>>(
        logits, V, R, chunks, maxes, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
    cut_round_kernel<0><<<grid, CUT_THREADS, 0, stream>>>(logits, V, R, chunks, temperature, top_k,
                                                          top_p, maxes, states, hc, hm);
    cut_round_kernel<1><<<grid, CUT_THREADS, 0, stream>>>(logits, V, R, chunks, temperature, top_k,
                                                          top_p, maxes, states, hc, hm);
    cut_round_kernel<2><<<grid, CUT_THREADS, 0, stream>>>(logits, V, R, chunks, temperature, top_k,
                                                          top_p, maxes, states, hc, hm);
    cut_round_kernel<3><<<grid, CUT_THREADS, 0, stream>>>(logits, V, R, chunks, temperature, top_k,
                                                          top_p, maxes, states, hc, hm);
    const char* e = sl_launch_status();
    if (e) return e;
    argmax_partial_kernel<<<grid, CUT_THREADS, 0, stream>>>(
        logits, V, R, chunks, bests, temperature, seeds, draws, top_p, states, hc, hm);
  }
  const char* e = sl_launch_status();
  if (e) return e;
  argmax_final_kernel<<<R, 64, 0, stream>>>((const Best*)work, chunks, out);
  return sl_launch_status();
}

// ---------------------------------------------------------------------------
// The entry point that allocates nothing (declared and described in
// sampling_api.h).  `scratch` is a host-side stand-in in host code, not a device
// address: the address of each GPU's copy is looked up once per device, with
// that device current, and only that address is ever handed to a kernel.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[SL_SAMPLE_STATIC_BYTES];

constexpr int STATIC_MAX_DEVICES = 64;
static void* scratch_address[STATIC_MAX_DEVICES];     // by device ordinal; nullptr: not looked up yet
static std::mutex scratch_mutex;

static const char* scratch_of_current_device(void** address) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) return "sample_static: no current device";
  SL_CHECK(device >= 0 && device < STATIC_MAX_DEVICES, "sample_static: device ordinal beyond 63");
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_address[device] == nullptr) {
    void* found = nullptr;
    const hipError_t e = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hipGetErrorString(e);
    SL_CHECK(found != nullptr, "sample_static: the scratch array has no address on this device");
    scratch_address[device] = found;
  }
  *address = scratch_address[device];
  return nullptr;
}

extern "C" const char* sl_sample_static(const float* logits, int R, int V, const float* temperature,
                                        const int* top_k, const float* top_p, const int64_t* seeds,
                                        const int64_t* draws, int* out, hipStream_t stream) {
  SL_CHECK(R >= 0 && V > 0, "sample_static: sizes must be positive");
  SL_CHECK((top_k == nullptr) == (top_p == nullptr), "sample_static: top_k and top_p go together");
  if (R == 0) return nullptr;
  const bool cuts = top_k != nullptr;
  // slices of about 2,048 logits (4,096 when cuts are searched: every workgroup
  // adds up the tables of all slices of its row), as the callers of sl_sample choose
  int chunks = cuts ? V / 4096 : V / 2048;
  const int most = cuts ? 16 : 64;
  chunks = chunks < 1 ? 1 : chunks > most ? most : chunks;
  void* work = nullptr;
  if (!(cuts && chunks < 2)) {             // (short rows with cuts take one workgroup a row, no scratch)
    SL_CHECK(sl_sample_workspace(R, chunks, cuts) <= (size_t)SL_SAMPLE_STATIC_BYTES,
             "sample_static: these rows need more scratch than the static 8 MiB array holds "
             "(rows x slices x 6,160 bytes with cuts, x 8 without); use sl_sample with a workspace");
    const char* e = scratch_of_current_device(&work);
    if (e) return e;
  }
  return sl_sample(logits, R, V, temperature, top_k, top_p, seeds, draws, chunks, work, out, stream);
}
