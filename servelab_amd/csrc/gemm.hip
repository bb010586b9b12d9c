// y[M, N] = x[M, K] * W[N, K]^T (+ bias[N]); W rows are K-contiguous
// (checkpoint layout, servelab/parallel/layers.py:164-180).  Accumulation is
// float with plain FMA in both builds; the float build is the true 32-bit path.
//
//   sl_gemm_rows  few rows (decode): one wavefront per output column streams
//                 one row of W with 16-byte loads; bound by reading W once
//                 per group of SL_ROWS rows of x.
//   sl_gemm_tiled any M: 64x64 LDS tiles, 4x4 outputs per thread.
#include "common.h"

#if defined(SL_F32)
#define SL_VEC 4
#else
#define SL_VEC 8
#endif

struct __attribute__((aligned(16))) vec_t { act_t v[SL_VEC]; };

// ------------------------------------------------------------------ few rows
template <int MB>
__global__ __launch_bounds__(256) void gemm_rows_kernel(
    const act_t* __restrict__ x, const act_t* __restrict__ w, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32) {
  const int lane = threadIdx.x % SL_WAVE;
  const int n = blockIdx.x * (blockDim.x / SL_WAVE) + threadIdx.x / SL_WAVE;
  if (n >= N) return;
  const act_t* wr = w + (size_t)n * K;
  for (int m0 = 0; m0 < M; m0 += MB) {
    float acc[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) acc[i] = 0.f;
    for (int k = lane * SL_VEC; k < K; k += SL_WAVE * SL_VEC) {
      const vec_t wv = *(const vec_t*)(wr + k);
      float wf[SL_VEC];
#pragma unroll
      for (int j = 0; j < SL_VEC; ++j) wf[j] = to_f(wv.v[j]);
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        if (m0 + i < M) {
          const vec_t xv = *(const vec_t*)(x + (size_t)(m0 + i) * K + k);
#pragma unroll
          for (int j = 0; j < SL_VEC; ++j) acc[i] += wf[j] * to_f(xv.v[j]);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      const float s = wave_sum(acc[i]);
      if (lane == 0 && m0 + i < M) {
        const float r = s + (bias != nullptr ? bias[n] : 0.f);
        if (out_f32) ((float*)y)[(size_t)(m0 + i) * N + n] = r;
        else ((act_t*)y)[(size_t)(m0 + i) * N + n] = from_f<act_t>(r);
      }
    }
  }
}

extern "C" const char* sl_gemm_rows(const void* x, const void* w, const float* bias, void* y,
                                    int M, int N, int K, int out_f32, hipStream_t stream) {
  SL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_rows: sizes must be positive");
  SL_CHECK(K % SL_VEC == 0, "gemm_rows: K must be a multiple of the 16-byte vector");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
           "gemm_rows: x and W must be 16-byte aligned");
  if (M == 0) return nullptr;
  const int waves = 4;
  const dim3 grid((N + waves - 1) / waves);
  if (M == 1)
    gemm_rows_kernel<1><<<grid, waves * SL_WAVE, 0, stream>>>(
        (const act_t*)x, (const act_t*)w, bias, y, M, N, K, out_f32);
  else if (M == 2)
    gemm_rows_kernel<2><<<grid, waves * SL_WAVE, 0, stream>>>(
        (const act_t*)x, (const act_t*)w, bias, y, M, N, K, out_f32);
  else if (M <= 4)
    gemm_rows_kernel<4><<<grid, waves * SL_WAVE, 0, stream>>>(
        (const act_t*)x, (const act_t*)w, bias, y, M, N, K, out_f32);
  else
    gemm_rows_kernel<8><<<grid, waves * SL_WAVE, 0, stream>>>(
        (const act_t*)x, (const act_t*)w, bias, y, M, N, K, out_f32);
  return sl_launch_status();
}

// --------------------------------------------------------------------- tiled
#define TM 64
#define TN 64
#define TK 16

__global__ __launch_bounds__(256) void gemm_tiled_kernel(
    const act_t* __restrict__ x, const act_t* __restrict__ w, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32) {
  __shared__ float xs[TK][TM + 4];
  __shared__ float ws[TK][TN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int tx = tid % 16, ty = tid / 16;          // 4 columns at tx*4, 4 rows at ty*4
  const int lr = tid / 4, lk = (tid % 4) * 4;      // loader: row lr, k offset lk..lk+3
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const int m = m0 + lr, n = n0 + lr;
      xs[lk + j][lr] = (m < M && k < K) ? to_f(x[(size_t)m * K + k]) : 0.f;
      ws[lk + j][lr] = (n < N && k < K) ? to_f(w[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      const float r = acc[i][j] + (bias != nullptr ? bias[n] : 0.f);
      if (out_f32) ((float*)y)[(size_t)m * N + n] = r;
      else ((act_t*)y)[(size_t)m * N + n] = from_f<act_t>(r);
    }
  }
}

extern "C" const char* sl_gemm_tiled(const void* x, const void* w, const float* bias, void* y,
                                     int M, int N, int K, int out_f32, hipStream_t stream) {
  SL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled: sizes must be positive");
  if (M == 0) return nullptr;
  const dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  SL_CHECK(grid.y <= 65535, "gemm_tiled: more than 65535 row tiles");
  gemm_tiled_kernel<<<grid, 256, 0, stream>>>((const act_t*)x, (const act_t*)w, bias, y, M, N, K,
                                              out_f32);
  return sl_launch_status();
}

// ------------------------------------------------ few rows on the matrix cores
#if !defined(SL_F32)
// y[M, N] for M <= 64 in bfloat16: bound by streaming W from HBM once.
// A workgroup of 8 wavefronts owns 16 * NT columns of y (rows of W); each
// wavefront takes an eighth of K, so that every row of W is read in long
// contiguous runs and every wavefront has many loads in flight at once; the
// eight partial tiles are summed through LDS.  Per 32 values of k one
// mfma 16x16x32 per (16 rows of W) x (16 rows of x): A = W, B = x; the rows of
// x are loaded once per k-step and used for all NT tiles of W.  Rows beyond M
// or N repeat the last row and are not stored; k-steps beyond the wavefront's
// share are loaded from its last step and zeroed, so the loop has no serial tail.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 load_stream(const __bf16* p) {
  // W is read once per call: a non-temporal load keeps it from displacing x in the caches
  const i32x4 v = __builtin_nontemporal_load((const i32x4*)p);
  return __builtin_bit_cast(bf16x8, v);
}

template <int MB, int WAVES, bool NT_LOAD>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(
    const __bf16* __restrict__ x, const __bf16* __restrict__ w, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32) {
  constexpr int U = 8;
  __shared__ f32x4 red[WAVES][MB][64];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, i = lane & 15, gq = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int KT = K / 32;
  const int ks0 = (int)((long long)KT * wave / WAVES), ks1 = (int)((long long)KT * (wave + 1) / WAVES);
  const int nrow = n0 + i < N ? n0 + i : N - 1;
  const __bf16* wp = w + (size_t)nrow * K + 8 * gq;
  const __bf16* xp[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + i < M ? 16 * b + i : M - 1;
    xp[b] = x + (size_t)m * K + 8 * gq;
  }
  f32x4 acc[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
  int ks = ks0;
  for (; ks + U <= ks1; ks += U) {
    bf16x8 a[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      a[u] = NT_LOAD ? load_stream(wp + 32 * (size_t)(ks + u)) : *(const bf16x8*)(wp + 32 * (size_t)(ks + u));
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int b = 0; b < MB; ++b) {
        const bf16x8 bv = *(const bf16x8*)(xp[b] + 32 * (size_t)(ks + u));
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], bv, acc[b], 0, 0, 0);
      }
  }
  for (; ks < ks1; ++ks) {
    const bf16x8 a = NT_LOAD ? load_stream(wp + 32 * (size_t)ks) : *(const bf16x8*)(wp + 32 * (size_t)ks);
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const bf16x8 bv = *(const bf16x8*)(xp[b] + 32 * (size_t)ks);
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bv, acc[b], 0, 0, 0);
    }
  }
#pragma unroll
  for (int b = 0; b < MB; ++b) red[wave][b][lane] = acc[b];
  __syncthreads();
  // lane (m_local + 16 (n_local / 4)) holds y[m_local, n_local] in element n_local % 4
  for (int idx = threadIdx.x; idx < MB * 256; idx += WAVES * 64) {
    const int b = idx / 256, rem = idx % 256, m_local = rem / 16, n_local = rem % 16;
    const int m = 16 * b + m_local, n = n0 + n_local;
    if (m < M && n < N) {
      float s = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) s += red[wv][b][m_local + 16 * (n_local / 4)][n_local % 4];
      if (bias != nullptr) s += bias[n];
      if (out_f32) ((float*)y)[(size_t)m * N + n] = s;
      else ((__bf16*)y)[(size_t)m * N + n] = (__bf16)s;
    }
  }
}

template <int MB>
static const char* launch_skinny(int variant, const __bf16* x, const __bf16* w, const float* bias,
                                 void* y, int M, int N, int K, int out_f32, hipStream_t stream) {
  const dim3 grid((N + 15) / 16);
  switch (variant) {
    case 1: gemm_skinny_kernel<MB, 8, true><<<grid, 512, 0, stream>>>(x, w, bias, y, M, N, K, out_f32); break;
    case 2: gemm_skinny_kernel<MB, 4, false><<<grid, 256, 0, stream>>>(x, w, bias, y, M, N, K, out_f32); break;
    case 3: gemm_skinny_kernel<MB, 16, false><<<grid, 1024, 0, stream>>>(x, w, bias, y, M, N, K, out_f32); break;
    case 4: gemm_skinny_kernel<MB, 4, true><<<grid, 256, 0, stream>>>(x, w, bias, y, M, N, K, out_f32); break;
    default: gemm_skinny_kernel<MB, 8, false><<<grid, 512, 0, stream>>>(x, w, bias, y, M, N, K, out_f32);
  }
  return sl_launch_status();
}

extern "C" const char* sl_gemm_skinny(const void* x, const void* w, const float* bias, void* y,
                                      int M, int N, int K, int out_f32, int nt,
                                      hipStream_t stream) {
  SL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_skinny: sizes must be positive");
  SL_CHECK(M <= 64, "gemm_skinny: at most 64 rows");
  SL_CHECK(K % 32 == 0, "gemm_skinny: K must be a multiple of 32");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
           "gemm_skinny: x and W must be 16-byte aligned");
  if (M == 0) return nullptr;
  const __bf16* xx = (const __bf16*)x;
  const __bf16* ww = (const __bf16*)w;
  if (M <= 16) return launch_skinny<1>(nt, xx, ww, bias, y, M, N, K, out_f32, stream);
  if (M <= 32) return launch_skinny<2>(nt, xx, ww, bias, y, M, N, K, out_f32, stream);
  return launch_skinny<4>(nt, xx, ww, bias, y, M, N, K, out_f32, stream);
}
#endif
