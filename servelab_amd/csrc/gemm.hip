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
