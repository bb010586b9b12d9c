// y[M, N] = x[M, K] * W[N, K]^T (+ bias[N]); W rows are K-contiguous
// (checkpoint layout, servelab/parallel/layers.py:164-180).  Accumulation is
// float with plain FMA in both builds; the float build is the true 32-bit path.
//
//   sl_gemm_rows  few rows (decode): a wavefront streams the rows of W of one
//                 or four output columns with 16-byte loads against up to 8
//                 rows of x at a time.
//   sl_gemm_tiled any M: 64x64 LDS tiles, 4x4 outputs per thread.
#include "common.h"
#include <type_traits>

#if defined(SL_F32)
#define SL_VEC 4
#else
#define SL_VEC 8
#endif

struct __attribute__((aligned(16))) vec_t { act_t v[SL_VEC]; };

// ------------------------------------------------------------------ few rows
// A wavefront owns NC consecutive output columns: every 16-byte piece of x it
// loads meets NC rows of W, so x is read once per NC columns instead of once
// per column (with 8 rows of x that was 8 times the bytes of W itself).
template <int MB, int NC>
__global__ __launch_bounds__(256) void gemm_rows_kernel(
    const act_t* __restrict__ x, const act_t* __restrict__ w, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32) {
  const int lane = threadIdx.x % SL_WAVE;
  const int n0 = (blockIdx.x * (blockDim.x / SL_WAVE) + threadIdx.x / SL_WAVE) * NC;
  if (n0 >= N) return;
  const act_t* wr[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) wr[c] = w + (size_t)(n0 + c < N ? n0 + c : N - 1) * K;
  for (int m0 = 0; m0 < M; m0 += MB) {
    float acc[MB][NC];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int c = 0; c < NC; ++c) acc[i][c] = 0.f;
    for (int k = lane * SL_VEC; k < K; k += SL_WAVE * SL_VEC) {
      float wf[NC][SL_VEC];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const vec_t wv = *(const vec_t*)(wr[c] + k);
#pragma unroll
        for (int j = 0; j < SL_VEC; ++j) wf[c][j] = to_f(wv.v[j]);
      }
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        if (m0 + i < M) {
          const vec_t xv = *(const vec_t*)(x + (size_t)(m0 + i) * K + k);
#pragma unroll
          for (int j = 0; j < SL_VEC; ++j) {
            const float xf = to_f(xv.v[j]);
#pragma unroll
            for (int c = 0; c < NC; ++c) acc[i][c] += wf[c][j] * xf;
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const float s = wave_sum(acc[i][c]);
        if (lane == 0 && m0 + i < M && n0 + c < N) {
          const float r = s + (bias != nullptr ? bias[n0 + c] : 0.f);
          if (out_f32) ((float*)y)[(size_t)(m0 + i) * N + n0 + c] = r;
          else ((act_t*)y)[(size_t)(m0 + i) * N + n0 + c] = from_f<act_t>(r);
        }
      }
  }
}

// The same product with the rows of x staged through LDS: the eight wavefronts of a workgroup own
// four columns each and share every chunk of x, so x leaves the cache hierarchy once per 32 columns
// of W instead of once per 4 (with 8 rows of x that was twice the bytes of W itself, and what the
// float32 decode step spent most of its time pulling).  A lane keeps its own running sums over its
// share of K, as above.
template <int MB>
__global__ __launch_bounds__(512) void gemm_rows_shared_kernel(
    const act_t* __restrict__ x, const act_t* __restrict__ w, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32) {
  constexpr int NC = 4, KC = 256 * SL_VEC;           // values of k in a chunk: four steps of a wavefront
  __shared__ vec_t xs[MB][KC / SL_VEC];
  const int lane = threadIdx.x % SL_WAVE, wave = threadIdx.x / SL_WAVE;
  const int n0 = (blockIdx.x * (blockDim.x / SL_WAVE) + wave) * NC;
  const act_t* wr[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) wr[c] = w + (size_t)(n0 + c < N ? n0 + c : N - 1) * K;
  float acc[MB][NC];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[i][c] = 0.f;
  for (int k0 = 0; k0 < K; k0 += KC) {
    const int kv = (K - k0 < KC ? K - k0 : KC) / SL_VEC;       // vectors of this chunk in a row
    __syncthreads();                                           // the last chunk has been read
    for (int idx = threadIdx.x; idx < MB * kv; idx += blockDim.x) {
      const int m = idx / kv, v = idx % kv;
      xs[m][v] = *(const vec_t*)(x + (size_t)(m < M ? m : M - 1) * K + k0 + v * SL_VEC);
    }
    __syncthreads();
    for (int v = lane; v < kv; v += SL_WAVE) {
      float wf[NC][SL_VEC];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const vec_t wv = *(const vec_t*)(wr[c] + k0 + v * SL_VEC);
#pragma unroll
        for (int j = 0; j < SL_VEC; ++j) wf[c][j] = to_f(wv.v[j]);
      }
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        const vec_t xv = xs[i][v];
#pragma unroll
        for (int j = 0; j < SL_VEC; ++j) {
          const float xf = to_f(xv.v[j]);
#pragma unroll
          for (int c = 0; c < NC; ++c) acc[i][c] += wf[c][j] * xf;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const float s = wave_sum(acc[i][c]);
      if (lane == 0 && i < M && n0 + c < N) {
        const float r = s + (bias != nullptr ? bias[n0 + c] : 0.f);
        if (out_f32) ((float*)y)[(size_t)i * N + n0 + c] = r;
        else ((act_t*)y)[(size_t)i * N + n0 + c] = from_f<act_t>(r);
      }
    }
}

// `shared`: 4 to 16 rows of x (to 8 of bfloat16) go through LDS once per 32 columns (gemm_rows_shared_kernel).
extern "C" const char* sl_gemm_rows(const void* x, const void* w, const float* bias, void* y,
                                    int M, int N, int K, int out_f32, int shared, hipStream_t stream) {
  SL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_rows: sizes must be positive");
  SL_CHECK(K % SL_VEC == 0, "gemm_rows: K must be a multiple of the 16-byte vector");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
           "gemm_rows: x and W must be 16-byte aligned");
  if (M == 0) return nullptr;
  const int waves = 4;
  const act_t* xx = (const act_t*)x;
  const act_t* ww = (const act_t*)w;
  // (measured, float32, 7B shape: from 4 rows on the staged form wins, 8 rows 139 -> 113 us for gate/up and
  // 176 -> 114 us for down, 16 rows 281 -> 172 and 494 -> 174 us; with 1 to 3 rows it loses up to 18 us of 44)
  constexpr int SHARED_MAX_M = sizeof(act_t) == 4 ? 16 : 8;   // (16 rows of bfloat16 spill registers)
  if (shared && M >= 4 && M <= SHARED_MAX_M) {
    // (eight wavefronts a workgroup also for matrices of few rows: four, for twice the workgroups, measured
    // slower: down of the 7B shape at 8 / 16 rows 125 / 214 us against 114 / 174)
    const int threads = 512;
    const int cols = 4 * threads / SL_WAVE;
    const dim3 grid((N + cols - 1) / cols);
    if (M <= 4) gemm_rows_shared_kernel<4><<<grid, threads, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
    else if (M <= 8) gemm_rows_shared_kernel<8><<<grid, threads, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
    else if constexpr (SHARED_MAX_M == 16) gemm_rows_shared_kernel<16><<<grid, threads, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
    return sl_launch_status();
  }
  // one row of x: a column per wavefront keeps the most wavefronts in flight;
  // more rows: 4 columns per wavefront share each load of x
  if (M == 1) {
    gemm_rows_kernel<1, 1><<<(N + waves - 1) / waves, waves * SL_WAVE, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
    return sl_launch_status();
  }
  const dim3 grid((N + 4 * waves - 1) / (4 * waves));
  if (M == 2) gemm_rows_kernel<2, 4><<<grid, waves * SL_WAVE, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
  else if (M <= 4) gemm_rows_kernel<4, 4><<<grid, waves * SL_WAVE, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
  else gemm_rows_kernel<8, 4><<<grid, waves * SL_WAVE, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
  return sl_launch_status();
}

// --------------------------------------------------------------------- tiled
#define TM 64
#define TN 64
#define TK 16
#define SEGMENT_K 512      // terms a running sum takes before it is added to the total (a multiple of 16)

__global__ __launch_bounds__(256) void gemm_tiled_kernel(
    const act_t* __restrict__ x, const act_t* __restrict__ w, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32) {
  __shared__ float xs[TK][TM + 4];
  __shared__ float ws[TK][TN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int tx = tid % 16, ty = tid / 16;          // 4 columns at tx*4, 4 rows at ty*4
  const int lr = tid / 4, lk = (tid % 4) * 4;      // loader: row lr, k offset lk..lk+3
  // Sums of K products in one running float32 sum lose with the length of the sum; the sum is kept
  // in segments of SEGMENT_K terms, each started from zero and added to the total when it is full.
  float acc[4][4], total[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
    if (k0 != 0 && k0 % SEGMENT_K == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
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
      const float r = total[i][j] + acc[i][j] + (bias != nullptr ? bias[n] : 0.f);
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

// ------------------------------------- float32 products on the matrix cores
#if defined(SL_F32)
// y = x W^T in float32 for many rows: v_mfma_f32_32x32x2_f32 multiplies and adds
// float32 values as they are (no reduced-precision inputs, float32 sums), at
// twice the rate the vector ALU reaches without packed instructions.  A
// workgroup of four wavefronts owns a tile of x rows by W rows, a wavefront its
// part of it as tiles of 32 x 32; chunks of 16 values of k go through
// double-buffered LDS (rows padded to 17 floats: the 32 rows one operand read
// touches fall into 32 banks).  K % 16 == 0.
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int FK = 16, FS = FK + 1;

// WM x WN wavefronts (four in all), each TI x TJ tiles of 32 x 32: a workgroup
// owns 32 TI WM rows of x by 32 TJ WN rows of W.  <2, 2, 2, 2>: 128 x 128 for
// many rows; <1, 1, 1, 4>: 32 x 128 up to 64 rows (7B shape, 64 rows: a decode
// step of 95 ms against 129 ms with the large tiles and 175 ms with the FMA
// tiles; at 8 rows the wavefront-per-column kernel is twice as fast as either:
// 8 KB of W per barrier is too little in flight to stream it).
template <int TI, int TJ, int WM, int WN>
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
    float* __restrict__ y, int M, int N, int K) {
  static_assert(WM * WN == 4, "four wavefronts");
  constexpr int FM = 32 * TI * WM, FN = 32 * TJ * WN;
  constexpr int XL = (FM * 4 + 255) / 256, WL = (FN * 4 + 255) / 256;    // 16-byte loads a thread makes per chunk
  __shared__ float xs[2][FM * FS];
  __shared__ float ws[2][FN * FS];
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int m0 = blockIdx.y * FM, n0 = blockIdx.x * FN;
  // loader: 16-byte piece idx of a tile is row idx / 4, values of k from (idx % 4) * 4;
  // rows past the end load the last row (never stored)
  const float* xp[XL];
  const float* wp[WL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int idx = t + 256 * i, r = idx / 4 < FM ? idx / 4 : FM - 1;
    const int m = m0 + r < M ? m0 + r : M - 1;
    xp[i] = x + (size_t)m * K + (idx & 3) * 4;
  }
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int idx = t + 256 * i, r = idx / 4 < FN ? idx / 4 : FN - 1;
    const int n = n0 + r < N ? n0 + r : N - 1;
    wp[i] = w + (size_t)n * K + (idx & 3) * 4;
  }
  // running sums of SEGMENT_K terms (acc) and the sums of the full ones (total): a sum of 18,944
  // products in one float32 accumulator loses about six times what 37 sums of 512 lose
  f32x16 acc[TI][TJ], total[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = total[i][j][r] = 0.f;
  float4 xr[XL], wr[WL];
  auto load = [&](int k0) {
#pragma unroll
    for (int i = 0; i < XL; ++i) xr[i] = *(const float4*)(xp[i] + k0);
#pragma unroll
    for (int i = 0; i < WL; ++i) wr[i] = *(const float4*)(wp[i] + k0);
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      const int idx = t + 256 * i;
      if (idx < FM * 4) {
        float* d = &xs[buf][(idx / 4) * FS + (idx & 3) * 4];
        d[0] = xr[i].x; d[1] = xr[i].y; d[2] = xr[i].z; d[3] = xr[i].w;
      }
    }
#pragma unroll
    for (int i = 0; i < WL; ++i) {
      const int idx = t + 256 * i;
      if (idx < FN * 4) {
        float* d = &ws[buf][(idx / 4) * FS + (idx & 3) * 4];
        d[0] = wr[i].x; d[1] = wr[i].y; d[2] = wr[i].z; d[3] = wr[i].w;
      }
    }
  };
  const int nchunks = K / FK;
  load(0);
  store(0);
  __syncthreads();
  // operand element of this lane in a 32 x 2 step: row lane % 32, k lane / 32
  const int orow = lane & 31, ok = lane >> 5;
  constexpr int SEG = SEGMENT_K / FK;                 // chunks a running sum takes
  for (int c0 = 0; c0 < nchunks; c0 += SEG) {
    const int c1 = c0 + SEG < nchunks ? c0 + SEG : nchunks;
    for (int c = c0; c < c1; ++c) {
      const int buf = c & 1;
      if (c + 1 < nchunks) load((c + 1) * FK);
      const float* xa = &xs[buf][(wm * 32 * TI + orow) * FS + ok];
      const float* wb = &ws[buf][(wn * 32 * TJ + orow) * FS + ok];
#pragma unroll
      for (int kk = 0; kk < FK; kk += 2) {
        float a[TI], b[TJ];
#pragma unroll
        for (int i = 0; i < TI; ++i) a[i] = xa[32 * i * FS + kk];
#pragma unroll
        for (int j = 0; j < TJ; ++j) b[j] = wb[32 * j * FS + kk];
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
          for (int j = 0; j < TJ; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
      }
      if (c + 1 < nchunks) store(buf ^ 1);
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        total[i][j] += acc[i][j];
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
      }
  }
  // element r of a tile: row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32
#pragma unroll
  for (int j = 0; j < TJ; ++j) {
    const int n = n0 + (wn * TJ + j) * 32 + (lane & 31);
    if (n >= N) continue;
    const float bv = bias != nullptr ? bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + (wm * TI + i) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < M) y[(size_t)m * N + n] = total[i][j][r] + bv;
      }
  }
}

extern "C" const char* sl_gemm_f32_mfma(const void* x, const void* w, const float* bias, void* y,
                                        int M, int N, int K, hipStream_t stream) {
  SL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_f32_mfma: sizes must be positive");
  SL_CHECK(K % FK == 0, "gemm_f32_mfma: K must be a multiple of 16");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
           "gemm_f32_mfma: x and W must be 16-byte aligned");
  if (M == 0) return nullptr;
  const int rows = M <= 64 ? 32 : 128;
  const dim3 grid((N + 127) / 128, (M + rows - 1) / rows);
  SL_CHECK(grid.y <= 65535, "gemm_f32_mfma: more than 65535 row tiles");
  if (M <= 64)
    gemm_f32_mfma_kernel<1, 1, 1, 4><<<grid, 256, 0, stream>>>((const float*)x, (const float*)w, bias,
                                                              (float*)y, M, N, K);
  else
    gemm_f32_mfma_kernel<2, 2, 2, 2><<<grid, 256, 0, stream>>>((const float*)x, (const float*)w, bias,
                                                              (float*)y, M, N, K);
  return sl_launch_status();
}
#endif

// ------------------------------------------------ few rows on the matrix cores
#if !defined(SL_F32)
// y[M, N] for M <= 64 in bfloat16: bound by streaming W from HBM once.
//
// W comes in the tiled layout that `sl_tile_weight` makes of the row-major
// matrix: [N / 16][K / 32][64 lanes][8], lane = 16 * (k / 8 % 4) + n % 16,
// which is the A operand of mfma 16x16x32 as it sits in registers.  One load
// instruction of a wavefront is then 1 KB of consecutive memory and a
// wavefront's share of K one consecutive run; measured on MI355X this streams
// 10-30 % faster than 16 rows x 64 bytes out of the row-major matrix.
//
// A workgroup of 8 wavefronts owns 16 columns of y; each wavefront takes an
// eighth of K and the eight partial tiles are summed through LDS.  Per k-step
// one mfma per block of 16 rows of x: A = W tile, B = 16 rows of x (rows beyond
// M repeat the last row and are not stored).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// Eight weights that this kernel reads once and nobody reads again before the caches have
// turned over: loaded with the streaming hint, so that they do not push x and the partial
// results out of the caches (MI355X, 1 GiB read once: 7.0 TB/s with the hint, 6.3 without).
__device__ __forceinline__ bf16x8 stream_load(const __bf16* p) {
  return __builtin_nontemporal_load((const bf16x8*)p);
}

//
// GATED: the 16 rows of a tile are 8 gate rows followed by the 8 up rows of the
// same channels; the workgroup then writes silu(gate) * up, 8 columns of an
// [M, N / 2] result, instead of 16 columns of y (servelab/parallel/tp_model.py:68).
//
// Residual add and RMSNorm fused into the products around them (decode steps
// are bound by the number of kernels as much as by bytes):
//   PRODUCER  the product's result is a delta of the residual stream.  The
//             workgroup adds it to its 16 columns of the float stream, writes
//             the stream times the next norm's gain in bfloat16 ("un-normalised
//             rows": everything of y = x * rsqrt(mean x^2 + eps) * w but the
//             rsqrt), and the sum of squares of its 16 columns per row into
//             parts[workgroup][16].
//   CONSUMER  x are such un-normalised rows; the workgroup first adds up the
//             parts in a fixed order (so the result does not depend on timing),
//             and scales row m of the result by rsqrt(sum / K + eps) before
//             the bias.  `rows` optionally picks which rows of x are multiplied.
#define SL_MAX_PARTS_PER_THREAD 16      // 32 * 16 parts of 16 columns: rows of up to 8192 values
                                        // (8 per thread, and fewer registers, for rows of up to 4096)

struct NormFusion {
  const float* in_parts;     // CONSUMER: [in_nparts][16] sums of squares by row
  int in_nparts;
  float eps;
  const int* rows;           // CONSUMER: result row m reads row rows[m] of x, or nullptr
  float* resid;              // PRODUCER: float stream [M, N], updated in place
  const float* next_w;       // PRODUCER: gain of the norm that reads the stream next [N]
  float* out_parts;          // PRODUCER: [gridDim.x][16]
  // Few rows of activations "tiled by k-step": element (m, k) of [M, K] at (k / 32) * (M * 32) + m * 32 + k % 32, so
  // that the 64 bytes a row contributes to a k-step lie beside the other rows' (M * 64 contiguous bytes a k-step
  // instead of M pieces K * 2 bytes apart: half as many cache lines touched per load of x; down of the 7B shape at
  // 8 rows: 27.9 -> 25.1 us).  Only between the few-rows kernels: what a gated product or a producer writes (y_tiled)
  // for the product that reads it (x_tiled: the number of rows M the tensor was written with, 0 = plain rows).
  int x_tiled;
  int y_tiled;
  // PRODUCER: rows of W per tile, 8..16 and even (W then lies as [ceil(N / th)][K / 32][4][th][8], see
  // sl_tile_weight).  A product of few rows takes as long as its busiest CU needs to pull its tiles of W
  // and its re-read of x, so a matrix whose 16-row tiles do not go round the CUs evenly gets lower tiles
  // that do (N = 5120 on 256 CUs: 512 tiles of 10 rows instead of 320 of 16).  Other forms: 16.
  int th;
  int pair_x;                // at most 8 rows and one tile a workgroup: a load of x takes two k-steps (see stream_k2)
};

// Rotary embedding and the write to the cache pages fused into the q/k/v
// product (ROPE): the rows of W are ordered so that a tile of 16 result columns
// of a q or k head holds channels 8b..8b+7 and their partners rot/2+8b..rot/2+8b+7
// (rot: the rotated width, the whole head for Qwen2; tiles beyond it pass unrotated);
// the epilogue rotates each pair, writes q into the result buffer and the
// rotated k and the v of token m into the cache row slots[m]
// (servelab/parallel/tp_model.py:128-129).  q and the cached k keep that
// channel order (scores do not depend on it); v is in its own order.
struct RopeStore {
  const float* cosv;         // [M, rot / 2] or nullptr (no rotation)
  const float* sinv;
  const int* slots;          // [M] cache rows, or nullptr (nothing is written)
  __bf16* kc;                // [pages, nkv, page, D]
  __bf16* vc;                // [pages, nkv, D, page]
  int nh, nkv, D, page;
  int rot;                   // the first rot channels of a head are rotated (rot % 16 == 0), the rest pass
  float qscale;              // q heads are multiplied by this before their rounding (1: as they are)
};

// NT tiles (16 columns of y each) per workgroup share every load of x: with 8
// to 16 rows the re-reads of x through L1 are a third to a half of all bytes a
// CU pulls, and halving them shows (MI355X, gate/up of the 7B shape at 16 rows:
// 66 us with one tile).  Matrices with few tiles keep one tile per workgroup so
// that every CU has work.
template <bool GATED, bool CONSUMER, bool PRODUCER, int PARTS, bool ROPE = false, int NT = 1, int WAVES = 8>
__global__ __launch_bounds__(64 * WAVES) void gemm_skinny_kernel(
    const __bf16* __restrict__ x, const __bf16* __restrict__ wt, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32, const NormFusion F,
    const RopeStore R = RopeStore{}) {
  constexpr int U = NT == 1 ? 8 : 4;
  static_assert(WAVES == 8 || !CONSUMER, "the shares of the sums of squares are laid out for 512 threads");
  __shared__ f32x4 red[NT][WAVES][64];
  __shared__ float wsum[WAVES][16];
  // the wavefront's index as a scalar: what depends on it (its share of K, its tiles) then steers
  // real branches; matrix instructions ignore the execution mask, so they must not sit under a
  // condition the compiler takes for divergent and may turn into masking
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int lane = threadIdx.x % 64, i = lane & 15, gq = lane >> 4;
  const int th = PRODUCER ? F.th : 16;
  const int ntiles = (N + th - 1) / th;
  const int KT = K / 32;
  const int ks0 = (int)((long long)KT * wave / WAVES), ks1 = (int)((long long)KT * (wave + 1) / WAVES);
  const __bf16* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int tile = blockIdx.x * NT + t < ntiles ? blockIdx.x * NT + t : ntiles - 1;
    // (lanes of rows a lower tile does not have read its last row; their columns of the result are dropped)
    wp[t] = wt + ((size_t)tile * KT * (4 * th) + gq * th + (i < th ? i : th - 1)) * 8;
  }
  int xrow = i < M ? i : M - 1;
  if (CONSUMER && F.rows != nullptr) xrow = F.rows[xrow];
  const __bf16* xp = F.x_tiled ? x + (size_t)xrow * 32 + 8 * gq : x + (size_t)xrow * K + 8 * gq;
  const size_t xstep = F.x_tiled ? (size_t)F.x_tiled * 32 : 32;     // elements from one k-step of a row to the next
  // Loads that only the epilogue needs are issued here, before W streams, so
  // that their latency is hidden: the consumer's share of the sums of squares
  // (thread t takes parts t / 16, t / 16 + 32, ... of row t % 16) and the
  // producer's elements of the stream and of the next gain.
  float pv[PARTS];
  if (CONSUMER) {
#pragma unroll
    for (int j = 0; j < PARTS; ++j) {
      const int p = threadIdx.x / 16 + 32 * j;
      pv[j] = p < F.in_nparts ? F.in_parts[p * 16 + i] : 0.f;
    }
  }
  const int em = threadIdx.x / 16;                                   // epilogue row of threads < 256
  float r_old[NT], g_next[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int en = (blockIdx.x * NT + t) * th + threadIdx.x % 16;
    r_old[t] = g_next[t] = 0.f;
    if (PRODUCER && threadIdx.x < 256 && em < M && (int)(threadIdx.x % 16) < th && en < N) {
      r_old[t] = F.resid[(size_t)em * N + en];
      g_next[t] = F.next_w[en];
    }
  }
  // (ROPE: the bias, the angle's cosine and sine and the cache row of this thread's element)
  float b_pre[NT], c_pre[NT], s_pre[NT];
  int slot_pre = 0;
  if (ROPE) {
    if (threadIdx.x < 256 && em < M && R.slots != nullptr) slot_pre = R.slots[em];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int en = (blockIdx.x * NT + t) * 16 + threadIdx.x % 16;
      b_pre[t] = 0.f;
      c_pre[t] = 1.f;
      s_pre[t] = 0.f;
      if (threadIdx.x < 256 && em < M && en < N) {
        if (bias != nullptr) b_pre[t] = bias[en];
        const int hd = en / R.D, p = en % R.D;
        if (R.cosv != nullptr && hd < R.nh + R.nkv && p < R.rot) {
          const int j = 8 * (p / 16) + p % 8, half = R.rot / 2;
          c_pre[t] = R.cosv[(size_t)em * half + j];
          s_pre[t] = R.sinv[(size_t)em * half + j];
        }
      }
    }
  }
  f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  // The K loop, written once for plain rows of x (a constant step from one k-step to the next,
  // folded into the loads' offsets) and once for rows laid out by k-step.
  auto stream_k = [&](auto tiled_tag, auto th_tag) {
    const size_t xs_ = decltype(tiled_tag)::value ? xstep : (size_t)32;
    constexpr size_t WS = 32 * decltype(th_tag)::value;             // elements of W from one k-step of a tile to the next
    int ks = ks0;
    for (; ks + U <= ks1; ks += U) {
      bf16x8 a[NT][U];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) a[t][u] = stream_load(wp[t] + WS * (size_t)(ks + u));
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const bf16x8 bv = *(const bf16x8*)(xp + xs_ * (size_t)(ks + u));
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], bv, acc[t], 0, 0, 0);
      }
    }
    if (ks < ks1) {
      // the last k-steps, fewer than U: all their loads are issued before the
      // first product, so they cost one trip to memory, not one each
      bf16x8 a[NT][U], bv[U];
#pragma unroll
      for (int u = 0; u < U - 1; ++u)
        if (ks + u < ks1) {
#pragma unroll
          for (int t = 0; t < NT; ++t) a[t][u] = stream_load(wp[t] + WS * (size_t)(ks + u));
          bv[u] = *(const bf16x8*)(xp + xs_ * (size_t)(ks + u));
        }
#pragma unroll
      for (int u = 0; u < U - 1; ++u)
        if (ks + u < ks1) {
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], bv[u], acc[t], 0, 0, 0);
        }
    }
  };
  // The same loop for at most 8 rows of x and one tile: a load of x takes two k-steps.  The matrix
  // instruction has 16 columns for the rows of x; with at most 8 rows the lanes of columns 8..15 load the
  // same rows one k-step further on, the products of even k-steps go to one accumulator (columns 0..7
  // valid) and those of odd k-steps to a second (columns 8..15 valid), and the second is added to the
  // first at the end.  Half as many loads of x: a load takes a place in the CU's queue of outstanding
  // requests whatever its size, and that queue is what these kernels run on.
  f32x4 acc_odd = f32x4{0.f, 0.f, 0.f, 0.f};
  auto stream_k2 = [&](auto tiled_tag, auto th_tag) {
    static_assert(NT == 1 && U % 2 == 0, "two k-steps a load of x: one tile, an even number of loads in flight");
    const size_t xs_ = decltype(tiled_tag)::value ? xstep : (size_t)32;
    constexpr size_t WS = 32 * decltype(th_tag)::value;
    int row = (i & 7) < M ? (i & 7) : M - 1;
    if (CONSUMER && F.rows != nullptr) row = F.rows[row];
    const __bf16* x0 = (F.x_tiled ? x + (size_t)row * 32 + 8 * gq : x + (size_t)row * K + 8 * gq);
    const __bf16* x2 = x0 + (i >= 8 ? xs_ : 0);          // columns 8..15: one k-step further
    int ks = ks0;
    for (; ks + U <= ks1; ks += U) {
      bf16x8 a[U];
#pragma unroll
      for (int u = 0; u < U; ++u) a[u] = stream_load(wp[0] + WS * (size_t)(ks + u));
#pragma unroll
      for (int u = 0; u < U; u += 2) {
        const bf16x8 bv = *(const bf16x8*)(x2 + xs_ * (size_t)(ks + u));
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], bv, acc[0], 0, 0, 0);
        acc_odd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u + 1], bv, acc_odd, 0, 0, 0);
      }
    }
    if (ks < ks1) {
      // the last k-steps, fewer than U, in one trip to memory; an odd one at the end has its x in all
      // 16 columns (nothing lies one k-step further that would be this wavefront's, or the row's)
      bf16x8 a[U], bv[U / 2], last;
#pragma unroll
      for (int u = 0; u < U - 1; ++u)
        if (ks + u < ks1) a[u] = stream_load(wp[0] + WS * (size_t)(ks + u));
#pragma unroll
      for (int u = 0; u + 1 < U - 1; u += 2)
        if (ks + u + 1 < ks1) bv[u / 2] = *(const bf16x8*)(x2 + xs_ * (size_t)(ks + u));
      const bool odd = (ks1 - ks) & 1;
      if (odd) last = *(const bf16x8*)(x0 + xs_ * (size_t)(ks1 - 1));
#pragma unroll
      for (int u = 0; u + 1 < U - 1; u += 2)
        if (ks + u + 1 < ks1) {
          acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], bv[u / 2], acc[0], 0, 0, 0);
          acc_odd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u + 1], bv[u / 2], acc_odd, 0, 0, 0);
        }
      if (odd) {
        // (its W is a[ks1 - 1 - ks]: picked by a chain of selects, the index is the same for the wavefront)
        bf16x8 w_last = a[0];
#pragma unroll
        for (int u = 1; u < U - 1; ++u)
          if (ks + u == ks1 - 1) w_last = a[u];
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_last, last, acc[0], 0, 0, 0);
      }
    }
  };
  // (each form of the loop is straight-line code with constant steps; the tile height is a run-time
  // choice only for producers)
  auto stream_th = [&](auto th_tag) {
    if constexpr (NT == 1) {
      if (M <= 8 && F.pair_x) {
        if (F.x_tiled) stream_k2(std::true_type{}, th_tag);
        else stream_k2(std::false_type{}, th_tag);
        return;
      }
    }
    if (F.x_tiled) stream_k(std::true_type{}, th_tag);
    else stream_k(std::false_type{}, th_tag);
  };
  if constexpr (!PRODUCER) {
    stream_th(std::integral_constant<int, 16>{});
  } else {
    if (th == 16) stream_th(std::integral_constant<int, 16>{});
    else if (th == 14) stream_th(std::integral_constant<int, 14>{});
    else if (th == 12) stream_th(std::integral_constant<int, 12>{});
    else if (th == 10) stream_th(std::integral_constant<int, 10>{});
    else stream_th(std::integral_constant<int, 8>{});
  }
  if constexpr (NT == 1) {
    if (M <= 8 && F.pair_x) {         // column m + 8 of the odd k-steps' sums belongs to column m
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[0][r] += __shfl(acc_odd[r], lane + 8, 64);
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) red[t][wave][lane] = acc[t];
  if (CONSUMER) {            // this wavefront's share of the sums of squares, by row
    float sacc = 0.f;
#pragma unroll
    for (int j = 0; j < PARTS; ++j) sacc += pv[j];
    sacc += __shfl_xor(sacc, 16, 64);
    sacc += __shfl_xor(sacc, 32, 64);
    if (lane < 16) wsum[wave][lane] = sacc;
  }
  __syncthreads();
  auto inv_of = [&](int m) {   // rsqrt(mean x^2 + eps) of the row of x behind result row m
    const int tok = F.rows != nullptr ? F.rows[m] : m;
    float ss = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) ss += wsum[wv][tok];
    return rsqrtf(ss / (float)K + F.eps);
  };
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int tile = blockIdx.x * NT + t;
    if (tile >= ntiles) break;
    const int n0 = tile * th;
    // lane (m + 16 (n_local / 4)) holds y[m, n_local] in element n_local % 4
    if (GATED) {
      if (threadIdx.x < 128) {
        const int m = threadIdx.x / 8, j = threadIdx.x % 8;
        const int n = tile * 8 + j;
        if (m < M && n < N / 2) {
          float gsum = 0.f, usum = 0.f;
#pragma unroll
          for (int wv = 0; wv < WAVES; ++wv) {
            gsum += red[t][wv][m + 16 * (j / 4)][j % 4];
            usum += red[t][wv][m + 16 * (2 + j / 4)][j % 4];
          }
          if (CONSUMER) {
            const float inv = inv_of(m);
            gsum *= inv;
            usum *= inv;
          }
          const size_t at = F.y_tiled ? (size_t)(n / 32) * (M * 32) + m * 32 + n % 32 : (size_t)m * (N / 2) + n;
          ((__bf16*)y)[at] = (__bf16)(gsum / (1.f + expf(-gsum)) * usum);
        }
      }
      continue;
    }
    if (threadIdx.x < 256) {
      const int m = em, n_local = threadIdx.x % 16, n = n0 + n_local;
      const bool live = m < M && n_local < th && n < N;
      float s = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) s += red[t][wv][m + 16 * (n_local / 4)][n_local % 4];
      if (CONSUMER && live) s *= inv_of(m);
      if (ROPE) {
        s += b_pre[t];
        const float partner = __shfl_xor(s, 8, 64);      // the other half of the pair, same row
        if (!live) continue;
        const int hd = n / R.D, p = n % R.D;
        const int slot = slot_pre;
        if (hd < R.nh + R.nkv) {
          float val = s;
          if (R.cosv != nullptr && p < R.rot)
            val = p % 16 < 8 ? s * c_pre[t] - partner * s_pre[t] : s * c_pre[t] + partner * s_pre[t];
          if (hd < R.nh) {
            ((__bf16*)y)[(size_t)m * N + n] = (__bf16)(val * R.qscale);
          } else if (R.slots != nullptr) {
            R.kc[(((size_t)(slot / R.page) * R.nkv + (hd - R.nh)) * R.page + slot % R.page) * R.D + p] = (__bf16)val;
          }
        } else if (R.slots != nullptr) {
          R.vc[(((size_t)(slot / R.page) * R.nkv + (hd - R.nh - R.nkv)) * R.D + p) * R.page + slot % R.page] = (__bf16)s;
        }
        continue;
      }
      if (live && bias != nullptr) s += bias[n];
      if (PRODUCER) {
        float sq = 0.f;
        if (live) {
          const float r = r_old[t] + s;
          F.resid[(size_t)m * N + n] = r;
          const size_t at = F.y_tiled ? (size_t)(n / 32) * (M * 32) + m * 32 + n % 32 : (size_t)m * N + n;
          ((__bf16*)y)[at] = (__bf16)(r * g_next[t]);
          sq = r * r;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);     // over the 16 columns of row m
        if (n_local == 0) F.out_parts[(size_t)tile * 16 + m] = sq;
      } else if (live) {
        if (out_f32) ((float*)y)[(size_t)m * N + n] = s;
        else ((__bf16*)y)[(size_t)m * N + n] = (__bf16)s;
      }
    }
  }
}

// CUs of the current device (asked once per device).
static int device_cus() {
  static int cus[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cus[dev] == 0 &&
      hipDeviceGetAttribute(&cus[dev], hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  return cus[dev];
}

// wt: W in the tiled layout, ceil(N / 16) * 16 rows (rows beyond N are zero).
// At most 16 rows.  Fusion: in_parts != nullptr makes x un-normalised rows
// (consumer), resid != nullptr makes the result a delta of the stream (producer).
// pair_tiles: two tiles of W per workgroup.  th: rows of W per tile (16, or what sl_tile_weight was given
// for a producer's matrix).
extern "C" const char* sl_gemm_skinny(const void* x, const void* wt, const float* bias, void* y,
                                      int M, int N, int K, int out_f32, int gated,
                                      const float* in_parts, int in_nparts, float eps,
                                      const int* rows, float* resid, const float* next_w,
                                      float* out_parts, const RopeStore* rope, int pair_tiles,
                                      int x_tiled, int y_tiled, int th, int pair_x, hipStream_t stream) {
  SL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_skinny: sizes must be positive");
  SL_CHECK(M <= 16, "gemm_skinny: at most 16 rows");
  SL_CHECK(K % 32 == 0, "gemm_skinny: K must be a multiple of 32");
  SL_CHECK(!gated || (N % 16 == 0 && bias == nullptr && !out_f32),
           "gemm_skinny: the gated form needs N % 16 == 0, no bias, activation output");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)wt % 16) == 0,
           "gemm_skinny: x and W must be 16-byte aligned");
  const bool consumer = in_parts != nullptr, producer = resid != nullptr;
  SL_CHECK(!(consumer && producer), "gemm_skinny: a product is a consumer or a producer, not both");
  SL_CHECK(!consumer || (in_nparts > 0 && eps > 0.f), "gemm_skinny: a consumer needs parts and eps");
  SL_CHECK(!consumer || in_nparts <= 32 * SL_MAX_PARTS_PER_THREAD,
           "gemm_skinny: un-normalised rows of more than 8192 values");
  SL_CHECK(rows == nullptr || consumer, "gemm_skinny: a row gather belongs to a consumer");
  SL_CHECK(!producer || (next_w != nullptr && out_parts != nullptr && !gated && !out_f32),
           "gemm_skinny: a producer needs the next gain and a parts buffer, and is neither gated nor float");
  SL_CHECK(th == 16 || (producer && th >= 8 && th < 16 && th % 2 == 0),
           "gemm_skinny: tiles of 16 rows, or of 8, 10, 12 or 14 for a producer");
  if (M == 0) return nullptr;
  const dim3 grid((N + th - 1) / th);
  const __bf16* xx = (const __bf16*)x;
  const __bf16* ww = (const __bf16*)wt;
  SL_CHECK(x_tiled >= 0 && (x_tiled == 0 || rows != nullptr || x_tiled == M),
           "gemm_skinny: x tiled by k-step has as many rows as the product, or rows are picked from it");
  SL_CHECK(!y_tiled || (gated && (N / 2) % 32 == 0) || (resid != nullptr && N % 32 == 0),
           "gemm_skinny: a tiled result is a gated one or a producer's, of a multiple of 32 columns");
  const NormFusion F{in_parts, in_nparts, eps, rows, resid, next_w, out_parts, x_tiled, y_tiled, th, pair_x};
  const bool few = in_nparts <= 32 * 8;
  if (rope != nullptr) {
    const RopeStore R = *rope;
    SL_CHECK(!gated && !producer && !out_f32, "gemm_skinny: q/k/v with rotary is a plain or a consumer product");
    SL_CHECK(R.D % 16 == 0 && R.nh > 0 && R.nkv > 0 && N == (R.nh + 2 * R.nkv) * R.D,
             "gemm_skinny: q/k/v columns must be (heads + 2 kv heads) * head_dim, head_dim % 16 == 0");
    SL_CHECK((R.cosv == nullptr) == (R.sinv == nullptr), "gemm_skinny: cos and sin go together");
    SL_CHECK(R.rot >= 0 && R.rot <= R.D && R.rot % 16 == 0 && (R.cosv == nullptr || R.rot > 0),
             "gemm_skinny: the rotated width must be a multiple of 16, at most head_dim");
    SL_CHECK(R.slots == nullptr || (R.kc != nullptr && R.vc != nullptr && R.page > 0),
             "gemm_skinny: cache rows need the pages");
    const dim3 grid2(((N + 15) / 16 + 1) / 2);
    if (pair_tiles) {
      if (!consumer) gemm_skinny_kernel<false, false, false, 1, true, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, R);
      else if (few) gemm_skinny_kernel<false, true, false, 8, true, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, R);
      else gemm_skinny_kernel<false, true, false, 16, true, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, R);
    } else {
      if (!consumer) gemm_skinny_kernel<false, false, false, 1, true><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, R);
      else if (few) gemm_skinny_kernel<false, true, false, 8, true><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, R);
      else gemm_skinny_kernel<false, true, false, 16, true><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, R);
    }
    return sl_launch_status();
  }
  const RopeStore none{};
  if (pair_tiles) {                              // two tiles per workgroup
    const dim3 grid2((grid.x + 1) / 2);
    if (producer) gemm_skinny_kernel<false, false, true, 1, false, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, none);
    else if (consumer && gated && few) gemm_skinny_kernel<true, true, false, 8, false, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, none);
    else if (consumer && gated) gemm_skinny_kernel<true, true, false, 16, false, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, none);
    else if (consumer && few) gemm_skinny_kernel<false, true, false, 8, false, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32, F, none);
    else if (consumer) gemm_skinny_kernel<false, true, false, 16, false, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32, F, none);
    else if (gated) gemm_skinny_kernel<true, false, false, 1, false, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F, none);
    else gemm_skinny_kernel<false, false, false, 1, false, 2><<<grid2, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32, F, none);
    return sl_launch_status();
  }
  // a matrix with fewer tiles than the chip has CUs leaves each CU one workgroup: sixteen
  // wavefronts then have twice the loads in flight (7B shape, batch 1: 349 -> 356 tok/s)
  if (producer && (int)grid.x <= device_cus() && K >= 2048) gemm_skinny_kernel<false, false, true, 1, false, 1, 16><<<grid, 1024, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F);
  else if (producer) gemm_skinny_kernel<false, false, true, 1><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F);
  else if (consumer && gated && few) gemm_skinny_kernel<true, true, false, 8><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F);
  else if (consumer && gated) gemm_skinny_kernel<true, true, false, 16><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F);
  else if (consumer && few) gemm_skinny_kernel<false, true, false, 8><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32, F);
  else if (consumer) gemm_skinny_kernel<false, true, false, 16><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32, F);
  else if (gated) gemm_skinny_kernel<true, false, false, 1><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0, F);
  else gemm_skinny_kernel<false, false, false, 1><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32, F);
  return sl_launch_status();
}

// ------------------------------- few rows, x resident, tile after tile
// The consumer products with many tiles (gate/up, the head).  The kernel above
// starts a workgroup per tile, and each one begins by asking for its share of
// the sums of squares and for x (with 8 rows a third of the bytes it pulls
// through L1) before its weights stream.  Here a workgroup stays: grid =
// what the chip holds at once, tiles blockIdx.x, blockIdx.x + grid, ...  A
// wavefront keeps its share of K throughout (NS k-steps, the same for all
// eight: K = 256 NS), so its part of x sits in registers, the row scales are
// computed once, and the loads of the next tile's weights are issued as this
// tile's are used up (a ring of R k-steps per wavefront), so they are in flight
// during the reduction and the epilogue.  NS is a template argument: the loop is
// straight-line code whose every wait the compiler can count (with a run-time
// number of steps it waited for all loads at every step).  Result as
// gemm_skinny_kernel's CONSUMER forms, bit for bit: the same products in the same
// order.
template <bool GATED, int PARTS, int NS, int R>
__global__ __launch_bounds__(512) void gemm_resident_kernel(
    const __bf16* __restrict__ x, const __bf16* __restrict__ wt, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int out_f32, const NormFusion F) {
  constexpr int WAVES = 8, KT = WAVES * NS, K = 32 * KT;
  static_assert(NS % R == 0, "the ring divides the steps");
  __shared__ f32x4 red[2][WAVES][64];
  __shared__ float wsum[WAVES][16];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);     // (a scalar: see gemm_skinny_kernel)
  const int lane = threadIdx.x % 64, i = lane & 15, gq = lane >> 4;
  const int ntiles = (N + 15) / 16;
  const int ks0 = NS * wave;
  int xrow = i < M ? i : M - 1;
  if (F.rows != nullptr) xrow = F.rows[xrow];
  const __bf16* xp = F.x_tiled ? x + (size_t)ks0 * F.x_tiled * 32 + (size_t)xrow * 32 + 8 * gq
                               : x + (size_t)xrow * K + 32 * (size_t)ks0 + 8 * gq;
  const size_t xstep = F.x_tiled ? (size_t)F.x_tiled * 32 : 32;
  const __bf16* wbase = wt + ((size_t)ks0 * 64 + lane) * 8;
  constexpr size_t tile_stride = (size_t)KT * 512;
  bf16x8 a[R];
  int tile = blockIdx.x;                           // < ntiles: the grid is no larger
#pragma unroll
  for (int u = 0; u < R; ++u) a[u] = stream_load(wbase + tile * tile_stride + 512 * u);
  float pv[PARTS];
#pragma unroll
  for (int j = 0; j < PARTS; ++j) {
    const int p = threadIdx.x / 16 + 32 * j;
    pv[j] = p < F.in_nparts ? F.in_parts[p * 16 + i] : 0.f;
  }
  bf16x8 xr[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) xr[s] = *(const bf16x8*)(xp + xstep * s);
  {
    float sacc = 0.f;
#pragma unroll
    for (int j = 0; j < PARTS; ++j) sacc += pv[j];
    sacc += __shfl_xor(sacc, 16, 64);
    sacc += __shfl_xor(sacc, 32, 64);
    if (lane < 16) wsum[wave][lane] = sacc;
  }
  __syncthreads();
  // the epilogue row of this thread and its scale
  const int em = GATED ? threadIdx.x / 8 : threadIdx.x / 16;
  float inv = 0.f;
  if (em < M) {
    const int tok = F.rows != nullptr ? F.rows[em] : em;
    float ss = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) ss += wsum[wv][tok];
    inv = rsqrtf(ss / (float)K + F.eps);
  }
  // one tile: its products, the refills of the ring, the reduction and the epilogue
  auto one_tile = [&](auto has_next, int buf) {
    const __bf16* wcur = wbase + tile * tile_stride;
    const __bf16* wnext = wcur + gridDim.x * tile_stride;
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s % R], xr[s], acc, 0, 0, 0);
      if (s + R < NS) a[s % R] = stream_load(wcur + 512 * (s + R));
      else if (decltype(has_next)::value) a[s % R] = stream_load(wnext + 512 * (s + R - NS));
    }
    red[buf][wave][lane] = acc;
    __syncthreads();
    // lane (m + 16 (n_local / 4)) holds y[m, n_local] in element n_local % 4
    if (GATED) {
      if (threadIdx.x < 128) {
        const int m = em, j = threadIdx.x % 8;
        const int col = tile * 8 + j;
        if (m < M && col < N / 2) {
          float gsum = 0.f, usum = 0.f;
#pragma unroll
          for (int wv = 0; wv < WAVES; ++wv) {
            gsum += red[buf][wv][m + 16 * (j / 4)][j % 4];
            usum += red[buf][wv][m + 16 * (2 + j / 4)][j % 4];
          }
          gsum *= inv;
          usum *= inv;
          const size_t at = F.y_tiled ? (size_t)(col / 32) * (M * 32) + m * 32 + col % 32 : (size_t)m * (N / 2) + col;
          ((__bf16*)y)[at] = (__bf16)(gsum / (1.f + expf(-gsum)) * usum);
        }
      }
    } else if (threadIdx.x < 256) {
      const int m = em, n_local = threadIdx.x % 16, col = tile * 16 + n_local;
      if (m < M && col < N) {
        float sum = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) sum += red[buf][wv][m + 16 * (n_local / 4)][n_local % 4];
        sum *= inv;
        if (bias != nullptr) sum += bias[col];
        if (out_f32) ((float*)y)[(size_t)m * N + col] = sum;
        else ((__bf16*)y)[(size_t)m * N + col] = (__bf16)sum;
      }
    }
  };
  int buf = 0;
  for (; tile + (int)gridDim.x < ntiles; tile += gridDim.x, buf ^= 1) one_tile(std::true_type{}, buf);
  one_tile(std::false_type{}, buf);
}

// How many workgroups of 512 threads of a kernel the current device holds at once.
template <typename Kernel>
static int resident_workgroups(Kernel kernel) {
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 512, 0) != hipSuccess) return 0;
  return device_cus() * per_cu;
}

// The row lengths sl_gemm_resident is built for (K = 256 * NS: the number of k-steps a
// wavefront takes is a template argument, so that the compiler can count the loads in
// flight), each with the number of k-steps R a wavefront asks for at once.  They are the
// widths whose consumers have many tiles per CU among the models this was measured on
// (1536, 2048, 3584, 4096, 5120); every other K, and K = 8192, where this form measured
// slower, takes sl_gemm_skinny, which gives the same result bit for bit.
#define SL_RESIDENT_WIDTHS(X) X(6, 6) X(8, 8) X(14, 14) X(16, 16) X(20, 10)
constexpr int resident_parts_per_thread(int NS) { return NS <= 16 ? 8 : 16; }

// How many sums of squares a row (K / 16 or more) the kernel for rows of K values adds up,
// 0 when sl_gemm_resident has no kernel for that K.
extern "C" int sl_gemm_resident_parts(int K) {
  switch (K) {
#define SL_CASE(NS, R) case 256 * NS: return 32 * resident_parts_per_thread(NS);
    SL_RESIDENT_WIDTHS(SL_CASE)
#undef SL_CASE
    default: return 0;
  }
}

// The consumer forms of sl_gemm_skinny (x: un-normalised rows) for matrices of
// many tiles; same arguments, same result.
extern "C" const char* sl_gemm_resident(const void* x, const void* wt, const float* bias, void* y,
                                        int M, int N, int K, int out_f32, int gated,
                                        const float* in_parts, int in_nparts, float eps,
                                        const int* rows, int x_tiled, int y_tiled, hipStream_t stream) {
  SL_CHECK(M >= 0 && N > 0 && K > 0, "gemm_resident: sizes must be positive");
  SL_CHECK(M <= 16, "gemm_resident: at most 16 rows");
  SL_CHECK(sl_gemm_resident_parts(K) > 0, "gemm_resident: no kernel for rows of this length");
  SL_CHECK(!gated || (N % 16 == 0 && bias == nullptr && !out_f32),
           "gemm_resident: the gated form needs N % 16 == 0, no bias, activation output");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)wt % 16) == 0,
           "gemm_resident: x and W must be 16-byte aligned");
  SL_CHECK(in_parts != nullptr && in_nparts > 0 && eps > 0.f, "gemm_resident: needs parts and eps");
  SL_CHECK(in_nparts <= 32 * SL_MAX_PARTS_PER_THREAD, "gemm_resident: un-normalised rows of more than 8192 values");
  if (M == 0) return nullptr;
  const int ntiles = (N + 15) / 16;
  SL_CHECK(!y_tiled || (gated && (N / 2) % 32 == 0), "gemm_resident: a tiled result is a gated one of a multiple of 32 columns");
  SL_CHECK(x_tiled >= 0 && (x_tiled == 0 || rows != nullptr || x_tiled == M),
           "gemm_resident: x tiled by k-step has as many rows as the product, or rows are picked from it");
  const NormFusion F{in_parts, in_nparts, eps, rows, nullptr, nullptr, nullptr, x_tiled, y_tiled};
  const __bf16* xx = (const __bf16*)x;
  const __bf16* ww = (const __bf16*)wt;
#define SL_RESIDENT(G, NS, R)                                                                   \
  do {                                                                                          \
    constexpr int PARTS = resident_parts_per_thread(NS);   /* K / 16 parts or more, 32 per pass */ \
    SL_CHECK(in_nparts <= 32 * PARTS, "gemm_resident: more sums of squares a row than this form adds up"); \
    static int slots = 0;                                                                       \
    if (slots == 0) slots = resident_workgroups(gemm_resident_kernel<G, PARTS, NS, R>);         \
    SL_CHECK(slots > 0, "gemm_resident: the device holds no workgroup of this kernel");         \
    const int rounds = (ntiles + slots - 1) / slots;                                            \
    const int grid = (ntiles + rounds - 1) / rounds;                                            \
    gemm_resident_kernel<G, PARTS, NS, R><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N,      \
                                                                   out_f32, F);                 \
  } while (0)
#define SL_RESIDENT_CASE(NS, R)                                     \
  case 256 * NS:                                                    \
    if (gated) SL_RESIDENT(true, NS, R); else SL_RESIDENT(false, NS, R); \
    break;
  switch (K) { SL_RESIDENT_WIDTHS(SL_RESIDENT_CASE) }
#undef SL_RESIDENT_CASE
#undef SL_RESIDENT
  return sl_launch_status();
}

// ----------------------------------------------- 17 to 64 rows, matrix cores
// With more rows of x the few-rows kernel above would read all of x once per
// 16 rows of W, several times the bytes of W itself.  Here a workgroup owns two
// tiles (32 rows) of W and all rows of x: per k-step 2 loads of W, MB loads of
// x and 2 * MB mfma, so x is read half as often.  The 8 wavefronts split K and
// reduce through LDS, one tile of W at a time.  (Measured on MI355X against
// 1 and 4 tiles per workgroup and against deeper unrolling: this is the
// fastest of them for the projection sizes of 7B to 72B models at 32 and 64 rows.)
template <int MB, bool GATED>
__global__ __launch_bounds__(512) void gemm_wide_kernel(
    const __bf16* __restrict__ x, const __bf16* __restrict__ wt, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32) {
  constexpr int WAVES = 8, U = 2, NT = 2;
  __shared__ f32x4 red[WAVES][MB][64];
  // the wavefront's index as a scalar: what depends on it (its share of K, its tiles) then steers
  // real branches; matrix instructions ignore the execution mask, so they must not sit under a
  // condition the compiler takes for divergent and may turn into masking
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int lane = threadIdx.x % 64, i = lane & 15, gq = lane >> 4;
  const int ntiles = (N + 15) / 16;
  const int tile0 = blockIdx.x * NT;
  const int KT = K / 32;
  const int ks0 = (int)((long long)KT * wave / WAVES), ks1 = (int)((long long)KT * (wave + 1) / WAVES);
  const __bf16* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int tile = tile0 + t < ntiles ? tile0 + t : ntiles - 1;
    wp[t] = wt + ((size_t)tile * KT * 64 + lane) * 8;
  }
  const __bf16* xp[MB];
#pragma unroll
  for (int b = 0; b < MB; ++b) {
    const int m = 16 * b + i < M ? 16 * b + i : M - 1;
    xp[b] = x + (size_t)m * K + 8 * gq;
  }
  f32x4 acc[NT][MB];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  // Groups of U k-steps.  Up to 32 rows, two sets of registers: the loads of
  // the next group are in flight while this one is multiplied, and every load
  // of the loop is unconditional so that the waits can count them exactly
  // (MI355X, q/k/v of the 7B shape at 32 rows: 14.8 us against 17.1 us).  With
  // 64 rows the second set costs a wavefront per SIMD and measured slower
  // (21.2 us against 19.7 us), so there a group is loaded, then multiplied.
  constexpr bool AHEAD = MB <= 2;
  const int nfull = (ks1 - ks0) / U;
  auto load_group = [&](int g, bf16x8 (&a)[NT][U], bf16x8 (&bv)[MB][U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t ks = (size_t)(ks0 + g * U + u);
#pragma unroll
      for (int t = 0; t < NT; ++t) a[t][u] = stream_load(wp[t] + 512 * ks);
#pragma unroll
      for (int b = 0; b < MB; ++b) bv[b][u] = *(const bf16x8*)(xp[b] + 32 * ks);
    }
  };
  auto multiply_group = [&](const bf16x8 (&a)[NT][U], const bf16x8 (&bv)[MB][U]) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int b = 0; b < MB; ++b)
          acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], bv[b][u], acc[t][b], 0, 0, 0);
  };
  if (!AHEAD) {
    for (int ks = ks0; ks + U <= ks1; ks += U) {
      bf16x8 a[NT][U], bv[MB][U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int t = 0; t < NT; ++t) a[t][u] = stream_load(wp[t] + 512 * (size_t)(ks + u));
#pragma unroll
        for (int b = 0; b < MB; ++b) bv[b][u] = *(const bf16x8*)(xp[b] + 32 * (size_t)(ks + u));
      }
      multiply_group(a, bv);
    }
  } else if (nfull > 0) {
    bf16x8 a0[NT][U], b0[MB][U], a1[NT][U], b1[MB][U];
    load_group(0, a0, b0);
    int g = 0;
    for (; g + 2 < nfull; g += 2) {
      load_group(g + 1, a1, b1);
      multiply_group(a0, b0);
      load_group(g + 2, a0, b0);
      multiply_group(a1, b1);
    }
    if (g + 1 < nfull) {
      load_group(g + 1, a1, b1);
      multiply_group(a0, b0);
      multiply_group(a1, b1);
    } else {
      multiply_group(a0, b0);
    }
  }
  int ks = ks0 + nfull * U;
  for (; ks < ks1; ++ks) {
    bf16x8 bv[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) bv[b] = *(const bf16x8*)(xp[b] + 32 * (size_t)ks);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const bf16x8 a = stream_load(wp[t] + 512 * (size_t)ks);
#pragma unroll
      for (int b = 0; b < MB; ++b)
        acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bv[b], acc[t][b], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    __syncthreads();
#pragma unroll
    for (int b = 0; b < MB; ++b) red[wave][b][lane] = acc[t][b];
    __syncthreads();
    if (tile0 + t >= ntiles) continue;
    if (GATED) {
      // lane (m + 16 (j / 4)) element j % 4 is gate j, lane (m + 16 (2 + j / 4)) its up
      for (int idx = threadIdx.x; idx < MB * 128; idx += WAVES * 64) {
        const int b = idx / 128, rem = idx % 128, m_local = rem / 8, j = rem % 8;
        const int m = 16 * b + m_local, n = (tile0 + t) * 8 + j;
        if (m < M && n < N / 2) {
          float gsum = 0.f, usum = 0.f;
#pragma unroll
          for (int wv = 0; wv < WAVES; ++wv) {
            gsum += red[wv][b][m_local + 16 * (j / 4)][j % 4];
            usum += red[wv][b][m_local + 16 * (2 + j / 4)][j % 4];
          }
          ((__bf16*)y)[(size_t)m * (N / 2) + n] = (__bf16)(gsum / (1.f + expf(-gsum)) * usum);
        }
      }
      continue;
    }
    for (int idx = threadIdx.x; idx < MB * 256; idx += WAVES * 64) {
      const int b = idx / 256, rem = idx % 256, m_local = rem / 16, n_local = rem % 16;
      const int m = 16 * b + m_local, n = (tile0 + t) * 16 + n_local;
      if (m < M && n < N) {
        float sum = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) sum += red[wv][b][m_local + 16 * (n_local / 4)][n_local % 4];
        if (bias != nullptr) sum += bias[n];
        if (out_f32) ((float*)y)[(size_t)m * N + n] = sum;
        else ((__bf16*)y)[(size_t)m * N + n] = (__bf16)sum;
      }
    }
  }
}

extern "C" const char* sl_gemm_wide(const void* x, const void* wt, const float* bias, void* y,
                                    int M, int N, int K, int out_f32, int gated,
                                    hipStream_t stream) {
  SL_CHECK(M > 0 && N > 0 && K > 0, "gemm_wide: sizes must be positive");
  SL_CHECK(M <= 64, "gemm_wide: at most 64 rows");
  SL_CHECK(K % 32 == 0, "gemm_wide: K must be a multiple of 32");
  SL_CHECK(!gated || (N % 16 == 0 && bias == nullptr && !out_f32),
           "gemm_wide: the gated form needs N % 16 == 0, no bias, activation output");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)wt % 16) == 0,
           "gemm_wide: x and W must be 16-byte aligned");
  const dim3 grid(((N + 15) / 16 + 1) / 2);
  const __bf16* xx = (const __bf16*)x;
  const __bf16* ww = (const __bf16*)wt;
  if (gated) {
    if (M <= 32) gemm_wide_kernel<2, true><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0);
    else gemm_wide_kernel<4, true><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, 0);
  } else {
    if (M <= 32) gemm_wide_kernel<2, false><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
    else gemm_wide_kernel<4, false><<<grid, 512, 0, stream>>>(xx, ww, bias, y, M, N, K, out_f32);
  }
  return sl_launch_status();
}

// ------------------------------------ 17 to 128 rows, x staged through LDS
// The kernel above reads x from L2 once per 32 rows of W.  Here a workgroup of
// 4 wavefronts owns 128 rows of W (each wavefront two tiles over the
// workgroup's whole share of K, so nothing is reduced across wavefronts) and
// stages x through LDS in chunks of 128 values of k, already in the order of
// the mfma B operand and double-buffered: x leaves L2 once per 128 rows of W.
// The next chunk of x and of W is loaded while the current one is multiplied.
// When N is small, K is split over `KS` workgroups (grid.y) that write float
// partials [KS, M, N]; `splitk_reduce_kernel` adds them, the bias, and rounds.
template <int MB, int NT, int KC, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemm_mid_kernel(
    const __bf16* __restrict__ x, const __bf16* __restrict__ wt, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32, int gated, int KS) {
  constexpr int THREADS = 64 * WAVES;
  // chunks of W in flight or in use (LDS holds as many of x): three for the workgroups of eight
  // wavefronts where the registers and LDS allow it (gate/up of the 7B shape at 64 rows: 52 -> 49 us);
  // with four wavefronts (K split over workgroups) the third set measured slower (17.1 -> 17.8 us)
  constexpr int DEPTH = MB <= 4 && WAVES == 8 ? 3 : 2;
  __shared__ bf16x8 xs[DEPTH][KC][MB][64];
  // the wavefront's index as a scalar: what depends on it (its share of K, its tiles) then steers
  // real branches; matrix instructions ignore the execution mask, so they must not sit under a
  // condition the compiler takes for divergent and may turn into masking
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int lane = threadIdx.x % 64, i = lane & 15, gq = lane >> 4;
  const int ntiles = (N + 15) / 16;
  // The workgroups share the tiles as evenly as the grid allows: workgroup g of
  // G takes tiles [ntiles g / G, ntiles (g + 1) / G), at most WAVES * NT of
  // them; wavefront v takes the v-th and the (WAVES + v)-th.  A wavefront
  // without a (second) tile loads its first one again, which hits L1 and costs
  // no bandwidth, and drops the result.
  const int tbeg = (int)((long long)ntiles * blockIdx.x / gridDim.x);
  const int tcount = (int)((long long)ntiles * (blockIdx.x + 1) / gridDim.x) - tbeg;
  int tile_of[NT];
  bool live[NT];
  const int KT = K / 32;
  const int kbeg = (int)((long long)KT * blockIdx.y / KS), kend = (int)((long long)KT * (blockIdx.y + 1) / KS);
  const int nchunks = (kend - kbeg + KC - 1) / KC;
  const __bf16* wp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    live[t] = WAVES * t + wave < tcount;
    tile_of[t] = live[t] ? tbeg + WAVES * t + wave : (t > 0 && live[0] ? tile_of[0] : tbeg);
    wp[t] = wt + ((size_t)tile_of[t] * KT * 64 + lane) * 8;
  }
  // This thread's share of a chunk of x: XF fragments of 16 bytes.  A wavefront's load takes 8 rows
  // and, of each, 8 pieces (two k-steps: a whole 128-byte line; with one k-step a load touched 16
  // lines and used half of each, and x is a third to a half of what these kernels pull through L1);
  // lanes 0..7 take the 8 rows of one piece, so that they store to neighbouring places in LDS.
  constexpr int XF = MB * KC * 64 / THREADS;
  static_assert(XF * THREADS == MB * KC * 64 && KC % 2 == 0, "a chunk of x must divide evenly over the threads");
  const __bf16* xsrc[XF];
  int xks[XF], xmb[XF], xfl[XF];
#pragma unroll
  for (int j = 0; j < XF; ++j) {
    const int idx = threadIdx.x + THREADS * j;
    const int l = idx % 64, blk = idx / 64;
    const int r = 8 * (blk % (MB * 2)) + l % 8;           // row of the chunk
    const int p = 8 * (blk / (MB * 2)) + l / 8;           // piece of the row: k-step p / 4 of the chunk, channels 8 (p % 4)..
    xks[j] = p / 4;
    xmb[j] = r / 16;
    xfl[j] = 16 * (p % 4) + r % 16;                        // the lane whose B operand this is
    const int m = r < M ? r : M - 1;
    xsrc[j] = x + (size_t)m * K + 8 * (p % 4);
  }
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // Every load of the main loop is issued unconditionally (past the end: from
  // the last k-step, replaced by zeros when it is stored): a load under a
  // branch would make each later wait count it as possibly absent, which ends
  // in waiting for all loads at once.
  auto load_x = [&](int c, bf16x8 (&xr)[XF]) {
#pragma unroll
    for (int j = 0; j < XF; ++j) {
      const int ks = kbeg + c * KC + xks[j];
      xr[j] = *(const bf16x8*)(xsrc[j] + 32 * (size_t)(ks < kend ? ks : kend - 1));
    }
  };
  auto store_x = [&](int buf, int c, const bf16x8 (&xr)[XF]) {
#pragma unroll
    for (int j = 0; j < XF; ++j)
      xs[buf][xks[j]][xmb[j]][xfl[j]] = kbeg + c * KC + xks[j] < kend ? xr[j] : zero;
  };
  f32x4 acc[NT][MB];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[t][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  // The chunk loop, written once for a wavefront with all NT tiles and once for one with fewer
  // (the last workgroups of an uneven share): a wavefront takes the branch as a whole, so each
  // form is straight-line code whose loads the compiler can count, and a wavefront without a
  // second tile neither loads nor multiplies for it (its loads would take places in the CU's
  // queue of outstanding requests, which is what limits these kernels).
  auto run = [&](auto ntl_tag) {
    constexpr int NTL = decltype(ntl_tag)::value;
    auto load_w = [&](int c, bf16x8 (&a)[NT][KC]) {
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        int ks = kbeg + c * KC + u;
        if (ks >= kend) ks = kend - 1;               // its x is zero
#pragma unroll
        for (int t = 0; t < NTL; ++t) a[t][u] = stream_load(wp[t] + 512 * (size_t)ks);
      }
    };
    // The x operands of a k-step are read from LDS two k-steps before their
    // products; the scheduling barriers keep the compiler from moving the reads
    // back next to their use, where every pair of products would wait out the
    // full latency of LDS (this made the kernel's time grow with the rows of x).
    auto multiply = [&](int buf, const bf16x8 (&a)[NT][KC]) {
      bf16x8 bv[2][MB];
#pragma unroll
      for (int u = 0; u < 2 && u < KC; ++u)
#pragma unroll
        for (int b = 0; b < MB; ++b) bv[u][b] = xs[buf][u][b][lane];
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
          for (int t = 0; t < NTL; ++t)
            acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], bv[u & 1][b], acc[t][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (u + 2 < KC) {
#pragma unroll
          for (int b = 0; b < MB; ++b) bv[u & 1][b] = xs[buf][u + 2][b][lane];
        }
      }
    };
    // Sets of W registers, the chunk loop unrolled over them: the loads of the chunks ahead stay
    // in flight until their own products need them (a copy from one set into another would wait
    // for them at once).
    bf16x8 a0[NT][KC], a1[NT][KC], xr[XF];
    if constexpr (DEPTH == 3) {
      // W and x are asked for two chunks ahead (x into registers, stored to LDS one chunk ahead).
      // Loads return in order, so a wait for a chunk's x must not have a later chunk's W before
      // it: every step asks for x, then W, of the chunk two ahead, and waits only for what is older.
      bf16x8 a2[NT][KC], xr1[XF], xr2[XF];
      load_x(0, xr);
      load_w(0, a0);
      load_x(1, xr1);                              // (past the end: the last k-step again; stored as zeros)
      load_w(1, a1);
      store_x(0, 0, xr);
      int c = 0;
      for (; c + 3 < nchunks; c += 3) {
        __syncthreads();
        load_x(c + 2, xr2);
        load_w(c + 2, a2);
        multiply(0, a0);
        store_x(1, c + 1, xr1);
        __syncthreads();
        load_x(c + 3, xr);
        load_w(c + 3, a0);
        multiply(1, a1);
        store_x(2, c + 2, xr2);
        __syncthreads();
        load_x(c + 4, xr1);
        load_w(c + 4, a1);
        multiply(2, a2);
        store_x(0, c + 3, xr);
      }
      // the last one to three chunks: W of c in a0 and of c + 1 in a1, x of c in LDS and of c + 1 in xr1
      __syncthreads();
      if (c + 2 < nchunks) {
        load_x(c + 2, xr2);
        load_w(c + 2, a2);
      }
      multiply(0, a0);
      if (c + 1 < nchunks) {
        store_x(1, c + 1, xr1);
        __syncthreads();
        multiply(1, a1);
        if (c + 2 < nchunks) {
          store_x(2, c + 2, xr2);
          __syncthreads();
          multiply(2, a2);
        }
      }
    } else {
      load_x(0, xr);
      load_w(0, a0);
      store_x(0, 0, xr);
      int c = 0;
      for (; c + 2 < nchunks; c += 2) {
        __syncthreads();
        load_x(c + 1, xr);
        load_w(c + 1, a1);
        multiply(0, a0);
        store_x(1, c + 1, xr);
        __syncthreads();
        load_x(c + 2, xr);
        load_w(c + 2, a0);
        multiply(1, a1);
        store_x(0, c + 2, xr);
      }
      // the last one or two chunks
      __syncthreads();
      if (c + 1 < nchunks) {
        load_x(c + 1, xr);
        load_w(c + 1, a1);
      }
      multiply(0, a0);
      if (c + 1 < nchunks) {
        store_x(1, c + 1, xr);
        __syncthreads();
        multiply(1, a1);
      }
    }
  };
  // (live[t] comes from the wavefront's index and the workgroup's: a scalar, so this is a real branch)
  if (live[NT - 1]) run(std::integral_constant<int, NT>{});
  else run(std::integral_constant<int, (NT > 1 ? NT - 1 : 1)>{});
  // lane: column m = 16 b + i of x, rows n = 16 tile + 4 gq + r of W
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (!live[t]) continue;
    const int n = tile_of[t] * 16 + 4 * gq;
#pragma unroll
    for (int b = 0; b < MB; ++b) {
      const int m = 16 * b + i;
      if (gated) {
        // rows 0..7 of a tile are gates, 8..15 their ups: lanes gq < 2 fetch the ups from gq + 2
        f32x4 up;
#pragma unroll
        for (int r = 0; r < 4; ++r) up[r] = __shfl(acc[t][b][r], lane + 32, 64);
        if (gq < 2 && m < M) {
          __bf16* o = (__bf16*)y + (size_t)m * (N / 2) + tile_of[t] * 8 + 4 * gq;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float g = acc[t][b][r];
            o[r] = (__bf16)(g / (1.f + expf(-g)) * up[r]);
          }
        }
        continue;
      }
      if (m >= M) continue;
      // four consecutive columns per lane: one 16-byte (8-byte) store where the row allows it
      const bool whole = n + 3 < N && N % 4 == 0;
      if (KS > 1) {
        float* o = (float*)y + ((size_t)blockIdx.y * M + m) * N + n;
        if (whole) {
          *(f32x4*)o = acc[t][b];
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < N) o[r] = acc[t][b][r];
        }
        continue;
      }
      f32x4 v = acc[t][b];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (bias != nullptr && n + r < N) v[r] += bias[n + r];
      if (whole && out_f32) {
        *(f32x4*)((float*)y + (size_t)m * N + n) = v;
      } else if (whole) {
        bf16x4 h;
#pragma unroll
        for (int r = 0; r < 4; ++r) h[r] = (__bf16)v[r];
        *(bf16x4*)((__bf16*)y + (size_t)m * N + n) = h;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (n + r >= N) continue;
          if (out_f32) ((float*)y)[(size_t)m * N + n + r] = v[r];
          else ((__bf16*)y)[(size_t)m * N + n + r] = (__bf16)v[r];
        }
      }
    }
  }
}

__global__ void splitk_reduce_kernel(const float* __restrict__ part, const float* __restrict__ bias,
                                     void* __restrict__ y, int M, int N, int KS, int out_f32) {
  const size_t total = (size_t)M * N;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    float v = bias != nullptr ? bias[idx % N] : 0.f;
    for (int j = 0; j < KS; ++j) v += part[(size_t)j * total + idx];
    if (out_f32) ((float*)y)[idx] = v;
    else ((__bf16*)y)[idx] = (__bf16)v;
  }
}

// ks > 1: `part` holds ks * M * N floats; with y == nullptr they are left there
// for the reader to add (and the bias with them).
extern "C" const char* sl_gemm_mid(const void* x, const void* wt, const float* bias, void* y,
                                   int M, int N, int K, int out_f32, int gated, int ks,
                                   int wide_min_wgs, int num_cus, float* part, hipStream_t stream) {
  SL_CHECK(M > 0 && N > 0 && K > 0, "gemm_mid: sizes must be positive");
  SL_CHECK(M <= 128, "gemm_mid: at most 128 rows");
  SL_CHECK(K % 32 == 0, "gemm_mid: K must be a multiple of 32");
  SL_CHECK(ks >= 1 && ks <= 16 && ks <= K / 32, "gemm_mid: ks must be in 1..16 and <= K / 32");
  SL_CHECK(ks == 1 || part != nullptr, "gemm_mid: a split of K needs the partial buffer");
  SL_CHECK(y != nullptr || ks > 1, "gemm_mid: no output");
  SL_CHECK(!gated || (ks == 1 && N % 16 == 0 && bias == nullptr && !out_f32),
           "gemm_mid: the gated form needs ks == 1, N % 16 == 0, no bias, activation output");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)wt % 16) == 0,
           "gemm_mid: x and W must be 16-byte aligned");
  const int ntiles = (N + 15) / 16;
  const __bf16* xx = (const __bf16*)x;
  const __bf16* ww = (const __bf16*)wt;
  void* dst = ks > 1 ? (void*)part : y;
  // chunks of four k-steps, two tiles per wavefront; 8 wavefronts (16 tiles
  // share one pass over x) when that still leaves wide_min_wgs workgroups.
  // An unsplit product that would keep more than half the CUs busy that way is
  // spread over a whole multiple of the CUs instead, fewer tiles each: the time
  // of these products is what the busiest CU has to pull through its L1.
  const int wide_min = ks > 1 && 4 * num_cus / 5 > wide_min_wgs ? 4 * num_cus / 5 : wide_min_wgs;   // a split must keep most CUs busy
  const bool wide = ((ntiles + 15) / 16) * ks >= wide_min;
  int groups = wide ? (ntiles + 15) / 16 : (ntiles + 7) / 8;
  if (ks == 1 && wide && num_cus > 0 && 2 * groups > num_cus)
    groups = num_cus * ((groups + num_cus - 1) / num_cus);
  // a split product whose workgroups would leave CUs idle is spread over all of them, fewer tiles each
  // (7B shape at 64 rows, K in 4 / 8 shares: q/k/v 144 -> 256 workgroups 11.0 -> 10.1 us, o 224 -> 256: 8.8 -> 8.5)
  if (ks > 1 && num_cus > 0 && groups * ks < num_cus && num_cus % ks == 0 && num_cus / ks <= ntiles)
    groups = num_cus / ks;
  const dim3 grid(groups, ks);
  // blocks of 16 rows of x a wavefront multiplies each tile of W with: as many as the rows need (80
  // rows in five, not in eight: the products of 65 and more rows are no longer bound by memory
  // alone); the workgroups of eight wavefronts share out a chunk of x evenly for even counts only
  const int mb = (M + 15) / 16;
#define SL_MID(MB_, WAVES_) gemm_mid_kernel<MB_, 2, 4, WAVES_><<<grid, 64 * WAVES_, 0, stream>>>( \
    xx, ww, bias, dst, M, N, K, out_f32, gated, ks)
  if (wide) {
    if (mb <= 2) SL_MID(2, 8);
    else if (mb <= 4) SL_MID(4, 8);
    else if (mb <= 6) SL_MID(6, 8);
    else SL_MID(8, 8);
  } else {
    switch (mb) {
      case 1: case 2: SL_MID(2, 4); break;
      case 3: SL_MID(3, 4); break;
      case 4: SL_MID(4, 4); break;
      case 5: SL_MID(5, 4); break;
      case 6: SL_MID(6, 4); break;
      case 7: SL_MID(7, 4); break;
      default: SL_MID(8, 4); break;
    }
  }
#undef SL_MID
  const char* e = sl_launch_status();
  if (e || ks == 1 || y == nullptr) return e;
  const size_t total = (size_t)M * N;
  splitk_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(part, bias, y, M, N, ks, out_f32);
  return sl_launch_status();
}

// y = sum of the ks partial sums [ks, M, N] (+ bias)
extern "C" const char* sl_splitk_reduce(const float* part, const float* bias, void* y, int M, int N,
                                        int ks, int out_f32, hipStream_t stream) {
  SL_CHECK(M > 0 && N > 0 && ks >= 1, "splitk_reduce: sizes must be positive");
  const size_t total = (size_t)M * N;
  splitk_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(part, bias, y, M, N, ks, out_f32);
  return sl_launch_status();
}

// Row-major W [N, K] -> tiled [ceil(N / th)][K / 32][4][th][8] (th = 16: [..][64][8], the matrix
// instruction's A operand as it sits in registers); rows beyond N are zero.
__global__ void tile_weight_kernel(const __bf16* __restrict__ w, __bf16* __restrict__ wt, int N,
                                   int K, int th, size_t total_vec) {
  const int KT = K / 32;
  for (size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec;
       v += (size_t)gridDim.x * blockDim.x) {
    const int at = (int)(v % (4 * th));                  // place inside the tile's k-step: quarter of k, row
    const size_t t = v / (4 * th);
    const int ks = (int)(t % KT);
    const size_t tile = t / KT;
    const size_t n = tile * th + at % th;
    const int k = ks * 32 + 8 * (at / th);
    bf16x8 val = {0, 0, 0, 0, 0, 0, 0, 0};
    if (n < (size_t)N) val = *(const bf16x8*)(w + n * K + k);
    *(bf16x8*)(wt + v * 8) = val;
  }
}

// wt: ceil(N / th) * th * K elements.
extern "C" const char* sl_tile_weight(const void* w, void* wt, int N, int K, int th, hipStream_t stream) {
  SL_CHECK(N > 0 && K > 0 && K % 32 == 0, "tile_weight: K must be a positive multiple of 32");
  SL_CHECK(th >= 8 && th <= 16 && th % 2 == 0, "tile_weight: tiles of 8, 10, 12, 14 or 16 rows");
  SL_CHECK(((uintptr_t)w % 16) == 0 && ((uintptr_t)wt % 16) == 0, "tile_weight: 16-byte alignment");
  const size_t total_vec = (size_t)((N + th - 1) / th) * (K / 32) * 4 * th;
  const size_t blocks = (total_vec + 255) / 256;
  tile_weight_kernel<<<(unsigned)(blocks < 262144 ? blocks : 262144), 256, 0, stream>>>(
      (const __bf16*)w, (__bf16*)wt, N, K, th, total_vec);
  return sl_launch_status();
}
// Tiled -> row-major [N, K] (the inverse), for products with many rows when only
// the tiled copy is kept.
__global__ void untile_weight_kernel(const __bf16* __restrict__ wt, __bf16* __restrict__ w, int N,
                                     int K, int th, size_t total_vec) {
  const int KT = K / 32;
  for (size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec;
       v += (size_t)gridDim.x * blockDim.x) {
    // v enumerates the row-major matrix in 16-byte vectors, so the stores are contiguous
    const size_t n = v / (K / 8);
    const int k8 = (int)(v % (K / 8));
    const int ks = k8 / 4, gq = k8 % 4;
    const size_t src = (((n / th) * KT + ks) * (4 * th) + gq * th + (n % th)) * 8;
    *(bf16x8*)(w + v * 8) = *(const bf16x8*)(wt + src);
  }
}

extern "C" const char* sl_untile_weight(const void* wt, void* w, int N, int K, int th, hipStream_t stream) {
  SL_CHECK(N > 0 && K > 0 && K % 32 == 0, "untile_weight: K must be a positive multiple of 32");
  SL_CHECK(th >= 8 && th <= 16 && th % 2 == 0, "untile_weight: tiles of 8, 10, 12, 14 or 16 rows");
  SL_CHECK(((uintptr_t)w % 16) == 0 && ((uintptr_t)wt % 16) == 0, "untile_weight: 16-byte alignment");
  const size_t total_vec = (size_t)N * (K / 8);
  const size_t blocks = (total_vec + 255) / 256;
  untile_weight_kernel<<<(unsigned)(blocks < 262144 ? blocks : 262144), 256, 0, stream>>>(
      (const __bf16*)wt, (__bf16*)w, N, K, th, total_vec);
  return sl_launch_status();
}

// ------------------------------------------------- 129 rows and more, matrix cores
// y[M, N] = x[M, K] W[N, K]^T for steps of a few hundred rows (a newcomer's prompt beside decoded
// tokens) and matrices of few rows (q/k/v, o, down), where the product is neither bound by
// streaming W (the kernels above) nor large enough for the tiles of a library kernel to fill the
// chip.  Both operands are row-major; a workgroup of WM x WN wavefronts owns a tile of 64 WM rows
// of x by 64 WN rows of W over a share of K (grid.z shares write float partial sums [KS, M, N]
// that the reader or splitk_reduce adds), a wavefront 64 x 64 of it (16 matrix instructions per
// 8 operand reads).
//
// Chunks of 64 values of k travel from global memory straight into a ring of three LDS stages
// (global_load_lds_dwordx4: a wavefront's 64 loads of 16 bytes land side by side in 1 KB), two
// chunks in flight while the third is multiplied: at the 50 GB/s a CU pulls and 2 us of loaded
// latency that is what keeps the stream going.  A stage holds the rows of x, then those of W, 8
// units of 16 bytes a row; a lane can put any unit anywhere at no cost, so unit c of row r lies
// at place c ^ f(r), f(r) = ((r >> 1) & 7) ^ 4 (r & 1): the 16 lanes that read one operand
// column (rows r .. r + 15, same c) then touch 16 different 16-byte slots of a 256-byte line of
// banks, and each half of them 8 different slots of a 128-byte one.
__device__ __forceinline__ void block_load_to_lds(const void* from, unsigned lds_at) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(lds_at) : "m0");
}
template <int N_> __device__ __forceinline__ void block_wait_loads() {
  __builtin_amdgcn_s_waitcnt((N_ & 15) | (7 << 4) | (15 << 8) | ((N_ >> 4) << 14));
}

template <int WM, int WN, int STAGES>
__global__ __launch_bounds__(64 * WM * WN) void gemm_block_kernel(
    const __bf16* __restrict__ x, const __bf16* __restrict__ w, const float* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int out_f32, int KS) {
  constexpr int WAVES = WM * WN, BM = 64 * WM, BN = 64 * WN;
  static_assert(STAGES == 2 || STAGES == 3, "a ring of two or three stages");
  constexpr int ROWS = BM + BN;                      // rows of a stage: x, then W; 128 bytes each
  constexpr int STAGE_BYTES = ROWS * 128;
  constexpr int LOADS = ROWS / 8 / WAVES;            // wavefront-wide loads (8 rows) a wavefront makes per chunk
  static_assert(LOADS * 8 * WAVES == ROWS, "the rows of a stage must divide evenly over the wavefronts");
  __shared__ __attribute__((aligned(1024))) char ring[STAGES * STAGE_BYTES];
  const int t = threadIdx.x, lane = t & 63, i = lane & 15, gq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave / WN, wn = wave % WN;
  // Workgroups go to the eight chiplets in turn, each with an L2 of its own, and the workgroups of
  // one share of K read the same columns of x: the grid is one-dimensional and chiplet c takes a
  // contiguous eighth of the (share, column tile, row tile) triples, so that a share's slice of x
  // lies in one or two L2s instead of eight and the rows of W that two row tiles share come from
  // memory once.
  const int gx = (N + BN - 1) / BN, gy = (M + BM - 1) / BM, total = gx * gy * KS;
  const int per = (total + 7) / 8;
  const int triple = (int)(blockIdx.x & 7) * per + (int)(blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per || triple >= total) return;       // (the whole workgroup)
  // (row tiles fastest: the workgroups that read the same rows of W run side by side on one chiplet)
  const int share = triple / (gx * gy);
  const int m0 = triple % gy * BM, n0 = triple / gy % gx * BN;
  const int chunks = K / 64;
  const int cbeg = (int)((long long)chunks * share / KS);
  const int cend = (int)((long long)chunks * (share + 1) / KS);

  // what this lane fetches of every chunk: unit `cu ^ f(row)` of row 8 q + lane / 8 of the stage
  const __bf16* src[LOADS];
#pragma unroll
  for (int j = 0; j < LOADS; ++j) {
    const int row = 8 * (wave + WAVES * j) + (lane >> 3);
    const int c = (lane & 7) ^ (((row >> 1) & 7) ^ (4 * (row & 1)));
    if (row < BM) {
      const int m = m0 + row < M ? m0 + row : M - 1;           // rows past the end: the last row again, never stored
      src[j] = x + (size_t)m * K + 8 * c;
    } else {
      const int n = n0 + row - BM < N ? n0 + row - BM : N - 1;
      src[j] = w + (size_t)n * K + 8 * c;
    }
  }
  const unsigned ring_at = (unsigned)(size_t)(__attribute__((address_space(3))) char*)ring;
  auto fetch = [&](int c, int stage) {
    const unsigned at = ring_at + STAGE_BYTES * stage + 1024 * wave;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) block_load_to_lds(src[j] + 64 * (size_t)c, at + 1024 * WAVES * j);
  };
  // where this lane reads its operands: row R0 + i (R0 a multiple of 16), unit 4 kk + gq
  int at_kk[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) at_kk[kk] = 128 * i + 16 * ((4 * kk + gq) ^ (((i >> 1) & 7) ^ (4 * (i & 1))));

  f32x4 acc[4][4];                                   // [tile of W rows][tile of x rows]
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (cbeg < cend) {
    fetch(cbeg, 0);
    if (STAGES == 3 && cbeg + 1 < cend) {
      fetch(cbeg + 1, 1);
      block_wait_loads<LOADS>();
    } else {
      block_wait_loads<0>();
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" : : : "memory");
  }
  int stage = 0;
  for (int c = cbeg; c < cend; ++c) {
    const bool more = c + STAGES - 1 < cend;
    if (more) fetch(c + STAGES - 1, stage >= 1 ? stage - 1 : STAGES - 1);        // the stage the last chunk was read from
    const char* st = ring + STAGE_BYTES * stage;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      bf16x8 a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        a[u] = *(const bf16x8*)(st + 128 * (BM + 64 * wn + 16 * u) + at_kk[kk]);
        b[u] = *(const bf16x8*)(st + 128 * (64 * wm + 16 * u) + at_kk[kk]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          acc[u][v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[v], acc[u][v], 0, 0, 0);
    }
    if (more && STAGES == 3) block_wait_loads<LOADS>();        // all but the chunk just asked for
    else block_wait_loads<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" : : : "memory");
    stage = stage == STAGES - 1 ? 0 : stage + 1;
  }

  // lane: row m of x (16 v + i), four consecutive rows n of W (16 u + 4 gq ..)
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int m = m0 + 64 * wm + 16 * v + i;
    if (m >= M) continue;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int n = n0 + 64 * wn + 16 * u + 4 * gq;
      if (n >= N) continue;
      const bool whole = n + 3 < N && N % 4 == 0;
      f32x4 r = acc[u][v];
      if (KS > 1) {
        float* o = (float*)y + ((size_t)share * M + m) * N + n;
        if (whole) {
          *(f32x4*)o = r;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) o[e] = r[e];
        }
        continue;
      }
      if (bias != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) r[e] += bias[n + e];
      }
      if (whole && out_f32) {
        *(f32x4*)((float*)y + (size_t)m * N + n) = r;
      } else if (whole) {
        bf16x4 h;
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = (__bf16)r[e];
        *(bf16x4*)((__bf16*)y + (size_t)m * N + n) = h;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (n + e >= N) continue;
          if (out_f32) ((float*)y)[(size_t)m * N + n + e] = r[e];
          else ((__bf16*)y)[(size_t)m * N + n + e] = (__bf16)r[e];
        }
      }
    }
  }
}

// x and W row-major.  ks > 1: `part` holds ks * M * N floats; with y == nullptr they are left
// there for the reader to add (and the bias with them), else splitk_reduce adds them into y.
extern "C" const char* sl_gemm_block(const void* x, const void* w, const float* bias, void* y,
                                     int M, int N, int K, int out_f32, int ks, int square, float* part,
                                     hipStream_t stream) {
  SL_CHECK(M > 0 && N > 0 && K > 0, "gemm_block: sizes must be positive");
  SL_CHECK(K % 64 == 0, "gemm_block: K must be a multiple of 64");
  SL_CHECK(ks >= 1 && ks <= 64 && ks <= K / 64, "gemm_block: ks must be in 1..64 and <= K / 64");
  SL_CHECK(ks == 1 || part != nullptr, "gemm_block: a split of K needs the partial buffer");
  SL_CHECK(y != nullptr || ks > 1, "gemm_block: no output");
  SL_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_block: x and W must be 16-byte aligned");
  void* dst = ks > 1 ? (void*)part : y;
  const __bf16* xx = (const __bf16*)x;
  const __bf16* ww = (const __bf16*)w;
  // (Tiles of 64 x 256 and 128 x 256 for fewer rows of x were built and measured: alone they beat the
  // LDS-staged kernel above, in a decode step of 24 to 128 requests they lost 2-5 % tokens/s to it,
  // so that kernel keeps those rows and this one starts where it ends.)
  // square: tiles of 256 x 256 (sixteen wavefronts, a ring of two stages in 128 KB of LDS) instead of
  // 256 x 128 (eight wavefronts, three stages): a workgroup pulls 512 rows for 256 x 256 of result
  // instead of 384 for 256 x 128, which is what the time of these products follows.
  const int bn = square ? 256 : 128;
  const long long triples = (long long)((N + bn - 1) / bn) * ((M + 255) / 256) * ks;
  SL_CHECK(triples < (1ll << 28), "gemm_block: too many tiles");
  const dim3 grid((unsigned)(8 * ((triples + 7) / 8)));              // laid out by chiplet (see the kernel)
  if (square) gemm_block_kernel<4, 4, 2><<<grid, 1024, 0, stream>>>(xx, ww, bias, dst, M, N, K, out_f32, ks);
  else gemm_block_kernel<4, 2, 3><<<grid, 512, 0, stream>>>(xx, ww, bias, dst, M, N, K, out_f32, ks);
  const char* e = sl_launch_status();
  if (e || ks == 1 || y == nullptr) return e;
  const size_t total = (size_t)M * N;
  splitk_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(part, bias, y, M, N, ks, out_f32);
  return sl_launch_status();
}
#endif
