// Shared definitions of the servelab_amd kernels (gfx950, 64-wide wavefronts).
//
// Every source is compiled twice: with -DSL_F32 the activation type is float
// (the true 32-bit path: no reduced-precision matrix instruction anywhere),
// without it the activation type is bfloat16.  Accumulation, softmax, norms
// and rotation are float in both.
//
// Every extern "C" entry point returns nullptr on success or a static message
// that says which size it refuses; nothing here allocates device memory.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#if defined(SL_F32)
typedef float act_t;
#define SL_ACT_NAME "float32"
#else
typedef __bf16 act_t;
#define SL_ACT_NAME "bfloat16"
#endif

#define SL_WAVE 64

__device__ __forceinline__ float to_f(float x) { return x; }
__device__ __forceinline__ float to_f(__bf16 x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f(float x);
template <> __device__ __forceinline__ float from_f<float>(float x) { return x; }
template <> __device__ __forceinline__ __bf16 from_f<__bf16>(float x) { return (__bf16)x; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = SL_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, SL_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = SL_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, SL_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / SL_WAVE, lane = threadIdx.x % SL_WAVE;
  const int nwaves = (blockDim.x + SL_WAVE - 1) / SL_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

#define SL_CHECK(cond, msg) \
  do { if (!(cond)) return msg; } while (0)

static inline const char* sl_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? nullptr : hipGetErrorString(e);
}
