// RMSNorm fused with the residual add that precedes it.
//   resid (float, in place) += delta;  out = resid * rsqrt(mean(resid^2) + eps) * w
// Formula and float32 math: servelab/attention/triton/paged_attention.py:76-91,
// tests/test_triton_kernels.py:57-59; the adds it absorbs are
// servelab/parallel/tp_model.py:131,133.  One block per row.
#include "common.h"

// rows == nullptr: row r of the stream, which is updated in place.
// rows != nullptr: row rows[r] of the stream (and of delta) is read, nothing
// but out[r] is written.
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const act_t* __restrict__ delta,
                                   const int* __restrict__ rows, const float* __restrict__ w,
                                   act_t* __restrict__ out, int H, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* d = delta != nullptr ? delta + src * H : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (d != nullptr) {
      v += to_f(d[i]);
      if (rows == nullptr) x[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)H + eps);
  act_t* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (d != nullptr && rows != nullptr) v += to_f(d[i]);
    o[i] = from_f<act_t>(v * inv * w[i]);
  }
}

// The same for rows of up to 4 * 8 * blockDim values that are a multiple of 4
// wide: every value is read once with 16-byte loads and kept in registers
// between the sum of squares and the scaling.
struct __attribute__((aligned(16))) f4 { float v[4]; };
#if defined(SL_F32)
struct __attribute__((aligned(16))) a4 { act_t v[4]; };
#else
struct __attribute__((aligned(8))) a4 { act_t v[4]; };
#endif

template <int ITERS>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ resid, const act_t* __restrict__ delta,
                                       const int* __restrict__ rows, const float* __restrict__ w,
                                       act_t* __restrict__ out, int H, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* d = delta != nullptr ? delta + src * H : nullptr;
  const int H4 = H / 4;
  f4 v[ITERS];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = threadIdx.x + it * blockDim.x;
    if (i < H4) {
      v[it] = ((const f4*)x)[i];
      if (d != nullptr) {
        const a4 dv = ((const a4*)d)[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[it].v[j] += to_f(dv.v[j]);
        if (rows == nullptr) ((f4*)x)[i] = v[it];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) ss += v[it].v[j] * v[it].v[j];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)H + eps);
  act_t* o = out + (size_t)r * H;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = threadIdx.x + it * blockDim.x;
    if (i < H4) {
      const f4 wv = ((const f4*)w)[i];
      a4 ov;
#pragma unroll
      for (int j = 0; j < 4; ++j) ov.v[j] = from_f<act_t>(v[it].v[j] * inv * wv.v[j]);
      ((a4*)o)[i] = ov;
    }
  }
}

extern "C" const char* sl_add_rmsnorm(float* resid, const void* delta, const int* rows,
                                      const float* w, void* out, int R, int H, float eps,
                                      hipStream_t stream) {
  SL_CHECK(R >= 0 && H > 0, "add_rmsnorm: sizes must be positive");
  if (R == 0) return nullptr;
  if (H % 4 == 0 && H <= 4 * 8 * 512) {
    const int H4 = H / 4;
    const int threads = H4 <= 64 ? 64 : (H4 <= 128 ? 128 : (H4 <= 256 ? 256 : 512));
    const int iters = (H4 + threads - 1) / threads;
    const act_t* dl = (const act_t*)delta;
    act_t* o = (act_t*)out;
    if (iters == 1) add_rmsnorm_vec_kernel<1><<<R, threads, 0, stream>>>(resid, dl, rows, w, o, H, eps);
    else if (iters == 2) add_rmsnorm_vec_kernel<2><<<R, threads, 0, stream>>>(resid, dl, rows, w, o, H, eps);
    else if (iters <= 4) add_rmsnorm_vec_kernel<4><<<R, threads, 0, stream>>>(resid, dl, rows, w, o, H, eps);
    else add_rmsnorm_vec_kernel<8><<<R, threads, 0, stream>>>(resid, dl, rows, w, o, H, eps);
    return sl_launch_status();
  }
  const int threads = H >= 2048 ? 512 : 256;
  add_rmsnorm_kernel<<<R, threads, 0, stream>>>(resid, (const act_t*)delta, rows, w,
                                                (act_t*)out, H, eps);
  return sl_launch_status();
}
