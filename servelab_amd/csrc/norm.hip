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

extern "C" const char* sl_add_rmsnorm(float* resid, const void* delta, const int* rows,
                                      const float* w, void* out, int R, int H, float eps,
                                      hipStream_t stream) {
  SL_CHECK(R >= 0 && H > 0, "add_rmsnorm: sizes must be positive");
  if (R == 0) return nullptr;
  const int threads = H >= 2048 ? 512 : 256;
  add_rmsnorm_kernel<<<R, threads, 0, stream>>>(resid, (const act_t*)delta, rows, w,
                                                (act_t*)out, H, eps);
  return sl_launch_status();
}
