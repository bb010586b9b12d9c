// RMSNorm fused with the residual add that precedes it.
//   resid (float, in place) += delta;  out = resid * rsqrt(mean(resid^2) + eps) * w
// delta is a tensor in the activation dtype, or the float partial sums of a
// product whose K was split over workgroups (parts [nparts][T][H], optionally a
// bias [H]): the partial sums are then added here instead of by a kernel of
// their own.
// Formula and float32 math: servelab/attention/triton/paged_attention.py:76-91,
// tests/test_triton_kernels.py:57-59; the adds it absorbs are
// servelab/parallel/tp_model.py:131,133.  One block per row.
#include "common.h"

// rows == nullptr: row r of the stream, which is updated in place.
// rows != nullptr: row rows[r] of the stream (and of delta) is read, nothing
// but out[r] is written.
struct SplitDelta {
  const float* parts;            // [nparts][stride], or nullptr
  int nparts;
  size_t stride;                 // T * H
  const float* bias;             // [H] or nullptr
};

__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const act_t* __restrict__ delta,
                                   const SplitDelta sd, const int* __restrict__ rows,
                                   const float* __restrict__ w, act_t* __restrict__ out, int H,
                                   float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* d = delta != nullptr ? delta + src * H : nullptr;
  const float* p = sd.parts != nullptr ? sd.parts + src * H : nullptr;
  const bool adds = d != nullptr || p != nullptr;
  auto delta_at = [&](int i) {
    float v = d != nullptr ? to_f(d[i]) : 0.f;
    if (p != nullptr) {
      for (int j = 0; j < sd.nparts; ++j) v += p[j * sd.stride + i];
      if (sd.bias != nullptr) v += sd.bias[i];
    }
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (adds) {
      v += delta_at(i);
      if (rows == nullptr) x[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)H + eps);
  act_t* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = x[i];
    if (adds && rows != nullptr) v += delta_at(i);
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
                                       const SplitDelta sd, const int* __restrict__ rows,
                                       const float* __restrict__ w, act_t* __restrict__ out, int H,
                                       float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * H;
  const act_t* d = delta != nullptr ? delta + src * H : nullptr;
  const float* p = sd.parts != nullptr ? sd.parts + src * H : nullptr;
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
      }
      if (p != nullptr) {
#pragma unroll 4
        for (int q = 0; q < sd.nparts; ++q) {
          const f4 pv = ((const f4*)(p + q * sd.stride))[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[it].v[j] += pv.v[j];
        }
        if (sd.bias != nullptr) {
          const f4 bv = ((const f4*)sd.bias)[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[it].v[j] += bv.v[j];
        }
      }
      if ((d != nullptr || p != nullptr) && rows == nullptr) ((f4*)x)[i] = v[it];
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

// parts != nullptr: nparts float partial sums [nparts][T][H] (T rows in each)
// and an optional bias [H] are the delta (or are added to it).
extern "C" const char* sl_add_rmsnorm(float* resid, const void* delta, const float* parts,
                                      int nparts, int T, const float* bias, const int* rows,
                                      const float* w, void* out, int R, int H, float eps,
                                      hipStream_t stream) {
  SL_CHECK(R >= 0 && H > 0, "add_rmsnorm: sizes must be positive");
  SL_CHECK(parts == nullptr || (nparts >= 1 && T >= 1), "add_rmsnorm: partial sums need their counts");
  SL_CHECK(parts != nullptr || bias == nullptr, "add_rmsnorm: a bias comes with partial sums only");
  if (R == 0) return nullptr;
  const SplitDelta sd{parts, nparts, (size_t)T * H, bias};
  const bool aligned = ((uintptr_t)resid % 16) == 0 && ((uintptr_t)out % sizeof(a4)) == 0 &&
                       ((uintptr_t)delta % sizeof(a4)) == 0 && ((uintptr_t)parts % 16) == 0 &&
                       ((uintptr_t)bias % 16) == 0 && ((uintptr_t)w % 16) == 0;
  if (H % 4 == 0 && H <= 4 * 8 * 512 && aligned) {
    const int H4 = H / 4;
    const int threads = H4 <= 64 ? 64 : (H4 <= 128 ? 128 : (H4 <= 256 ? 256 : 512));
    const int iters = (H4 + threads - 1) / threads;
    const act_t* dl = (const act_t*)delta;
    act_t* o = (act_t*)out;
    if (iters == 1) add_rmsnorm_vec_kernel<1><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    else if (iters == 2) add_rmsnorm_vec_kernel<2><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    else if (iters <= 4) add_rmsnorm_vec_kernel<4><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    else add_rmsnorm_vec_kernel<8><<<R, threads, 0, stream>>>(resid, dl, sd, rows, w, o, H, eps);
    return sl_launch_status();
  }
  const int threads = H >= 2048 ? 512 : 256;
  add_rmsnorm_kernel<<<R, threads, 0, stream>>>(resid, (const act_t*)delta, sd, rows, w,
                                                (act_t*)out, H, eps);
  return sl_launch_status();
}
