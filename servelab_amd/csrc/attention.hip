// Attention over the paged cache: general kernel.
//
// For every query token t of the batch (sequence s = tok_seq[t], position
// p = positions[t]) and every query head h: keys r in [lo, p] of sequence s,
// lo = max(0, p - window + 1) with a window, else 0, found through the
// sequence's block table; score = (q . k_r) * scale; softmax over r; output
// sum_r P_r v_r; all in float with a running maximum and sum.  kv head of h is
// h / (nh / nkv).
//
// Reference: the per-sequence loop of servelab/parallel/tp_model.py:136-157
// (scores, causal mask, softmax, PV in float32) and the running-softmax form of
// servelab/attention/triton/paged_attention.py:39-74.  A prompt portion sees
// itself through the cache (its keys are written before this runs), so a
// decode token is just a portion of one token.  The window is this build's own.
//
// One wavefront per (token, head, share of the keys); lanes split 64 keys for
// the scores and the head's channels for the output.  With more than one share
// (few tokens, long contexts: a decode step) every wavefront leaves its
// unnormalised output, maximum and sum, and attention_general_combine_kernel
// merges them.  Any head size up to 256, any head counts,
// page sizes 16 / 32 / 64.  This is the kernel of the float32 path and the
// fallback of the bfloat16 path for sizes its matrix-core kernels refuse.
#include "common.h"

#define MAX_D 256

__global__ __launch_bounds__(64) void attention_general_kernel(
    const act_t* __restrict__ qkv, int row_stride, const act_t* __restrict__ kc,
    const act_t* __restrict__ vc, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, int nh, int nkv, int D,
    int page, float scale, int window, act_t* __restrict__ out, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
  __shared__ float qs[MAX_D];
  __shared__ float ps[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = tok_seq[t], p = positions[t];
  const int kvh = h / (nh / nkv);
  const int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int* table = block_tables + (size_t)s * max_pages;
  const act_t* q = qkv + (size_t)t * row_stride + (size_t)h * D;
  for (int d = lane; d < D; d += 64) qs[d] = to_f(q[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[MAX_D / 64];
#pragma unroll
  for (int i = 0; i < MAX_D / 64; ++i) acc[i] = 0.f;

  // blocks of 64 keys [first, p / 64]; this wavefront takes share blockIdx.z of them
  const int first = lo / 64, nblk = p / 64 + 1 - first;
  const int b0 = first + (int)((long long)nblk * blockIdx.z / nsplit);
  const int b1 = first + (int)((long long)nblk * (blockIdx.z + 1) / nsplit);
  for (int kb = b0 * 64; kb < b1 * 64; kb += 64) {
    const int r = kb + lane;
    const bool valid = r >= lo && r <= p;
    float sc = -INFINITY;
    if (valid) {
      const int pg = table[r / page];
      const act_t* kr = kc + (((size_t)pg * nkv + kvh) * page + r % page) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * to_f(kr[d]);
      sc = dot * scale;
    }
    const float mn = fmaxf(m, wave_max(sc));       // every block holds a visible key
    const float alpha = expf(m - mn);              // exp(-inf) = 0 on the first block
    const float pr = valid ? expf(sc - mn) : 0.f;
    l = l * alpha + wave_sum(pr);
    m = mn;
    ps[lane] = pr;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MAX_D / 64; ++i) acc[i] *= alpha;
    for (int pb = 0; pb < 64; pb += page) {
      const int r0 = kb + pb;
      if (r0 > p) break;
      if (r0 + page <= lo) continue;               // wholly before the window: may be released
      const int pg = table[r0 / page];
      const act_t* vbase = vc + ((size_t)pg * nkv + kvh) * D * page;
#pragma unroll
      for (int i = 0; i < MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) {
          const act_t* vr = vbase + (size_t)d * page;
          float a = acc[i];
          for (int j = 0; j < page; ++j) a += ps[pb + j] * to_f(vr[j]);
          acc[i] = a;
        }
      }
    }
    __syncthreads();
  }
  if (nsplit > 1) {
    const size_t pr = ((size_t)t * nh + h) * nsplit + blockIdx.z;
#pragma unroll
    for (int i = 0; i < MAX_D / 64; ++i) {
      const int d = lane + 64 * i;
      if (d < D) part_o[pr * D + d] = acc[i];
    }
    if (lane == 0) {
      part_ml[pr * 2] = m;
      part_ml[pr * 2 + 1] = l;
    }
    return;
  }
  const float inv = 1.f / l;
  act_t* o = out + ((size_t)t * nh + h) * D;
#pragma unroll
  for (int i = 0; i < MAX_D / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < D) o[d] = from_f<act_t>(acc[i] * inv);
  }
}

// out[t, h, :] = sum_j w_j o_j / sum_j w_j l_j,  w_j = exp(m_j - max m); a share
// without keys has m = -inf and l = 0 and drops out.  One wavefront per (t, h).
__global__ __launch_bounds__(64) void attention_general_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int nsplit, int nh, int D,
    act_t* __restrict__ out) {
  __shared__ float ws[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t base = ((size_t)t * nh + h) * nsplit;
  float m = -INFINITY, l = 0.f;
  if (lane < nsplit) {
    m = part_ml[(base + lane) * 2];
    l = part_ml[(base + lane) * 2 + 1];
  }
  const float mx = wave_max(m);
  const float w = m == -INFINITY ? 0.f : expf(m - mx);
  const float denom = wave_sum(w * l);
  ws[lane] = w;
  __syncthreads();
  act_t* o = out + ((size_t)t * nh + h) * D;
  for (int d = lane; d < D; d += 64) {
    float a = 0.f;
    for (int j = 0; j < nsplit; ++j) a += ws[j] * part_o[(base + j) * D + d];
    o[d] = from_f<act_t>(a / denom);
  }
}

// nsplit > 1: part_o holds T * nh * nsplit * D floats, part_ml T * nh * nsplit * 2.
extern "C" const char* sl_attention_general(
    const void* qkv, int row_stride, const void* kc, const void* vc, const int* block_tables,
    int max_pages, const int* tok_seq, const int* positions, int T, int nh, int nkv, int D,
    int page, float scale, int window, void* out, int nsplit, float* part_o, float* part_ml,
    hipStream_t stream) {
  SL_CHECK(T >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0,
           "attention: heads must be a positive multiple of kv heads");
  SL_CHECK(D > 0 && D <= MAX_D, "attention: head_dim must be in 1..256");
  SL_CHECK(page == 16 || page == 32 || page == 64, "attention: page size must be 16, 32 or 64");
  SL_CHECK(nh <= 65535, "attention: more than 65535 heads");
  SL_CHECK(window >= 0, "attention: window must be >= 0 (0 = none)");
  SL_CHECK(nsplit >= 1 && nsplit <= 64, "attention: 1..64 shares of the keys");
  SL_CHECK(nsplit == 1 || (part_o != nullptr && part_ml != nullptr),
           "attention: shares of the keys need the partial buffers");
  if (T == 0) return nullptr;
  attention_general_kernel<<<dim3(T, nh, nsplit), 64, 0, stream>>>(
      (const act_t*)qkv, row_stride, (const act_t*)kc, (const act_t*)vc, block_tables, max_pages,
      tok_seq, positions, nh, nkv, D, page, scale, window, (act_t*)out, nsplit, part_o, part_ml);
  const char* e = sl_launch_status();
  if (e || nsplit == 1) return e;
  attention_general_combine_kernel<<<dim3(T, nh), 64, 0, stream>>>(part_o, part_ml, nsplit, nh, D,
                                                                 (act_t*)out);
  return sl_launch_status();
}
