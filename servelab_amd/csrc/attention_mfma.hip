// Attention over the paged cache on the matrix cores (bfloat16 only), for
// prompt portions and for decode tokens.  Head size SL_HEAD_DIM is a compile
// time constant (a multiple of 32, at most 256); the library is built for the
// head size of the model at hand.
//
// Same contract as the general kernel (attention.hip): query token t of
// sequence s at position p sees keys lo..p of s through the block table;
// scores * scale, softmax and the weighted sum of values in float.  Reference:
// servelab/parallel/tp_model.py:136-157 and the running-softmax kernel
// servelab/attention/triton/paged_attention.py:39-74, which handles one query
// head per program, re-reads K and V once per head of a group and does not
// split the context (its own roadmap, lines 9-10).
//
// Work layout.  The queries of one (sequence, kv head) are a list of columns
// c = token * g + head_in_group: every column of the list shares the same keys
// and values.  A wavefront owns 16 * NB consecutive columns and walks the keys
// in blocks of 32.  Per block:
//   S^T[key, column] = K[key, :] . Q[column, :]        mfma 16x16x32, A = K, B = Q
//   running max / sum per column (a column lives in lanes n, n+16, n+32, n+48)
//   O^T[d, column] += V^T[d, key] * P^T[key, column]   mfma 16x16x32, A = V^T, B = P
// The rows of the two S^T tiles of a block are assigned to keys so that a lane
// ends up holding the probabilities of 8 consecutive keys: exactly the B
// operand of the second product, and the matching A operand is one 16-byte
// load from the V pages, which are stored channel-major ([page, nkv, D, page_size]).
// K pages are key-major ([page, nkv, page_size, D]): its A operand is one
// 16-byte load as well.  Nothing goes through LDS.
//
// Decode (one token per sequence, g columns) splits the context over several
// wavefronts; each writes an unnormalised partial (o, max, sum) and
// attention_combine_kernel merges them.
#include "common.h"

#if defined(SL_F32)
#error "attention_mfma is a bfloat16 kernel; the float32 path uses attention.hip"
#endif
#ifndef SL_HEAD_DIM
#error "SL_HEAD_DIM must be defined"
#endif
#if SL_HEAD_DIM % 32 != 0 || SL_HEAD_DIM > 256 || SL_HEAD_DIM < 32
#error "SL_HEAD_DIM must be a multiple of 32 in 32..256"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// 2^x by the hardware instruction; arguments here are <= 0 and tiny results may flush to 0
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int D = SL_HEAD_DIM;
constexpr int KK = D / 32;       // k-steps of the score product
constexpr int DD = D / 16;       // row tiles of the output product

struct AttnParams {
  const __bf16* qkv;             // [T, row_stride], q heads first
  int row_stride;
  const __bf16* kc;              // [pages, nkv, page, D]
  const __bf16* vc;              // [pages, nkv, D, page]
  const int* block_tables;       // [S, max_pages]
  int max_pages;
  const int* cu_q;               // [S + 1]
  const int* positions;          // [T]
  int seq_begin;                 // first sequence of this launch
  int nh, nkv, page;
  float scale;
  int window;                    // 0 = none
  int nsplit;
  __bf16* out;                   // [T, nh * D]
  float* part_o;                 // [rows, nh, nsplit, D]   (split launches)
  float* part_ml;                // [rows, nh, nsplit, 2]
  int part_row0;                 // token index of partial row 0
};

template <int NB, bool SPLIT>
__global__ __launch_bounds__(64) void attention_mfma_kernel(const AttnParams P) {
  const int lane = threadIdx.x, n = lane & 15, gq = lane >> 4;
  const int seq = P.seq_begin + blockIdx.z, kvh = blockIdx.y;
  const int g = P.nh / P.nkv;
  const int q0 = P.cu_q[seq];
  const int qlen = P.cu_q[seq + 1] - q0;
  const int ncols = qlen * g;
  const int ntiles = (ncols + 16 * NB - 1) / (16 * NB);
  const int tile_rev = blockIdx.x / P.nsplit, split = blockIdx.x % P.nsplit;
  if (tile_rev >= ntiles) return;
  const int tile = ntiles - 1 - tile_rev;          // long (late) tiles first
  const int c0 = tile * 16 * NB;
  const int pos0 = P.positions[q0];
  const int* table = P.block_tables + (size_t)seq * P.max_pages;
  const int page = P.page;

  // ---- columns of this lane
  int tok[NB], head[NB], pos_c[NB], lo_c[NB];
  bf16x8 qf[NB][KK];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    int c = c0 + 16 * b + n;
    const bool valid = c < ncols;
    if (!valid) c = ncols - 1;
    tok[b] = c / g;
    head[b] = kvh * g + c % g;
    pos_c[b] = valid ? pos0 + tok[b] : -1;         // padding: computed like its neighbour, never stored
    lo_c[b] = (P.window > 0 && pos_c[b] - P.window + 1 > 0) ? pos_c[b] - P.window + 1 : 0;
    const __bf16* q = P.qkv + (size_t)(q0 + tok[b]) * P.row_stride + (size_t)head[b] * D + 8 * gq;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[b][kk] = *(const bf16x8*)(q + 32 * kk);
  }

  // ---- key blocks of this wavefront
  const int tok_first = c0 / g;
  const int c_last = c0 + 16 * NB - 1 < ncols - 1 ? c0 + 16 * NB - 1 : ncols - 1;
  const int kmax = pos0 + c_last / g;
  int kmin = 0;
  if (P.window > 0 && pos0 + tok_first - P.window + 1 > 0) kmin = pos0 + tok_first - P.window + 1;
  int kb_begin = kmin / 32, kb_end = kmax / 32 + 1;
  if (SPLIT) {
    const int nblk = kb_end - kb_begin;
    const int first = kb_begin + (int)((long long)nblk * split / P.nsplit);
    kb_end = kb_begin + (int)((long long)nblk * (split + 1) / P.nsplit);
    kb_begin = first;
  }

  float m_run[NB], l_run[NB];
  f32x4 o[NB][DD];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    m_run[b] = -INFINITY;
    l_run[b] = 0.f;
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) o[b][dd] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // blocks every column of this wavefront sees whole need no mask
  const int full_end = (pos0 + tok_first + 1) / 32;             // blocks below: keys <= first position
  int full_begin = 0;
  if (P.window > 0) {
    const int lo_last = pos0 + c_last / g - P.window + 1;
    full_begin = lo_last > 0 ? (lo_last + 31) / 32 : 0;
  }
  const float scale_log2 = P.scale * 1.4426950408889634f;

  for (int kb = kb_begin; kb < kb_end; ++kb) {
    const int kbase = kb * 32;
    const bool edge = kb >= full_end || kb < full_begin;
    // K: row i of tile m is key kbase + 8 (i / 4) + 4 m + i % 4
    bf16x8 kf[2][KK];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const int key = kbase + 8 * (n >> 2) + 4 * m + (n & 3);
      const int pg = table[key / page];
      const __bf16* kr = P.kc + (((size_t)pg * P.nkv + kvh) * page + key % page) * D + 8 * gq;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kf[m][kk] = *(const bf16x8*)(kr + 32 * kk);
    }
    // V^T: row d, keys kbase + 8 gq .. + 7
    bf16x8 vf[DD];
    {
      const int key0 = kbase + 8 * gq;
      const int pg = table[key0 / page];
      const __bf16* vr = P.vc + ((size_t)pg * P.nkv + kvh) * D * page + key0 % page;
#pragma unroll
      for (int dd = 0; dd < DD; ++dd) vf[dd] = *(const bf16x8*)(vr + (size_t)(16 * dd + n) * page);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][kk], qf[b][kk], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][kk], qf[b][kk], s1, 0, 0, 0);
      }
      // this lane: column n, keys kbase + 8 gq + j, j = 0..7; scores in units of log 2
      float s[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) s[j] = (j < 4 ? s0[j] : s1[j - 4]) * scale_log2;
      if (edge) {                                  // a block some column does not see whole
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = kbase + 8 * gq + j;
          if (key > pos_c[b] || key < lo_c[b]) s[j] = -INFINITY;
        }
      }
      float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                       fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run[b], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const bool grew = m_new != m_run[b];
      float psum = 0.f;
      bf16x8 pb;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float p = fast_exp2(s[j] - m_safe);
        psum += p;
        pb[j] = (__bf16)p;
      }
      if (__any(grew)) {                           // rescale only when some column's maximum grew
        const float alpha = fast_exp2(m_run[b] - m_safe);
        m_run[b] = m_new;
        l_run[b] *= alpha;
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) o[b][dd] *= alpha;
      }
      l_run[b] += psum;
#pragma unroll
      for (int dd = 0; dd < DD; ++dd)
        o[b][dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dd], pb, o[b][dd], 0, 0, 0);
    }
  }

  // ---- write: lane holds column n, channels 16 dd + 4 gq + r
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    float l = l_run[b];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (pos_c[b] < 0) continue;
    const size_t row = (size_t)(q0 + tok[b]);
    if (SPLIT) {
      const size_t pr = ((row - P.part_row0) * P.nh + head[b]) * P.nsplit + split;
      float* po = P.part_o + pr * D + 4 * gq;
#pragma unroll
      for (int dd = 0; dd < DD; ++dd) *(f32x4*)(po + 16 * dd) = o[b][dd];
      if (gq == 0) {
        P.part_ml[pr * 2] = m_run[b];
        P.part_ml[pr * 2 + 1] = l;
      }
    } else {
      const float inv = 1.f / l;
      __bf16* po = P.out + (row * P.nh + head[b]) * D + 4 * gq;
#pragma unroll
      for (int dd = 0; dd < DD; ++dd) {
        bf16x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = (__bf16)(o[b][dd][j] * inv);
        *(bf16x4*)(po + 16 * dd) = r;
      }
    }
  }
}

// out[row, head, :] = sum_j w_j o_j / sum_j w_j l_j,  w_j = exp(m_j - max m).
// One wavefront per (row, head); lane j takes split j's (m, l), so nsplit <= 64;
// then the lanes split the channels and sum the partial outputs with the loads
// of eight splits in flight at a time.
__global__ __launch_bounds__(64) void attention_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int nsplit, int nh,
    int part_row0, __bf16* __restrict__ out) {
  __shared__ float ws[64];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t base = ((size_t)r * nh + h) * nsplit;
  float m = -INFINITY, l = 0.f;
  if (lane < nsplit) {
    m = part_ml[(base + lane) * 2];
    l = part_ml[(base + lane) * 2 + 1];
  }
  const float mx = wave_max(m);
  const float w = m == -INFINITY ? 0.f : fast_exp2(m - mx);     // maxima are in units of log 2
  const float denom = wave_sum(w * l);
  ws[lane] = w;
  __syncthreads();
  const float inv = 1.f / denom;
  const float* po = part_o + base * D;
  __bf16* o = out + ((size_t)(part_row0 + r) * nh + h) * D;
  for (int d = lane; d < D; d += 64) {
    float acc = 0.f;
    int j = 0;
    for (; j + 8 <= nsplit; j += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = po[(size_t)(j + u) * D + d];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += ws[j + u] * v[u];
    }
    for (; j < nsplit; ++j) acc += ws[j] * po[(size_t)j * D + d];
    o[d] = (__bf16)(acc * inv);
  }
}

extern "C" int sl_attention_mfma_head_dim() { return D; }

// One launch over sequences [seq_begin, seq_begin + num_seqs), all with at
// most max_q_len tokens.  nsplit > 1 needs part_o / part_ml for the rows
// [part_row0, part_row0 + part_rows) these sequences own (one token each).
extern "C" const char* sl_attention_mfma(
    const void* qkv, int row_stride, const void* kc, const void* vc, const int* block_tables,
    int max_pages, const int* cu_q, const int* positions, int seq_begin, int num_seqs,
    int max_q_len, int nh, int nkv, int head_dim, int page, float scale, int window, int nsplit,
    void* out, float* part_o, float* part_ml, int part_row0, int part_rows, hipStream_t stream) {
  SL_CHECK(head_dim == D, "attention_mfma: built for another head size");
  SL_CHECK(nh > 0 && nkv > 0 && nh % nkv == 0, "attention_mfma: heads must be a multiple of kv heads");
  SL_CHECK(page == 16 || page == 32 || page == 64, "attention_mfma: page size must be 16, 32 or 64");
  SL_CHECK(row_stride % 8 == 0, "attention_mfma: rows must be 16-byte aligned");
  SL_CHECK(((uintptr_t)qkv % 16) == 0 && ((uintptr_t)kc % 16) == 0 && ((uintptr_t)vc % 16) == 0,
           "attention_mfma: operands must be 16-byte aligned");
  SL_CHECK(window >= 0 && nsplit >= 1 && max_q_len >= 1, "attention_mfma: bad window, split or length");
  SL_CHECK(nkv <= 65535 && num_seqs <= 65535, "attention_mfma: grid too large");
  if (num_seqs == 0) return nullptr;
  const int g = nh / nkv;
  AttnParams P{(const __bf16*)qkv, row_stride, (const __bf16*)kc, (const __bf16*)vc, block_tables,
               max_pages, cu_q, positions, seq_begin, nh, nkv, page, scale, window, nsplit,
               (__bf16*)out, part_o, part_ml, part_row0};
  const long long cols = (long long)max_q_len * g;
  if (nsplit > 1) {
    SL_CHECK(max_q_len == 1, "attention_mfma: the context is split for single tokens only");
    SL_CHECK(part_o != nullptr && part_ml != nullptr && part_rows == num_seqs,
             "attention_mfma: a split launch needs partial buffers for its rows");
    SL_CHECK(g <= 64, "attention_mfma: more than 64 query heads per kv head");
    SL_CHECK(nsplit <= 64, "attention_mfma: at most 64 splits of the context");
    const dim3 grid(nsplit, nkv, num_seqs);
    if (g <= 16) attention_mfma_kernel<1, true><<<grid, 64, 0, stream>>>(P);
    else if (g <= 32) attention_mfma_kernel<2, true><<<grid, 64, 0, stream>>>(P);
    else attention_mfma_kernel<4, true><<<grid, 64, 0, stream>>>(P);
    const char* e = sl_launch_status();
    if (e) return e;
    attention_combine_kernel<<<dim3(num_seqs, nh), 64, 0, stream>>>(part_o, part_ml, nsplit, nh,
                                                                  part_row0, (__bf16*)out);
    return sl_launch_status();
  }
  // prompt portions: 32 columns per wavefront measured fastest on MI355X (7B shape,
  // 2,048 tokens: 133 us a layer against 154 us with 64 columns and 166 us with 16)
  if (cols <= 16) {
    attention_mfma_kernel<1, false><<<dim3(1, nkv, num_seqs), 64, 0, stream>>>(P);
  } else {
    const long long tiles = (cols + 31) / 32;
    SL_CHECK(tiles <= 1 << 30, "attention_mfma: too many column tiles");
    attention_mfma_kernel<2, false><<<dim3((unsigned)tiles, nkv, num_seqs), 64, 0, stream>>>(P);
  }
  return sl_launch_status();
}
