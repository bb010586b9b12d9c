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

// The same for up to GROUP_HEADS query heads of one kv head at a time: a decode
// row's heads of a group read the same keys and values, so one wavefront takes
// them together and every key row and value column is fetched once for all of
// them (the kernel above fetches it once per head).
constexpr int GROUP_HEADS = 8;

__global__ __launch_bounds__(64) void attention_general_group_kernel(
    const act_t* __restrict__ qkv, int row_stride, const act_t* __restrict__ kc,
    const act_t* __restrict__ vc, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, int nh, int nkv, int D,
    int page, float scale, int window, act_t* __restrict__ out, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
  __shared__ float qs[GROUP_HEADS][MAX_D];
  __shared__ float ps[GROUP_HEADS][64];
  const int t = blockIdx.x, lane = threadIdx.x;
  const int g = nh / nkv, chunks = (g + GROUP_HEADS - 1) / GROUP_HEADS;
  const int kvh = blockIdx.y / chunks, h0 = kvh * g + (blockIdx.y % chunks) * GROUP_HEADS;
  const int nheads = kvh * g + g - h0 < GROUP_HEADS ? kvh * g + g - h0 : GROUP_HEADS;
  const int s = tok_seq[t], p = positions[t];
  const int lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int* table = block_tables + (size_t)s * max_pages;
  for (int idx = lane; idx < GROUP_HEADS * D; idx += 64)      // rows past nheads: zeros, results never stored
    qs[idx / D][idx % D] = idx / D < nheads
        ? to_f(qkv[(size_t)t * row_stride + (size_t)(h0 + idx / D) * D + idx % D]) : 0.f;
  __syncthreads();

  float m[GROUP_HEADS], l[GROUP_HEADS], acc[GROUP_HEADS][MAX_D / 64];
#pragma unroll
  for (int h = 0; h < GROUP_HEADS; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_D / 64; ++i) acc[h][i] = 0.f;
  }
  const int first = lo / 64, nblk = p / 64 + 1 - first;
  const int b0 = first + (int)((long long)nblk * blockIdx.z / nsplit);
  const int b1 = first + (int)((long long)nblk * (blockIdx.z + 1) / nsplit);
  for (int kb = b0 * 64; kb < b1 * 64; kb += 64) {
    const int r = kb + lane;
    const bool valid = r >= lo && r <= p;
    float dot[GROUP_HEADS];
#pragma unroll
    for (int h = 0; h < GROUP_HEADS; ++h) dot[h] = 0.f;
    if (valid) {
      const int pg = table[r / page];
      const act_t* kr = kc + (((size_t)pg * nkv + kvh) * page + r % page) * D;
      for (int d = 0; d < D; ++d) {
        const float kv = to_f(kr[d]);
#pragma unroll
        for (int h = 0; h < GROUP_HEADS; ++h) dot[h] += qs[h][d] * kv;
      }
    }
    float alpha[GROUP_HEADS];
#pragma unroll
    for (int h = 0; h < GROUP_HEADS; ++h) {
      const float sc = valid ? dot[h] * scale : -INFINITY;
      const float mn = fmaxf(m[h], wave_max(sc));  // every block holds a visible key
      alpha[h] = expf(m[h] - mn);                  // exp(-inf) = 0 on the first block
      const float pr = valid ? expf(sc - mn) : 0.f;
      l[h] = l[h] * alpha[h] + wave_sum(pr);
      m[h] = mn;
      ps[h][lane] = pr;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < GROUP_HEADS; ++h)
#pragma unroll
      for (int i = 0; i < MAX_D / 64; ++i) acc[h][i] *= alpha[h];
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
          for (int j = 0; j < page; ++j) {
            const float v = to_f(vr[j]);
#pragma unroll
            for (int h = 0; h < GROUP_HEADS; ++h) acc[h][i] += ps[h][pb + j] * v;
          }
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int h = 0; h < GROUP_HEADS; ++h) {
    if (h >= nheads) break;
    const size_t row = (size_t)t * nh + h0 + h;
    if (nsplit > 1) {
#pragma unroll
      for (int i = 0; i < MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) part_o[(row * nsplit + blockIdx.z) * D + d] = acc[h][i];
      }
      if (lane == 0) {
        part_ml[(row * nsplit + blockIdx.z) * 2] = m[h];
        part_ml[(row * nsplit + blockIdx.z) * 2 + 1] = l[h];
      }
    } else {
      const float inv = 1.f / l[h];
#pragma unroll
      for (int i = 0; i < MAX_D / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < D) out[row * D + d] = from_f<act_t>(acc[h][i] * inv);
      }
    }
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
  // (the partial outputs of sixteen shares are asked for together: one after the other each is a trip to
  // memory; beyond the last share the weight is 0 and the value that of the last share; added in the
  // order of the shares)
  for (int d = lane; d < D; d += 64) {
    float a = 0.f;
    for (int j = 0; j < nsplit; j += 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = part_o[(base + (j + u < nsplit ? j + u : nsplit - 1)) * D + d];
#pragma unroll
      for (int u = 0; u < 16; ++u) a += (j + u < nsplit ? ws[j + u] : 0.f) * v[u];
    }
    o[d] = from_f<act_t>(a / denom);
  }
}

// ---------------------------------------------------------------------------
// Prompt portions, general sizes.  The kernel above gives a wavefront to every
// (token, head) and lets it read its keys from the cache itself: for a prompt
// of thousands of tokens every key row is fetched thousands of times.  Here a
// workgroup of four wavefronts owns TILE_COLS columns, a column being a (token,
// head of the group) pair of one sequence and one kv head, and walks the key
// blocks its columns see: a block of KB keys and values is staged in LDS as
// floats once and serves all columns; 16 lanes share a column, splitting a
// block's keys for the scores and the head's channels for the output.  Float
// FMAs only, running maximum and sum per column as above.
// ---------------------------------------------------------------------------
constexpr int TILE_COLS = 16;
constexpr int TILE_THREADS = 256;

template <int KB>
__global__ __launch_bounds__(TILE_THREADS) void attention_general_tile_kernel(
    const act_t* __restrict__ qkv, int row_stride, const act_t* __restrict__ kc,
    const act_t* __restrict__ vc, const int* __restrict__ block_tables, int max_pages,
    const int* __restrict__ cu_q, const int* __restrict__ positions, int nh, int nkv, int D,
    int page, float scale, int window, act_t* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int KS = D + 4, VS = D + 1;                  // row strides: K rows are read 16 bytes at a time, by 16 rows at once
  float* qs = lds;                                   // [TILE_COLS][D]
  float* ks = qs + TILE_COLS * D;                    // [KB][KS]
  float* vs = ks + KB * KS;                          // [KB][VS]
  float* ps = vs + KB * VS;                          // [TILE_COLS][KB]
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int sub = lane & 15;                         // this lane's place among the 16 of its column
  const int col = 4 * wave + (lane >> 4);            // column of the tile
  const int seq = blockIdx.z, kvh = blockIdx.y;
  const int g = nh / nkv;
  const int q0 = cu_q[seq], qlen = cu_q[seq + 1] - q0;
  const int ncols = qlen * g;
  const int c0 = blockIdx.x * TILE_COLS;
  if (c0 >= ncols) return;
  const int pos0 = positions[q0];
  const int* table = block_tables + (size_t)seq * max_pages;

  // the tile's columns and the keys any of them sees
  const int c = c0 + col;
  const bool live = c < ncols;
  const int tok = live ? c / g : 0, head = kvh * g + (live ? c % g : 0);
  const int pos_c = live ? pos0 + tok : -1;
  const int lo_c = window > 0 && pos_c - window + 1 > 0 ? pos_c - window + 1 : 0;
  const int tok_first = c0 / g;
  const int c_last = c0 + TILE_COLS - 1 < ncols - 1 ? c0 + TILE_COLS - 1 : ncols - 1;
  const int kmax = pos0 + c_last / g;
  int kmin = 0;
  if (window > 0 && pos0 + tok_first - window + 1 > 0) kmin = pos0 + tok_first - window + 1;

  for (int idx = t; idx < TILE_COLS * D; idx += TILE_THREADS) {
    const int cc = c0 + idx / D, d = idx % D;
    qs[idx] = cc < ncols ? to_f(qkv[(size_t)(q0 + cc / g) * row_stride + (size_t)(kvh * g + cc % g) * D + d]) : 0.f;
  }

  float m = -INFINITY, l = 0.f;
  float acc[MAX_D / 16];
#pragma unroll
  for (int j = 0; j < MAX_D / 16; ++j) acc[j] = 0.f;
  const int nd16 = D / 16;

  for (int kb = kmin / KB; kb <= kmax / KB; ++kb) {
    const int kbase = kb * KB;
    __syncthreads();                                 // the last block's readers are done (and qs is written)
    for (int idx = t; idx < KB * D; idx += TILE_THREADS) {
      {                                              // K: consecutive threads along a key's channels
        const int key = kbase + idx / D, d = idx % D;
        float v = 0.f;
        if (key >= kmin && key <= kmax) {
          const int pg = table[key / page];
          v = to_f(kc[(((size_t)pg * nkv + kvh) * page + key % page) * D + d]);
        }
        ks[(idx / D) * KS + d] = v;
      }
      {                                              // V^T in the cache: consecutive threads along a channel's keys
        const int kk = idx % KB, d = idx / KB, key = kbase + kk;
        float v = 0.f;
        if (key >= kmin && key <= kmax) {
          const int pg = table[key / page];
          v = to_f(vc[(((size_t)pg * nkv + kvh) * D + d) * page + key % page]);
        }
        vs[kk * VS + d] = v;
      }
    }
    __syncthreads();
    // scores of this lane's keys sub, sub + 16, ... of the block
    float sc[KB / 16];
#pragma unroll
    for (int r = 0; r < KB / 16; ++r) sc[r] = 0.f;
    const float* qrow = qs + col * D;
    for (int d = 0; d < D; d += 4) {
      const float4 q4 = *(const float4*)(qrow + d);
#pragma unroll
      for (int r = 0; r < KB / 16; ++r) {
        const float4 k4 = *(const float4*)(ks + (sub + 16 * r) * KS + d);
        sc[r] += q4.x * k4.x + q4.y * k4.y + q4.z * k4.z + q4.w * k4.w;
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < KB / 16; ++r) {
      const int key = kbase + sub + 16 * r;
      sc[r] = key >= lo_c && key <= pos_c ? sc[r] * scale : -INFINITY;
      mx = fmaxf(mx, sc[r]);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    const float mn = fmaxf(m, mx);
    // a column that has seen no key yet keeps m = -inf: nothing to rescale, nothing to add
    const float alpha = mn == -INFINITY ? 1.f : expf(m - mn);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < KB / 16; ++r) {
      const float pr = sc[r] == -INFINITY ? 0.f : expf(sc[r] - mn);
      psum += pr;
      ps[col * KB + sub + 16 * r] = pr;
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, 64);
    l = l * alpha + psum;
    m = mn;
    __syncthreads();                                 // ps is complete
#pragma unroll
    for (int j = 0; j < MAX_D / 16; ++j) acc[j] *= alpha;
    const float* prow = ps + col * KB;
    for (int kk = 0; kk < KB; ++kk) {
      const float pk = prow[kk];
      const float* vrow = vs + kk * VS + sub;
#pragma unroll
      for (int j = 0; j < MAX_D / 16; ++j)
        if (j < nd16) acc[j] += pk * vrow[16 * j];
    }
  }
  if (!live) return;
  const float inv = 1.f / l;
  act_t* o = out + ((size_t)(q0 + tok) * nh + head) * D + sub;
#pragma unroll
  for (int j = 0; j < MAX_D / 16; ++j)
    if (j < nd16) o[16 * j] = from_f<act_t>(acc[j] * inv);
}

// Sequences [0, num_seqs) of the batch, prompt portions of at most max_q_len
// tokens each (their tokens come first in the batch).  D % 16 == 0.
extern "C" const char* sl_attention_general_tiles(
    const void* qkv, int row_stride, const void* kc, const void* vc, const int* block_tables,
    int max_pages, const int* cu_q, const int* positions, int num_seqs, int max_q_len, int nh,
    int nkv, int D, int page, float scale, int window, void* out, hipStream_t stream) {
  SL_CHECK(num_seqs >= 0 && max_q_len >= 1 && nh > 0 && nkv > 0 && nh % nkv == 0,
           "attention tiles: heads must be a positive multiple of kv heads");
  SL_CHECK(D > 0 && D <= MAX_D && D % 16 == 0, "attention tiles: head_dim must be a multiple of 16 up to 256");
  SL_CHECK(page == 16 || page == 32 || page == 64, "attention tiles: page size must be 16, 32 or 64");
  SL_CHECK(nkv <= 65535 && num_seqs <= 65535, "attention tiles: grid too large");
  SL_CHECK(window >= 0, "attention tiles: window must be >= 0 (0 = none)");
  if (num_seqs == 0) return nullptr;
  const long long cols = (long long)max_q_len * (nh / nkv);
  const long long tiles = (cols + TILE_COLS - 1) / TILE_COLS;
  SL_CHECK(tiles <= 1 << 30, "attention tiles: too many column tiles");
  const dim3 grid((unsigned)tiles, nkv, num_seqs);
  const int KB = D <= 128 ? 32 : 16;
  const size_t bytes = sizeof(float) * ((size_t)TILE_COLS * D + (size_t)KB * (D + 4) + (size_t)KB * (D + 1) +
                                        (size_t)TILE_COLS * KB);
  SL_CHECK(bytes <= 65536, "attention tiles: LDS need exceeds 64 KB");
  if (KB == 32)
    attention_general_tile_kernel<32><<<grid, TILE_THREADS, bytes, stream>>>(
        (const act_t*)qkv, row_stride, (const act_t*)kc, (const act_t*)vc, block_tables, max_pages,
        cu_q, positions, nh, nkv, D, page, scale, window, (act_t*)out);
  else
    attention_general_tile_kernel<16><<<grid, TILE_THREADS, bytes, stream>>>(
        (const act_t*)qkv, row_stride, (const act_t*)kc, (const act_t*)vc, block_tables, max_pages,
        cu_q, positions, nh, nkv, D, page, scale, window, (act_t*)out);
  return sl_launch_status();
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
  const int g = nh / nkv;
  if (g > 1) {                                       // the heads of a group together
    const int chunks = (g + GROUP_HEADS - 1) / GROUP_HEADS;
    attention_general_group_kernel<<<dim3(T, nkv * chunks, nsplit), 64, 0, stream>>>(
        (const act_t*)qkv, row_stride, (const act_t*)kc, (const act_t*)vc, block_tables, max_pages,
        tok_seq, positions, nh, nkv, D, page, scale, window, (act_t*)out, nsplit, part_o, part_ml);
  } else {
    attention_general_kernel<<<dim3(T, nh, nsplit), 64, 0, stream>>>(
        (const act_t*)qkv, row_stride, (const act_t*)kc, (const act_t*)vc, block_tables, max_pages,
        tok_seq, positions, nh, nkv, D, page, scale, window, (act_t*)out, nsplit, part_o, part_ml);
  }
  const char* e = sl_launch_status();
  if (e || nsplit == 1) return e;
  attention_general_combine_kernel<<<dim3(T, nh), 64, 0, stream>>>(part_o, part_ml, nsplit, nh, D,
                                                                 (act_t*)out);
  return sl_launch_status();
}
