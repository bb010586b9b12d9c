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
// 16-byte load as well.
//
// Four launches share that inner block (struct Columns):
//   - decode (one token per sequence, g columns), few sequences: the context
//     is split over several wavefronts, each a workgroup of its own; each
//     writes an unnormalised partial (o, reference, sum) and
//     attention_combine_kernel merges them;
//   - decode, a (sequence, kv head) pair or more for every CU: a workgroup of
//     eight wavefronts per pair that split the context and merge in LDS
//     (attention_mfma_group_kernel);
//   - prompt portions, four wavefronts per workgroup that share each block of
//     keys and values through LDS (attention_mfma_shared_kernel), the launch
//     laid out by chiplet; tiles of a portion deep in its context cut into
//     shares of their keys, merged by attention_combine_kernel;
//   - prompt portions, one wavefront per 32 columns, operands straight from
//     the pages, two wavefronts per SIMD so that one computes while the other
//     waits for its loads: for head sizes whose blocks do not fit the LDS ring.
// The softmax keeps a reference point per column instead of the exact running
// maximum (see LAZY) and folds the scale into the exponent's multiply-add.
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

// Maximum / sum over the four lanes n, n + 16, n + 32, n + 48 that share a
// column, by the row-swap instructions of gfx950 (register to register, no
// trip through LDS): after a swap of x with itself one result holds the lower
// partner and the other the upper one, in every lane.
__device__ __forceinline__ float column_max(float x) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float column_sum(float x) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

constexpr int D = SL_HEAD_DIM;
constexpr int KK = D / 32;       // k-steps of the score product
constexpr int DD = D / 16;       // row tiles of the output product
constexpr float LAZY = 8.f;      // growth of a column's maximum (log 2 units) that moves its reference point

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
  int nh, nkv, page;             // page: 16, 32 or 64 keys
  float scale;
  int window;                    // 0 = none
  int nsplit;
  __bf16* out;                   // [T, nh * D]
  float* part_o;                 // [rows, nh, nsplit, D]   (split launches)
  float* part_ml;                // [rows, nh, nsplit, 2]
  int part_row0;                 // token index of partial row 0
  int pair;                      // prompt workgroups take a late tile and its early mirror
  int out_rows;                  // 0: out is [T, nh * D]; else its rows are laid out by k-step for the few-rows
                                 // product that reads them: element (t, c) at (c / 32) * (out_rows * 32) + t * 32 + c % 32
  int by_chiplet;                // a one-dimensional grid laid out by Place below (else x: workgroup of a pair, y: kv head, z: sequence;
                                 // split single tokens: x: kv head, y: sequence, z: share)
  int grid_x, num_seqs;          // ... its extent per (sequence, kv head) pair, and the sequences
  // Split single tokens: shares of one length for all sequences of the launch instead of nsplit shares each (see
  // share_count).  ctx_stats: the sum and the largest of the launch's context lengths, on the device (they change from
  // step to step under a captured graph); share_waves: the wavefronts the launch aims at; null / 0: nsplit shares each.
  const int* ctx_stats;
  int share_waves;
};

// where element (row, col) of the result goes (col = head * D + channel; runs of four channels stay together)
__device__ __forceinline__ size_t out_index(int out_rows, int nh, size_t row, int col) {
  return out_rows ? (size_t)(col / 32) * (out_rows * 32) + row * 32 + col % 32 : row * (size_t)(nh * D) + col;
}

// Workgroups go to the eight chiplets in turn (workgroup i to chiplet i % 8), and each chiplet has an L2 of
// its own.  The workgroups of one kv head read the same keys and values, so a launch laid out head by head
// spreads every head's keys over all eight L2s: eight times the footprint, and beyond a few thousand tokens
// the keys come from memory again and again (7B shape, 8,192 tokens: 644 us; laid out as below: 533 us).
// Laid out by chiplet, a kv head's workgroups all run on the 8 / nkv chiplets it has to itself (or, with
// 8, 16, .. kv heads, on the one chiplet it shares with nkv / 8 - 1 others); the workgroups of a head are
// dealt to its chiplets in turn, first workgroup of every sequence first, so each chiplet gets the same mix
// of long and short tiles.
struct Place {
  int x, kvh, seq;
  bool valid;
  __device__ __forceinline__ Place(const AttnParams& P) {
    if (!P.by_chiplet) {
      x = blockIdx.x, kvh = blockIdx.y, seq = P.seq_begin + blockIdx.z, valid = true;
      return;
    }
    const int chiplet = blockIdx.x & 7, idx = blockIdx.x >> 3;
    if (P.nkv < 8) {
      const int each = 8 / P.nkv;                  // chiplets a head: each takes every each-th workgroup of every sequence
      const int per_seq = (P.grid_x + each - 1) / each;
      kvh = chiplet % P.nkv;
      x = idx % per_seq * each + chiplet / P.nkv;
      seq = P.seq_begin + idx / per_seq;
    } else {
      const int share = P.nkv / 8;                 // heads a chiplet
      kvh = chiplet + 8 * (idx % share);
      x = idx / share % P.grid_x;
      seq = P.seq_begin + idx / share / P.grid_x;
    }
    valid = x < P.grid_x;
  }
};

// The columns of one wavefront: queries, reference points and sums, outputs.
//
// Vector work per score is what limits these kernels beside the matrix
// products (a block of 32 keys is 32 matrix instructions a wavefront, and was
// about 150 vector instructions), so the softmax is arranged to need few:
//   - FOLD: the queries arrive multiplied by scale * log2(e) (the producer of q
//     does that before its one rounding), and the score product starts from an
//     accumulator that holds -reference point: the matrix cores deliver
//     s * scale * log2(e) - m, ready for exp2, with no multiply-add per score;
//   - the sums of the probabilities come from the matrix cores as well (one
//     more product of P with a tile of ones), not from an add per score;
//   - a lane compares only its own largest score with the threshold, and takes
//     that largest over the scores' bit patterns as integers (v_max3_i32: no
//     quieting of NaNs around every maximum; above a positive threshold the
//     order of the patterns is the order of the floats); the maximum over the
//     lanes of a column is taken only when some lane's has crossed it and the
//     reference point has to move, which is rare.
template <int NB, bool FOLD>
struct Columns {
  int tok[NB], head[NB], pos_c[NB], lo_c[NB];
  bf16x8 qf[NB][KK];
  int thr[NB];                   // bit pattern of the score (less the reference) above which the reference moves;
                                 // UNSET before the column's first visible key, when there is no reference yet:
                                 // every pattern but that of -0 lies above it, and -0 no score is (the products
                                 // are added to an accumulator that starts at +0 then)
  static constexpr int UNSET = -2147483647 - 1;
  f32x4 negm[NB];                // -reference point (units of log 2) in all four entries; 0 before there is one
  f32x4 l_acc[NB];               // sum of the probabilities, every entry the same
  f32x4 o[NB][DD];
  int kb_begin, kb_end;          // key blocks (of 32) some column sees
  int full_begin, full_end;      // blocks in [full_begin, full_end) are seen whole by every column
  float scale_log2;

  __device__ __forceinline__ void init(const AttnParams& P, int q0, int ncols, int c0, int pos0,
                                       int kvh, int g, int n, int gq) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      int c = c0 + 16 * b + n;
      const bool valid = c < ncols;
      if (!valid) c = ncols - 1;
      tok[b] = c / g;
      head[b] = kvh * g + c % g;
      pos_c[b] = valid ? pos0 + tok[b] : -1;       // padding: computed like its neighbour, never stored
      lo_c[b] = (P.window > 0 && pos_c[b] - P.window + 1 > 0) ? pos_c[b] - P.window + 1 : 0;
      const __bf16* q = P.qkv + (size_t)(q0 + tok[b]) * P.row_stride + (size_t)head[b] * D + 8 * gq;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) qf[b][kk] = *(const bf16x8*)(q + 32 * kk);
      thr[b] = UNSET;
      negm[b] = f32x4{0.f, 0.f, 0.f, 0.f};
      l_acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dd = 0; dd < DD; ++dd) o[b][dd] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // The queries have to be in their registers before the loop over the key blocks starts: the
    // counter of outstanding loads is one for all of them, so a wait for a query inside the loop
    // would, on every pass, also wait for the keys and values just requested for the next block.
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) asm volatile("" : "+v"(qf[b][kk]));
    const int tok_first = c0 / g;
    const int c_last = c0 + 16 * NB - 1 < ncols - 1 ? c0 + 16 * NB - 1 : ncols - 1;
    const int kmax = pos0 + c_last / g;
    int kmin = 0;
    if (P.window > 0 && pos0 + tok_first - P.window + 1 > 0) kmin = pos0 + tok_first - P.window + 1;
    kb_begin = kmin / 32;
    kb_end = kmax / 32 + 1;
    full_end = (pos0 + tok_first + 1) / 32;        // blocks below: keys <= first position
    full_begin = 0;
    if (P.window > 0) {
      const int lo_last = pos0 + c_last / g - P.window + 1;
      full_begin = lo_last > 0 ? (lo_last + 31) / 32 : 0;
    }
    scale_log2 = P.scale * 1.4426950408889634f;
  }

  // Scores of tile b for one block of 32 keys, less the reference point and in
  // units of log 2: this lane gets column n, keys kbase + 8 gq + j, j = 0..7.
  // kf: row i of tile m is key kbase + 8 (i / 4) + 4 m + i % 4.
  __device__ __forceinline__ void scores(int b, const bf16x8 (&kf)[2][KK], f32x4& s0, f32x4& s1) const {
    s0 = FOLD ? negm[b] : f32x4{0.f, 0.f, 0.f, 0.f};
    s1 = s0;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][kk], qf[b][kk], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][kk], qf[b][kk], s1, 0, 0, 0);
    }
  }

  // From the products to what exp2 takes, with the keys a column does not see
  // masked out on edge blocks; returns the largest of this lane's bit patterns.
  __device__ __forceinline__ int settle(int b, const f32x4& s0, const f32x4& s1, bool edge, int kbase,
                                        int gq, float (&s)[8]) const {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float raw = j < 4 ? s0[j] : s1[j - 4];
      s[j] = FOLD ? raw : fmaf(raw, scale_log2, negm[b][0]);
    }
    if (edge) {                                    // a block some column does not see whole
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = kbase + 8 * gq + j;
        if (key > pos_c[b] || key < lo_c[b]) s[j] = -INFINITY;
      }
    }
    int top = __float_as_int(s[0]);
#pragma unroll
    for (int j = 1; j < 8; ++j) top = max(top, __float_as_int(s[j]));
    return top;
  }

  // The reference point of a column moves up to its largest score so far (and
  // is set by the first visible key): outputs and sums are rescaled, the
  // scores of this block shifted.  It is a reference, not the exact running
  // maximum: until a score exceeds it by LAZY (in units of log 2) it stays, so
  // probabilities reach 2^LAZY at most, far from any overflow, with the same
  // relative rounding, and this path is rare.
  __device__ __forceinline__ void move(int b, float (&s)[8]) {
    const float lane_max = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    const float top = column_max(lane_max) - negm[b][0];          // back in absolute units
    const float m_old = reference(b);
    if (!(top > m_old)) return;
    const float alpha = m_old == -INFINITY ? 0.f : fast_exp2(m_old - top);
    const float shift = -top - negm[b][0];
#pragma unroll
    for (int j = 0; j < 8; ++j) s[j] += shift;
    thr[b] = __float_as_int(LAZY);
    negm[b] = f32x4{-top, -top, -top, -top};
    l_acc[b] *= alpha;
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) o[b][dd] *= alpha;
  }

  __device__ __forceinline__ float reference(int b) const {
    return thr[b] == UNSET ? -INFINITY : -negm[b][0];
  }

  __device__ __forceinline__ bf16x8 probabilities(const float (&s)[8]) const {
    bf16x8 pb;
#pragma unroll
    for (int j = 0; j < 8; ++j) pb[j] = (__bf16)fast_exp2(s[j]);
    return pb;
  }

  // O^T += V^T P^T and the column sums of P (a tile of ones in the place of V^T).
  __device__ __forceinline__ void weigh(int b, const bf16x8 (&vf)[DD], const bf16x8& pb) {
    const __bf16 one = (__bf16)1.0f;
    const bf16x8 ones = {one, one, one, one, one, one, one, one};
    l_acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb, l_acc[b], 0, 0, 0);
#pragma unroll
    for (int dd = 0; dd < DD; ++dd)
      o[b][dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dd], pb, o[b][dd], 0, 0, 0);
  }

  // One block of 32 keys.  vf: row d of V^T, keys kbase + 8 gq .. + 7.
  __device__ __forceinline__ void block(int kb, const bf16x8 (&kf)[2][KK], const bf16x8 (&vf)[DD],
                                        int gq) {
    const int kbase = kb * 32;
    const bool edge = kb >= full_end || kb < full_begin;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      f32x4 s0, s1;
      float s[8];
      scores(b, kf, s0, s1);
      const int lane_top = settle(b, s0, s1, edge, kbase, gq, s);
      if (__builtin_expect(__any(lane_top > thr[b]), 0)) move(b, s);
      weigh(b, vf, probabilities(s));
    }
  }

  // The same block with the work of the NB column tiles side by side instead
  // of one after the other: all score products first, one check whether any
  // reference point has to move, then probabilities and output products, so
  // that the vector work of one tile has matrix work of the other beside it.
  __device__ __forceinline__ void block_abreast(int kb, const bf16x8 (&kf)[2][KK], const bf16x8 (&vf)[DD],
                                                int gq) {
    const int kbase = kb * 32;
    const bool edge = kb >= full_end || kb < full_begin;
    f32x4 s0[NB], s1[NB];
    float s[NB][8];
    bool crossed = false;
#pragma unroll
    for (int b = 0; b < NB; ++b) scores(b, kf, s0[b], s1[b]);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const int lane_top = settle(b, s0[b], s1[b], edge, kbase, gq, s[b]);
      crossed = crossed || lane_top > thr[b];
    }
    if (__builtin_expect(__any(crossed), 0)) {
#pragma unroll
      for (int b = 0; b < NB; ++b) move(b, s[b]);
    }
    bf16x8 pb[NB];
    pb[0] = probabilities(s[0]);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (b + 1 < NB) pb[b + 1] = probabilities(s[b + 1]);       // beside the products of tile b
      weigh(b, vf, pb[b]);
    }
  }

  // lane holds column n, channels 16 dd + 4 gq + r
  template <bool SPLIT>
  __device__ __forceinline__ void store(const AttnParams& P, int q0, int split, int gq) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const float l = l_acc[b][0];
      if (pos_c[b] < 0) continue;
      const size_t row = (size_t)(q0 + tok[b]);
      if (SPLIT) {
        const size_t pr = ((row - P.part_row0) * P.nh + head[b]) * P.nsplit + split;
        float* po = P.part_o + pr * D + 4 * gq;
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) *(f32x4*)(po + 16 * dd) = o[b][dd];
        if (gq == 0) {
          P.part_ml[pr * 2] = reference(b);
          P.part_ml[pr * 2 + 1] = l;
        }
      } else {
        const float inv = 1.f / l;
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) {
          bf16x4 r;
#pragma unroll
          for (int j = 0; j < 4; ++j) r[j] = (__bf16)(o[b][dd][j] * inv);
          *(bf16x4*)(P.out + out_index(P.out_rows, P.nh, row, head[b] * D + 16 * dd + 4 * gq)) = r;
        }
      }
    }
  }
};

// The key blocks [kb_begin, kb_end) of one wavefront's columns, operands straight from the pages.
template <int NB, bool FOLD, bool PAIRS>
__device__ __forceinline__ void walk_blocks(Columns<NB, FOLD>& C, const AttnParams& P, const int* table, int kvh,
                                            int n, int gq, int kb_begin, int kb_end) {
  const int page = P.page, page_shift = 31 - __builtin_clz(page);
  // The two table entries a block of 32 keys can touch are the same for every
  // lane, so they come through the scalar path, one block ahead of the keys.
  auto load_pages = [&](int kb, int (&pg)[2]) {
    const int kbase = kb * 32;
    pg[0] = table[kbase >> page_shift];
    pg[1] = table[(kbase + 16) >> page_shift];
  };
  auto load_block = [&](int kb, const int (&pg)[2], bf16x8 (&kf)[2][KK], bf16x8 (&vf)[DD]) {
    const int kbase = kb * 32;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const int ko = 8 * (n >> 2) + 4 * m + (n & 3);
      const int p = ko < 16 ? pg[0] : pg[1];
      const __bf16* kr = P.kc + (((size_t)p * P.nkv + kvh) * page + ((kbase + ko) & (page - 1))) * D + 8 * gq;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kf[m][kk] = __builtin_nontemporal_load((const bf16x8*)(kr + 32 * kk));
    }
    const int p = gq < 2 ? pg[0] : pg[1];
    const __bf16* vr = P.vc + ((size_t)p * P.nkv + kvh) * D * page + ((kbase + 8 * gq) & (page - 1));
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) vf[dd] = __builtin_nontemporal_load((const bf16x8*)(vr + (size_t)(16 * dd + n) * page));
  };

  // Two wavefronts share a SIMD where the registers allow it: one computes
  // while the other waits for its keys and values.  (Requesting the next block
  // into a second set of registers instead, at one wavefront per SIMD, measured
  // slower on MI355X for prompt tiles: 132 us against 97 us for 2,048 tokens of
  // the 7B shape.)  PAIRS, for split decode launches, whose wavefronts mostly
  // have a SIMD to themselves: two blocks are asked for at once and the page
  // ids of the next two before that, so a wavefront makes half as many trips to
  // memory (7B shape, contexts of 4,096: +1.5 % tokens/s at batch 8, +6.5 % at 64).
  if (kb_begin >= kb_end) return;
  if (PAIRS) {
    int kb = kb_begin;
    int pga[2], pgb[2], pga_next[2], pgb_next[2];
    const int last = kb_end - 1;
    load_pages(kb, pga_next);
    load_pages(kb < last ? kb + 1 : last, pgb_next);
    for (; kb + 1 < kb_end; kb += 2) {
      bf16x8 kfa[2][KK], vfa[DD], kfb[2][KK], vfb[DD];
      pga[0] = pga_next[0], pga[1] = pga_next[1], pgb[0] = pgb_next[0], pgb[1] = pgb_next[1];
      load_pages(kb + 2 < last ? kb + 2 : last, pga_next);
      load_pages(kb + 3 < last ? kb + 3 : last, pgb_next);
      load_block(kb, pga, kfa, vfa);
      load_block(kb + 1, pgb, kfb, vfb);
      C.block(kb, kfa, vfa, gq);
      C.block(kb + 1, kfb, vfb, gq);
    }
    if (kb < kb_end) {
      bf16x8 kf[2][KK], vf[DD];
      load_block(kb, pga_next, kf, vf);
      C.block(kb, kf, vf, gq);
    }
  } else {
    int pg[2], pg_next[2];
    const int last = kb_end - 1;
    load_pages(kb_begin, pg_next);
    for (int kb = kb_begin; kb < kb_end; ++kb) {
      bf16x8 kf[2][KK], vf[DD];
      pg[0] = pg_next[0];
      pg[1] = pg_next[1];
      load_pages(kb < last ? kb + 1 : last, pg_next);
      load_block(kb, pg, kf, vf);
      C.block(kb, kf, vf, gq);
    }
  }
}

// Into how many shares the nblk key blocks of a single token's sequence are cut, nsplit at most.  With
// contexts of different lengths, nsplit shares for every sequence would leave the launch waiting for
// the shares of its longest sequence while the wavefronts of the short ones have long finished (7B
// shape, 64 requests of which 8 have 4,096 keys and the others a few hundred, merged in the
// workgroup or in 4 shares each: 62 and 72 us a layer; streaming their keys takes 18).  So every share
// of the launch gets about the same number of blocks: the launch's blocks (from the sum of its
// contexts) over the wavefronts it aims at, no fewer than its longest sequence needs to fit nsplit
// shares; a long sequence is cut into many, a short one into one, and the wavefronts of the shares a
// sequence does not use leave at once.  Equal contexts give every sequence share_waves / pairs shares.
__device__ __forceinline__ int share_count(const AttnParams& P, int nblk) {
  if (P.ctx_stats == nullptr || P.share_waves <= 0) return P.nsplit;
  long long total = P.ctx_stats[0];
  int longest = P.ctx_stats[1];
  if (P.window > 0) {                                // (a window bounds what a sequence reads)
    longest = longest < P.window + 31 ? longest : P.window + 31;
    total = total < (long long)P.num_seqs * longest ? total : (long long)P.num_seqs * longest;
  }
  const long long blocks = (total / 32 + P.num_seqs) * P.nkv;                 // key blocks of all pairs, rounded up
  // (contexts of different lengths: up to twice the wavefronts, of shorter shares, which even out better;
  // equal contexts keep the count the launch was planned with, whose wavefronts fill whole rounds of the CUs)
  long long aim = (long long)P.share_waves * longest * P.num_seqs / (total > 0 ? total : 1);
  aim = aim < P.share_waves ? P.share_waves : aim < 2ll * P.share_waves ? aim : 2ll * P.share_waves;
  int each = (int)((blocks + aim - 1) / aim);
  const int fit = (longest / 32 + P.nsplit) / P.nsplit;                         // ceil((longest / 32 + 1) / nsplit)
  each = each > fit ? each : fit;
  each = each > 2 ? each : 2;
  const int n = (nblk + each - 1) / each;
  return n < 1 ? 1 : n < P.nsplit ? n : P.nsplit;
}

// One wavefront per workgroup; operands straight from the pages.  Used for
// decode tokens (SPLIT: the wavefront takes one share of the key blocks) and
// for prompt portions whose launch does not saturate L2.
template <int NB, bool SPLIT, bool FOLD, bool PAIRS = false, bool ONE_LENGTH = false>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(NB * D <= 256 ? 2 : 1))) void attention_mfma_kernel(const AttnParams P) {
  const int lane = threadIdx.x, n = lane & 15, gq = lane >> 4;
  // Split single tokens come as a grid of (kv head, sequence, share), which is handed out as all (sequence,
  // kv head) pairs of share 0, then those of share 1, ...  Workgroups go to the eight chiplets in turn
  // (workgroup L to chiplet L % 8), and both the shares of one pair and the pairs of one share should go
  // round them: a long sequence among short ones then loads all chiplets, and so do sequences that use only
  // the first few of their shares (with the share as the fastest index, eight slots and two shares in use,
  // two chiplets did all the work).  With a number of pairs that is no multiple of 8 the order does that by
  // itself (each share begins pairs % 8 chiplets further on); with a multiple of 8 the pairs of every eight
  // are rotated by the share and by the number of the eight, so that workgroup L is a pair with
  // (pair + share + pair / 8) % 8 = L % 8.  (No places are left empty to make eights: a workgroup that leaves
  // at once still takes its turn in the order in which a chiplet hands workgroups to its CUs, and with 4
  // pairs, one request of the 7B shape, half the CUs then got two wavefronts and half none: 12.0 against
  // 9.8 us a layer.)  Nothing here may stand between the kernel's arguments and its first read of memory
  // that need not: with one request the launch is a chain of five trips to memory and little else.
  int seq = P.seq_begin + blockIdx.y, kvh = SPLIT ? blockIdx.x : blockIdx.y;
  if (!SPLIT) seq = P.seq_begin + blockIdx.z;
  if (SPLIT && (gridDim.x * gridDim.y) % 8 == 0) {
    const int place = blockIdx.x + gridDim.x * blockIdx.y;
    const int pair_of = (place & ~7) | ((place - (int)blockIdx.z - (place >> 3)) & 7);
    seq = P.seq_begin + pair_of / (int)gridDim.x;
    kvh = pair_of % (int)gridDim.x;
  }
  const int g = P.nh / P.nkv;
  const int q0 = P.cu_q[seq];
  const int qlen = P.cu_q[seq + 1] - q0;
  const int ncols = qlen * g;
  const int ntiles = (ncols + 16 * NB - 1) / (16 * NB);
  const int tile_rev = SPLIT ? 0 : blockIdx.x / P.nsplit, split = SPLIT ? blockIdx.z : blockIdx.x % P.nsplit;
  if (tile_rev >= ntiles) return;
  const int tile = ntiles - 1 - tile_rev;          // long (late) tiles first
  const int pos0 = P.positions[q0];
  const int* table = P.block_tables + (size_t)seq * P.max_pages;
  int shares = P.nsplit;
  if (SPLIT && ONE_LENGTH) {
    // (a kernel of its own: the count needs the token's position, and a wavefront that has to wait for it
    // before it may ask for its queries starts a trip to memory later, 1.6 us of the 9.8 of a launch for one
    // request of the 7B shape at 4,096 keys)
    // (a single token: the blocks from its window's first key to its own position, as Columns::init finds them)
    const int kmin = P.window > 0 && pos0 - P.window + 1 > 0 ? pos0 - P.window + 1 : 0;
    shares = share_count(P, pos0 / 32 + 1 - kmin / 32);
    if (split >= shares) {
      // a share this sequence does not use: nothing but the mark that the combine kernel skips
      if (lane < g) {
        const size_t pr = (((size_t)q0 - P.part_row0) * P.nh + kvh * g + lane) * P.nsplit + split;
        P.part_ml[pr * 2] = -INFINITY;
        P.part_ml[pr * 2 + 1] = 0.f;
      }
      return;
    }
  }

  Columns<NB, FOLD> C;
  C.init(P, q0, ncols, tile * 16 * NB, pos0, kvh, g, n, gq);
  int kb_begin = C.kb_begin, kb_end = C.kb_end;
  if (SPLIT) {
    const int nblk = kb_end - kb_begin;
    const int first = kb_begin + (int)((long long)nblk * split / shares);
    kb_end = kb_begin + (int)((long long)nblk * (split + 1) / shares);
    kb_begin = first;
  }
  walk_blocks<NB, FOLD, PAIRS>(C, P, table, kvh, n, gq, kb_begin, kb_end);
  C.template store<SPLIT>(P, q0, split, gq);
}

// Decode tokens, a workgroup of GROUP_WAVES wavefronts per (sequence, kv head): the wavefronts cut the
// key blocks among themselves, each walks its own as above, and they merge their results in LDS:
// out = sum_w 2^(m_w - m) o_w / sum_w 2^(m_w - m) l_w, m the largest reference point.  The workgroup
// writes the rows of the result itself and no second kernel follows (a kernel that only waits for
// this one's partial results costs 4-5 us a layer whatever it does).  How a request's keys are cut
// depends on its own context and the workgroup's size only, not on what else is in the batch.
constexpr int GROUP_WAVES = 8;
// column tiles whose partial results fit LDS: two (up to 32 query heads a kv head) for head sizes up to 128, else one
constexpr int GROUP_MAX_NB = GROUP_WAVES * 32 * (D + 4) * 4 <= 150 * 1024 ? 2 : 1;
template <int NB, bool FOLD>
__global__ __launch_bounds__(64 * GROUP_WAVES) __attribute__((amdgpu_waves_per_eu(NB * D <= 256 ? 2 : 1)))
void attention_mfma_group_kernel(const AttnParams P) {
  constexpr int COLS = 16 * NB, PITCH = D + 4;       // (rows of D + 4 floats: the 16 lanes of a column tile write to different banks)
  __shared__ __attribute__((aligned(16))) float so[GROUP_WAVES][COLS][PITCH];
  __shared__ float sm[GROUP_WAVES][COLS], sl[GROUP_WAVES][COLS];
  const int t = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(t >> 6), lane = t & 63, n = lane & 15, gq = lane >> 4;
  const int seq = P.seq_begin + blockIdx.y, kvh = blockIdx.x;
  const int g = P.nh / P.nkv;                        // (one token a sequence: its g columns are one tile)
  const int q0 = P.cu_q[seq];
  const int pos0 = P.positions[q0];
  const int* table = P.block_tables + (size_t)seq * P.max_pages;

  Columns<NB, FOLD> C;
  C.init(P, q0, g, 0, pos0, kvh, g, n, gq);
  const int nblk = C.kb_end - C.kb_begin;
  // (two blocks asked for at once where the registers hold them: one column tile)
  walk_blocks<NB, FOLD, NB == 1>(C, P, table, kvh, n, gq, C.kb_begin + nblk * wave / GROUP_WAVES,
                              C.kb_begin + nblk * (wave + 1) / GROUP_WAVES);
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (C.pos_c[b] < 0) continue;                    // padding columns
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) *(f32x4*)&so[wave][16 * b + n][16 * dd + 4 * gq] = C.o[b][dd];
    if (gq == 0) {
      sm[wave][16 * b + n] = C.reference(b);
      sl[wave][16 * b + n] = C.l_acc[b][0];
    }
  }
  __syncthreads();
  for (int idx = t; idx < g * (D / 4); idx += 64 * GROUP_WAVES) {
    const int col = idx / (D / 4), d = 4 * (idx % (D / 4));
    float top = -INFINITY;
#pragma unroll
    for (int w = 0; w < GROUP_WAVES; ++w) top = fmaxf(top, sm[w][col]);
    f32x4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
#pragma unroll
    for (int w = 0; w < GROUP_WAVES; ++w) {
      const float m = sm[w][col];
      const float wt = m == -INFINITY ? 0.f : fast_exp2(m - top);
      num += wt * *(const f32x4*)&so[w][col][d];                      // (a wavefront without keys wrote zeros)
      den += wt * sl[w][col];
    }
    const float inv = 1.f / den;
    bf16x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = (__bf16)(num[j] * inv);
    *(bf16x4*)(P.out + out_index(P.out_rows, P.nh, (size_t)q0, (kvh * g + col) * D + d)) = r;
  }
}

// Prompt portions: four wavefronts, one per SIMD, take 32 columns each and
// share every block of keys and values through LDS, so a block leaves the
// cache hierarchy once per 128 columns instead of once per 32 (measured on
// MI355X: with one wavefront per workgroup the kernel ran at the rate at which
// L2 delivers the operands, 32 flop a byte, not at the rate of the matrix
// cores).
//
// The blocks travel from the pages straight into LDS (global_load_lds_dwordx4
// of gfx950: a wavefront's 64 loads of 16 bytes land side by side in 1 KB of
// LDS, each lane choosing its own source), into a ring of STAGES buffers:
// while block kb is computed, the loads of the next STAGES - 1 blocks are on
// their way, no register carries them, no wavefront writes them to LDS, and
// the one wait before the barrier at the end of a block is for loads asked for
// a whole block earlier.  (Measured with the loads going through registers
// and ds_write, one block ahead: the staging alone cost 28 % of the kernel's
// time at 8,192 tokens, the loads and the writes about equally.)
//
// A stage holds K as 32 rows of D / 8 units of 16 bytes, in the order the
// score product wants its rows (tile m, row i), and then V^T as D / 16 tiles of
// 64 units.  No padding: a lane can put any unit anywhere at no cost, so the units
// of K row r are rotated by r % 16 places, which spreads the 16 lanes that read one
// operand column of a tile (rows r..r+15, same channel) over the banks; the units
// of V^T lie in the order of the lanes that read them (tile dd: 1 KB, unit 16 q + i =
// keys 8 q.. of channel 16 dd + i).
typedef const __attribute__((address_space(4))) int* ConstInts;
constexpr int SHARED_WAVES = 4;
constexpr int KU = D / 8;                          // 16-byte units in a row of K
constexpr int STAGE_UNITS = 8 * D;                 // K: 32 rows x KU, then V^T: D rows x 4
constexpr int STAGE_BYTES = 16 * STAGE_UNITS;
constexpr int CHUNKS = STAGE_UNITS / 64;           // wavefront-wide loads a block: D / 8, half of them K
constexpr int LOADS = CHUNKS / SHARED_WAVES;       // ... per wavefront: D / 32
constexpr bool SHARED_FITS = 2 * STAGE_BYTES <= 65536;
struct Stage0 { static constexpr int value = 0; };
struct Stage1 { static constexpr int value = 1; };
struct Stage2 { static constexpr int value = 2; };

// One wavefront-wide load of 16 bytes a lane from `from` (any address per lane) to the 1 KB of
// LDS at byte `lds_at` (the same for all lanes): lane i's bytes land at lds_at + 16 i.  Written
// out as the instruction, with the compiler told nothing of what it writes: told, it waits for
// every such load before the next read of LDS that it cannot tell apart, which is all of them,
// and the loads would never be more than one block ahead.  The waits are explicit instead
// (wait_loads below; the loads complete in order).
__device__ __forceinline__ void load_to_lds(const void* from, unsigned lds_at) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(lds_at) : "m0");
}

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters left at their maxima)
template <int N> __device__ __forceinline__ void wait_loads() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// NB: column tiles of 16 a wavefront takes.  Two is the form for launches that fill the chip (a
// block read from LDS serves 32 columns); one makes twice the workgroups of half the registers,
// for launches too small to give every SIMD two wavefronts otherwise (a prompt of 2,048 tokens
// of the 7B shape: 224 workgroups of 128 columns for 256 CUs; MI355X: 88 us with two tiles a
// wavefront, 77 us with one).
template <bool FOLD, int NB>
__global__ __launch_bounds__(64 * SHARED_WAVES) __attribute__((amdgpu_waves_per_eu(D <= 128 ? (NB == 1 ? 3 : 2) : 1)))
void attention_mfma_shared_kernel(const AttnParams P) {
  constexpr int COLS = 16 * NB * SHARED_WAVES;
  // A stage of the ring holds SUB blocks of 32 keys, which a pass of the loop computes between
  // two barriers.  The wide form (two column tiles a wavefront) takes two blocks a pass where
  // two such stages fit the 64 KB (one barrier per 64 keys: 3-4 % at 4,096 tokens and beyond);
  // the narrow form one block a pass and three stages, which leaves LDS for three workgroups.
  constexpr int SUB = NB == 2 && 4 * STAGE_BYTES <= 65536 ? 2 : 1;
  constexpr int STAGES = SUB == 2 ? 2 : 3 * STAGE_BYTES <= 65536 ? 3 : 2;
  // one array per stage, so that the compiler can tell the loads into one from the reads of another
  __shared__ __attribute__((aligned(1024))) char ring0[SUB * STAGE_BYTES];
  __shared__ __attribute__((aligned(1024))) char ring1[SUB * STAGE_BYTES];
  __shared__ __attribute__((aligned(1024))) char ring2[STAGES == 3 ? SUB * STAGE_BYTES : 16];
  // (wave as a scalar: the products below sit under conditions that depend on it, and matrix
  // instructions ignore the execution mask)
  const int t = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(t >> 6), lane = t & 63, n = lane & 15, gq = lane >> 4;
  const Place at(P);
  if (!at.valid) return;                             // (the whole workgroup)
  const int seq = at.seq, kvh = at.kvh;
  const int g = P.nh / P.nkv;
  const int q0 = P.cu_q[seq];
  const int qlen = P.cu_q[seq + 1] - q0;
  const int ncols = qlen * g;
  const int ntiles = (ncols + COLS - 1) / COLS;
  const int pos0 = P.positions[q0];
  // (read through the constant address space: the same entries for all lanes, so they come by
  // scalar loads into scalar registers, and the addresses made from them cost no vector work)
  const ConstInts table = (ConstInts)(P.block_tables + (size_t)seq * P.max_pages);
  const int page = P.page, page_shift = 31 - __builtin_clz(page);

  // What a lane fetches is fixed for the whole kernel: unit u = 64 chunk + lane of a stage.
  // K unit (row r = 16 m + i, place s) holds channels 8 ((s - i) mod KU) of key
  // 8 (i / 4) + 4 m + i % 4; V^T unit 64 dd + 16 q + i holds keys 8 q .. 8 q + 7 of channel 16 dd + i: the place
  // of the lane that reads it as its operand of tile dd, so that a read takes 1 KB in the order of the lanes.
  int src[LOADS];                                    // offset inside the page's slice of this kv head, elements
  bool second[LOADS];                                // the unit lies in the second page of the block (16-key pages)
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int u = 64 * (wave + SHARED_WAVES * i) + lane;
    if (u < 32 * KU) {
      const int r = u / KU, c = (u % KU + KU - (r & 15) % KU) % KU;
      const int ko = 8 * ((r & 15) >> 2) + 4 * (r >> 4) + (r & 3);
      src[i] = (ko & (page - 1)) * D + 8 * c;
      second[i] = ko >= 16;
    } else {
      const int w = (u - 32 * KU) & 63, d = 16 * ((u - 32 * KU) >> 6) + (w & 15), q = w >> 4;
      src[i] = d * page + ((8 * q) & (page - 1));
      second[i] = q >= 2;
    }
  }
  const size_t per_page = (size_t)P.nkv * page * D, head_at = (size_t)kvh * page * D;   // elements
  // where this lane reads its operands in a stage: K row 16 m + n, channels 32 kk + 8 gq (the place
  // of unit 4 kk + gq rotated by the row); V^T row 16 dd + n, keys 8 gq
  int k_at[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) k_at[kk] = 16 * (n * KU + (4 * kk + gq + n) % KU);
  const int v_at = 16 * 32 * KU + 16 * lane;

  auto ring = [&](auto stage) -> char* {
    constexpr int S = decltype(stage)::value;
    return S == 0 ? ring0 : S == 1 ? ring1 : ring2;
  };
  // A pass of the loop computes SUB blocks of 32 keys out of one stage, with one barrier.  The
  // page ids of a pass are read (scalar loads) a pass before its blocks are asked for.
  int pg[SUB][2];
  auto load_pages = [&](int kb, int last) {
#pragma unroll
    for (int sub = 0; sub < SUB; ++sub) {
      const int kbase = (kb + sub < last ? kb + sub : last) * 32;
      pg[sub][0] = table[kbase >> page_shift];
      pg[sub][1] = table[(kbase + 16) >> page_shift];
    }
  };
  // ask for the blocks kb .. kb + SUB - 1 below `end` into a stage (their page ids are in pg)
  auto fetch = [&](int kb, int end, auto stage) {
#pragma unroll
    for (int sub = 0; sub < SUB; ++sub) {
      if (kb + sub >= end) break;                    // (the same for the whole workgroup)
      const int within = ((kb + sub) * 32) & (page - 1);   // where the block starts inside its page (64-key pages: 0 or 32)
      const __bf16* k0 = P.kc + ((size_t)pg[sub][0] * per_page + head_at + (size_t)within * D);
      const __bf16* k1 = P.kc + ((size_t)pg[sub][1] * per_page + head_at + (size_t)within * D);
      const __bf16* v0 = P.vc + ((size_t)pg[sub][0] * per_page + head_at + within);
      const __bf16* v1 = P.vc + ((size_t)pg[sub][1] * per_page + head_at + within);
      const unsigned base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)ring(stage) + STAGE_BYTES * sub;
#pragma unroll
      for (int i = 0; i < LOADS; ++i) {
        const int chunk = wave + SHARED_WAVES * i;
        const bool keys = chunk < CHUNKS / 2;          // the same for the whole wavefront
        const __bf16* from = (second[i] ? (keys ? k1 : v1) : (keys ? k0 : v0)) + src[i];
        load_to_lds(from, base + 1024 * chunk);
      }
    }
  };

  // A workgroup takes a late tile (many key blocks) and then the early tile
  // that mirrors it (few): every workgroup of a sequence then has about the
  // same number of blocks and none is left running alone at the end (MI355X,
  // 7B shape: 2,048 tokens 108 -> 80 us, 8,192 tokens 807 -> 737 us).  A
  // portion deep inside a long context has tiles of nearly one length already;
  // its caller leaves them unpaired, which makes twice the workgroups.
  // Unpaired tiles of a long context may also be cut into P.nsplit shares of
  // their key blocks, a workgroup each, whose partial results the combine
  // kernel merges: more and shorter workgroups for a launch of few tiles.
  const int tile_rev = P.pair ? at.x : at.x / P.nsplit;
  const int split = P.pair ? 0 : at.x % P.nsplit;
  for (int half = 0; half < 2; ++half) {
  if (P.pair ? 2 * tile_rev + half > ntiles - 1 : half > 0 || tile_rev >= ntiles)
    break;                                                  // no such tile; the whole workgroup leaves together
  const int tile = half == 0 ? ntiles - 1 - tile_rev : tile_rev;

  const int wg_c0 = tile * COLS;
  const int c0 = wg_c0 + 16 * NB * wave;
  const bool active = c0 < ncols;                  // a wavefront past the last column only helps loading
  Columns<NB, FOLD> C;
  C.init(P, q0, ncols, active ? c0 : wg_c0, pos0, kvh, g, n, gq);

  // key blocks of the workgroup: from the first block its first wavefront
  // needs to the last block its last active wavefront needs
  const int wg_tok_first = wg_c0 / g;
  const int wg_c_last = wg_c0 + COLS - 1 < ncols - 1 ? wg_c0 + COLS - 1 : ncols - 1;
  int kmin = 0;
  if (P.window > 0 && pos0 + wg_tok_first - P.window + 1 > 0) kmin = pos0 + wg_tok_first - P.window + 1;
  int wg_begin = kmin / 32, wg_end = (pos0 + wg_c_last / g) / 32 + 1;
  if (P.nsplit > 1) {
    const int nblk = wg_end - wg_begin, first = wg_begin;
    wg_begin = first + (int)((long long)nblk * split / P.nsplit);
    wg_end = first + (int)((long long)nblk * (split + 1) / P.nsplit);
  }
  const int last = wg_end - 1;

  // one pass: ask for the pass STAGES - 1 ahead (into the stage that the last pass was read from;
  // the barrier that ended that pass has been passed), compute this pass's blocks out of `here`,
  // then make sure that this wavefront's loads of the next pass have landed and meet the others
  auto step = [&](int kb, auto here, auto ahead) {
    const int next = kb + (STAGES - 1) * SUB;
    const bool more = next < wg_end;
    if (more) {
      fetch(next, wg_end, ahead);
      load_pages(next + SUB, last);
    }
    const char* at = ring(here);
#pragma unroll
    for (int sub = 0; sub < SUB; ++sub) {
      const int k = kb + sub;
      if (active && k < wg_end && k >= C.kb_begin && k < C.kb_end) {
        const char* from = at + STAGE_BYTES * sub;
        bf16x8 kf[2][KK], vf[DD];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int kk = 0; kk < KK; ++kk) kf[m][kk] = *(const bf16x8*)(from + 256 * KU * m + k_at[kk]);
#pragma unroll
        for (int dd = 0; dd < DD; ++dd) vf[dd] = *(const bf16x8*)(from + v_at + 1024 * dd);
        C.block_abreast(k, kf, vf, gq);
      }
    }
    if (more && STAGES == 3) wait_loads<LOADS * SUB>();    // all but the pass just asked for
    else wait_loads<0>();
    // (the bare barrier: __syncthreads() would first wait for every load on its way, the pass
    // just asked for included; what must be complete here is this wavefront's share of the next
    // pass, waited for above, and its reads of this pass, whose values the products have used)
    __builtin_amdgcn_s_barrier();
    asm volatile("" : : : "memory");               // (the compiler reads LDS again from here on, whatever it held)
  };

  if (wg_begin < wg_end) {                           // (a share may be empty; the same for the whole workgroup)
    load_pages(wg_begin, last);
    fetch(wg_begin, wg_end, Stage0{});
    load_pages(wg_begin + SUB, last);
    if (STAGES == 3) {
      if (wg_begin + SUB < wg_end) fetch(wg_begin + SUB, wg_end, Stage1{});
      load_pages(wg_begin + 2 * SUB, last);
      if (wg_begin + SUB < wg_end) wait_loads<LOADS * SUB>();
      else wait_loads<0>();
    } else {
      wait_loads<0>();
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" : : : "memory");
  }
  if (STAGES == 3) {
    for (int kb = wg_begin; kb < wg_end; kb += 3 * SUB) {
      step(kb, Stage0{}, Stage2{});
      if (kb + SUB < wg_end) step(kb + SUB, Stage1{}, Stage0{});
      if (kb + 2 * SUB < wg_end) step(kb + 2 * SUB, Stage2{}, Stage1{});
    }
  } else {
    for (int kb = wg_begin; kb < wg_end; kb += 2 * SUB) {
      step(kb, Stage0{}, Stage1{});
      if (kb + SUB < wg_end) step(kb + SUB, Stage1{}, Stage0{});
    }
  }
  if (active) {
    if (P.nsplit > 1) C.template store<true>(P, q0, split, gq);
    else C.template store<false>(P, q0, 0, gq);
  }
  }
}

// out[row, head, :] = sum_j w_j o_j / sum_j w_j l_j,  w_j = exp(m_j - max m).
// One wavefront per (row, head); lane j takes the (m, l) of splits j, j + 64, ..., so
// nsplit <= 64 * COMBINE_PER_LANE; then the lanes split the channels and sum the partial
// outputs, share after share.  SKIP: shares of weight 0 wrote no
// output, and what lies in their place may be anything (a kernel of its own: the test costs the
// plain one 1.9 of its 5.4 us for one request of the 7B shape in 16 shares).
constexpr int COMBINE_PER_LANE = 4;
template <bool SKIP>
__global__ __launch_bounds__(64) void attention_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int nsplit, int nh,
    int part_row0, __bf16* __restrict__ out, int out_rows) {
  __shared__ float ws[64 * COMBINE_PER_LANE];
  const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t base = ((size_t)r * nh + h) * nsplit;
  float m[COMBINE_PER_LANE], l[COMBINE_PER_LANE], top = -INFINITY;
#pragma unroll
  for (int i = 0; i < COMBINE_PER_LANE; ++i) {
    const int j = lane + 64 * i;
    m[i] = -INFINITY;
    l[i] = 0.f;
    if (j < nsplit) {
      m[i] = part_ml[(base + j) * 2];
      l[i] = part_ml[(base + j) * 2 + 1];
    }
    top = fmaxf(top, m[i]);
  }
  const float mx = wave_max(top);
  float mine = 0.f;
#pragma unroll
  for (int i = 0; i < COMBINE_PER_LANE; ++i) {
    const float w = m[i] == -INFINITY ? 0.f : fast_exp2(m[i] - mx);     // maxima are in units of log 2
    mine += w * l[i];
    ws[lane + 64 * i] = w;
  }
  const float denom = wave_sum(mine);
  __syncthreads();
  const float inv = 1.f / denom;
  const float* po = part_o + base * D;
  // A lane takes channels lane, lane + 64, ...; the partial outputs of sixteen shares are asked for
  // together, all channels of a lane at once (a batch is a trip to memory: with eight shares a batch
  // and the channels one after the other, 64 shares took 2 us longer than 32; with the last shares
  // below a whole batch one by one, 21 took 3 us longer than 16 or 24).  Added in the order of the
  // shares, whatever the batches.
  constexpr int DI = (D + 63) / 64, BATCH = 16;
  float acc[DI];
#pragma unroll
  for (int di = 0; di < DI; ++di) acc[di] = 0.f;
  for (int j = 0; j < nsplit; j += BATCH) {
    float v[BATCH][DI];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const float* row = po + (size_t)(j + u < nsplit ? j + u : nsplit - 1) * D;
#pragma unroll
      for (int di = 0; di < DI; ++di) v[u][di] = 64 * di + 64 <= D || lane + 64 * di < D ? row[lane + 64 * di] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      // (no branch here: under one the compiler may move each load down to its use; beyond the last share the
      // weight is 0 and the value that of the last share)
      const float w = j + u < nsplit ? ws[j + u] : 0.f;
#pragma unroll
      for (int di = 0; di < DI; ++di) acc[di] += SKIP && w == 0.f ? 0.f : w * v[u][di];
    }
  }
#pragma unroll
  for (int di = 0; di < DI; ++di) {
    const int d = lane + 64 * di;
    if (d < D) out[out_index(out_rows, nh, (size_t)(part_row0 + r), h * D + d)] = (__bf16)(acc[di] * inv);
  }
}

extern "C" int sl_attention_mfma_max_splits() { return 64 * COMBINE_PER_LANE; }
extern "C" int sl_attention_mfma_head_dim() { return D; }
// whether this head size has the prompt kernel that shares keys through LDS (its buffers fit)
extern "C" int sl_attention_mfma_shares_keys() { return SHARED_FITS ? 1 : 0; }
// the most query heads per kv head that the single-token workgroups which merge in LDS take
extern "C" int sl_attention_mfma_group_heads() { return 16 * GROUP_MAX_NB; }
// whether the workgroups that share keys through LDS are laid out by chiplet for this many kv heads (see Place)
extern "C" int sl_attention_mfma_by_chiplet(int nkv) { return nkv > 0 && (nkv < 8 ? 8 % nkv == 0 : nkv % 8 == 0) ? 1 : 0; }

// One launch over sequences [seq_begin, seq_begin + num_seqs), all with at
// most max_q_len tokens.  nsplit > 1 needs part_o / part_ml for the rows
// [part_row0, part_row0 + part_rows) these sequences own (one token each).
// group (single tokens, nsplit 1): the workgroups of eight wavefronts that merge in LDS.
// Prompt portions go to the workgroups that share keys through LDS once the
// launch would have shared_min_waves wavefronts of 32 columns or more;
// pair_tiles: see the kernel; narrow_below: with fewer workgroups of 128
// columns than this, workgroups of 64 columns are launched instead.
extern "C" const char* sl_attention_mfma(
    const void* qkv, int row_stride, const void* kc, const void* vc, const int* block_tables,
    int max_pages, const int* cu_q, const int* positions, int seq_begin, int num_seqs,
    int max_q_len, int nh, int nkv, int head_dim, int page, float scale, int window, int nsplit,
    int shared_min_waves, int pair_tiles, void* out, float* part_o, float* part_ml, int part_row0, int part_rows,
    int narrow_below, int out_rows, int group, const int* ctx_stats, int share_waves, hipStream_t stream) {
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
               (__bf16*)out, part_o, part_ml, part_row0, pair_tiles, out_rows, 0, 0, num_seqs, nullptr, 0};
  SL_CHECK(out_rows >= 0 && (out_rows == 0 || (max_q_len == 1 && seq_begin == 0 && out_rows == num_seqs)),
           "attention_mfma: a result laid out by k-step is that of a step of single tokens, all of its rows");
  const long long cols = (long long)max_q_len * g;
  // scale * log2(e) == 1: the caller's q is already in units of log 2 (see Columns)
  const bool fold = fabsf(scale * 1.4426950408889634f - 1.f) < 1e-6f;
  if (group) {
    // single tokens, a workgroup per (sequence, kv head) whose wavefronts merge in LDS
    SL_CHECK(max_q_len == 1 && nsplit == 1, "attention_mfma: the workgroups that merge in LDS take single tokens, unsplit");
    SL_CHECK(g <= 16 * GROUP_MAX_NB, "attention_mfma: too many query heads per kv head for the workgroups that merge in LDS");
    const dim3 grid(nkv, num_seqs);
    if (g <= 16) {
      if (fold) attention_mfma_group_kernel<1, true><<<grid, 64 * GROUP_WAVES, 0, stream>>>(P);
      else attention_mfma_group_kernel<1, false><<<grid, 64 * GROUP_WAVES, 0, stream>>>(P);
    } else {
      if (fold) attention_mfma_group_kernel<GROUP_MAX_NB, true><<<grid, 64 * GROUP_WAVES, 0, stream>>>(P);
      else attention_mfma_group_kernel<GROUP_MAX_NB, false><<<grid, 64 * GROUP_WAVES, 0, stream>>>(P);
    }
    return sl_launch_status();
  }
  if (nsplit > 1 && max_q_len == 1) {
    SL_CHECK(part_o != nullptr && part_ml != nullptr && part_rows == num_seqs,
             "attention_mfma: a split launch needs partial buffers for its rows");
    SL_CHECK(g <= 64, "attention_mfma: more than 64 query heads per kv head");
    SL_CHECK(nsplit <= 64 * COMBINE_PER_LANE, "attention_mfma: too many splits of the context");
    SL_CHECK(num_seqs <= 65535 && nsplit <= 65535, "attention_mfma: too many sequences in a split launch");
    const dim3 grid(nkv, num_seqs, nsplit);
    const bool one_length = ctx_stats != nullptr && share_waves > 0;
    P.ctx_stats = ctx_stats;
    P.share_waves = share_waves;
#define SL_SPLIT(NB_, FOLD_, PAIRS_)                                                                  \
  do {                                                                                                \
    if (one_length) attention_mfma_kernel<NB_, true, FOLD_, PAIRS_, true><<<grid, 64, 0, stream>>>(P); \
    else attention_mfma_kernel<NB_, true, FOLD_, PAIRS_, false><<<grid, 64, 0, stream>>>(P);           \
  } while (0)
    if (fold) {
      if (g <= 16) SL_SPLIT(1, true, true);
      else if (g <= 32) SL_SPLIT(2, true, false);
      else SL_SPLIT(4, true, false);
    } else {
      if (g <= 16) SL_SPLIT(1, false, false);
      else if (g <= 32) SL_SPLIT(2, false, false);
      else SL_SPLIT(4, false, false);
    }
#undef SL_SPLIT
    const char* e = sl_launch_status();
    if (e) return e;
    if (one_length) attention_combine_kernel<true><<<dim3(num_seqs, nh), 64, 0, stream>>>(
        part_o, part_ml, nsplit, nh, part_row0, (__bf16*)out, out_rows);
    else attention_combine_kernel<false><<<dim3(num_seqs, nh), 64, 0, stream>>>(
        part_o, part_ml, nsplit, nh, part_row0, (__bf16*)out, out_rows);
    return sl_launch_status();
  }
  // Prompt portions.  The workgroups that share a block through LDS, or one
  // wavefront per 32 columns, each reading its keys straight from the pages;
  // the caller sets the crossover.  (MI355X, 7B shape: with the launch laid out
  // by chiplet and a workgroup per tile the LDS form is as fast or faster at
  // every size measured: one prompt of 128 / 512 / 1,024 / 2,048 tokens 11.8 /
  // 19.1 / 31.8 / 57.5 us against 14.9 / 20.2 / 42.0 / 97 us; eight prompts of
  // 512: 46 against 99 us; 512 tokens after 7,680: 108 against 278 us.)
  const long long tiles = (cols + 31) / 32;
  SL_CHECK(tiles <= 1 << 30, "attention_mfma: too many column tiles");
  // (single tokens of at most 16 heads a kv head, unsplit: one wavefront each, as before)
  const bool shared = SHARED_FITS && (max_q_len > 1 || cols > 16) && tiles * nkv * num_seqs >= shared_min_waves;
  if (nsplit > 1) {
    SL_CHECK(shared && !pair_tiles, "attention_mfma: prompt portions are split only as unpaired tiles through LDS");
    SL_CHECK(nsplit <= 64 * COMBINE_PER_LANE && part_o != nullptr && part_ml != nullptr && part_rows > 0,
             "attention_mfma: a split launch needs partial buffers for its rows and not too many splits");
  }
  if (!shared && cols <= 16) {
    if (fold) attention_mfma_kernel<1, false, true><<<dim3(1, nkv, num_seqs), 64, 0, stream>>>(P);
    else attention_mfma_kernel<1, false, false><<<dim3(1, nkv, num_seqs), 64, 0, stream>>>(P);
  } else if (!shared) {
    const dim3 grid((unsigned)tiles, nkv, num_seqs);
    if (fold) attention_mfma_kernel<2, false, true><<<grid, 64, 0, stream>>>(P);
    else attention_mfma_kernel<2, false, false><<<grid, 64, 0, stream>>>(P);
  } else {
    // workgroups of 128 columns, or of 64 when those would leave SIMDs with one wavefront
    long long wg = (cols + 32 * SHARED_WAVES - 1) / (32 * SHARED_WAVES);
    const long long wide = (pair_tiles ? (wg + 1) / 2 : wg) * nkv * num_seqs;
    const bool narrow = nsplit == 1 && wide < narrow_below;
    if (narrow) wg = (cols + 16 * SHARED_WAVES - 1) / (16 * SHARED_WAVES);
    dim3 grid((unsigned)(pair_tiles ? (wg + 1) / 2 : wg * nsplit), nkv, num_seqs);
    if (sl_attention_mfma_by_chiplet(nkv)) {                     // (else the grid stays laid out pair by pair)
      P.by_chiplet = 1;
      P.grid_x = (int)grid.x;
      P.num_seqs = num_seqs;
      const long long each = nkv < 8 ? (long long)((grid.x + 8 / nkv - 1) / (8 / nkv)) * num_seqs
                                     : (long long)grid.x * num_seqs * (nkv / 8);
      SL_CHECK(8 * each < (1ll << 31), "attention_mfma: grid too large");
      grid = dim3((unsigned)(8 * each), 1, 1);
    }
    if (narrow) {
      if (fold) attention_mfma_shared_kernel<true, 1><<<grid, 64 * SHARED_WAVES, 0, stream>>>(P);
      else attention_mfma_shared_kernel<false, 1><<<grid, 64 * SHARED_WAVES, 0, stream>>>(P);
    } else {
      if (fold) attention_mfma_shared_kernel<true, 2><<<grid, 64 * SHARED_WAVES, 0, stream>>>(P);
      else attention_mfma_shared_kernel<false, 2><<<grid, 64 * SHARED_WAVES, 0, stream>>>(P);
    }
    if (nsplit > 1) {
      const char* e = sl_launch_status();
      if (e) return e;
      attention_combine_kernel<false><<<dim3(part_rows, nh), 64, 0, stream>>>(part_o, part_ml, nsplit, nh,
                                                                    part_row0, (__bf16*)out, out_rows);
    }
  }
  return sl_launch_status();
}
