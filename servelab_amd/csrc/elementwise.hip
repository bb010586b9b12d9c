// Embedding gather, SiLU-multiply, rotary tables, and rotary + cache write.
#include "common.h"

// ---------------------------------------------------------------- embedding
// out[t, :] = float(table[ids[t], :]).  Replaces the embedding lookup of
// servelab/parallel/tp_model.py:123; the residual stream it starts is float.
__global__ void embed_kernel(const int* __restrict__ ids, const act_t* __restrict__ table,
                             float* __restrict__ out, int H, int V) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);     // the host rejects such ids; never fault
  const act_t* row = table + (size_t)id * H;
  float* o = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f(row[i]);
}

extern "C" const char* sl_embed(const int* ids, const void* table, float* out, int T, int H,
                                int V, hipStream_t stream) {
  SL_CHECK(T >= 0 && H > 0 && V > 0, "embed: sizes must be positive");
  if (T == 0) return nullptr;
  embed_kernel<<<T, 256, 0, stream>>>(ids, (const act_t*)table, out, H, V);
  return sl_launch_status();
}

// ------------------------------------------------------------- silu * up
// out[t, i] = silu(gate[t, i]) * up[t, i], silu(z) = z * sigmoid(z)
// (servelab/parallel/tp_model.py:68), float inside.  A row of gate_up holds
// gate and up interleaved in blocks: gate i sits at 2 * block * (i / block) +
// i % block and up i one block further; block = I is plain [gate | up].
__global__ void silu_mul_kernel(const act_t* __restrict__ gate_up, act_t* __restrict__ out,
                                int I, int block, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / I;
    const int i = (int)(idx - t * I);
    const size_t at = t * 2 * I + (size_t)2 * block * (i / block) + i % block;
    const float g = to_f(gate_up[at]);
    const float u = to_f(gate_up[at + block]);
    out[idx] = from_f<act_t>(g / (1.f + expf(-g)) * u);
  }
}

// The same for blocks of 8 (gate and up rows interleaved as the few-rows GEMM
// wants them): a thread reads 8 gates and their 8 ups as two 16-byte vectors.
struct __attribute__((aligned(16))) act8 { act_t v[8]; };
#if defined(SL_F32)
struct __attribute__((aligned(16))) act8_half { act_t v[4]; };
#endif

__global__ void silu_mul_block8_kernel(const act_t* __restrict__ gate_up, act_t* __restrict__ out,
                                       size_t groups) {
  for (size_t gidx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gidx < groups;
       gidx += (size_t)gridDim.x * blockDim.x) {
    const act_t* src = gate_up + gidx * 16;
    act_t* dst = out + gidx * 8;
#if defined(SL_F32)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const act8_half g = *(const act8_half*)(src + 4 * h), u = *(const act8_half*)(src + 8 + 4 * h);
      act8_half o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o.v[j] = g.v[j] / (1.f + expf(-g.v[j])) * u.v[j];
      *(act8_half*)(dst + 4 * h) = o;
    }
#else
    const act8 g = *(const act8*)src, u = *(const act8*)(src + 8);
    act8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float gf = to_f(g.v[j]);
      o.v[j] = from_f<act_t>(gf / (1.f + __expf(-gf)) * to_f(u.v[j]));
    }
    *(act8*)dst = o;
#endif
  }
}

extern "C" const char* sl_silu_mul(const void* gate_up, void* out, int T, int I, int block,
                                   hipStream_t stream) {
  SL_CHECK(T >= 0 && I > 0, "silu_mul: sizes must be positive");
  SL_CHECK(block > 0 && I % block == 0, "silu_mul: the block must divide the width");
  if (T == 0) return nullptr;
  const size_t total = (size_t)T * I;
  if (block == 8 && ((uintptr_t)gate_up % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    const size_t groups = total / 8;
    const size_t blocks = (groups + 255) / 256;
    silu_mul_block8_kernel<<<(unsigned)(blocks < 262144 ? blocks : 262144), 256, 0, stream>>>(
        (const act_t*)gate_up, (act_t*)out, groups);
    return sl_launch_status();
  }
  const int blocks = (int)((total + 255) / 256 < 65535 * 4 ? (total + 255) / 256 : 65535 * 4);
  silu_mul_kernel<<<blocks, 256, 0, stream>>>((const act_t*)gate_up, (act_t*)out, I, block, total);
  return sl_launch_status();
}

// ------------------------------------------------------------ rotary tables
// cos/sin[t, j] of angle float(pos[t]) * inv_freq[j], float32 with the
// accurate cosf/sinf.  Once per step; every layer reads the same table.
__global__ void rope_tables_kernel(const int* __restrict__ pos, const float* __restrict__ inv_freq,
                                   float* __restrict__ cosv, float* __restrict__ sinv,
                                   int half, int total) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int t = idx / half, j = idx - t * half;
  const float ang = (float)pos[t] * inv_freq[j];
  cosv[idx] = cosf(ang);
  sinv[idx] = sinf(ang);
}

extern "C" const char* sl_rope_tables(const int* pos, const float* inv_freq, float* cosv,
                                      float* sinv, int T, int half, hipStream_t stream) {
  SL_CHECK(T >= 0 && half > 0, "rope_tables: sizes must be positive");
  if (T == 0) return nullptr;
  const int total = T * half;
  rope_tables_kernel<<<(total + 255) / 256, 256, 0, stream>>>(pos, inv_freq, cosv, sinv, half,
                                                              total);
  return sl_launch_status();
}

// ------------------------------------------------- rotary + write to pages
// qkv rows are [q heads | k heads | v heads], head-major.  The first `rot`
// channels of every q and k head are rotated in place with pairs (j, j + rot/2)
// (rot = D: servelab/parallel/tp_model.py:128; tables [T, rot/2]); the
// rotated k and the v of each token go to its cache row (:129,
// servelab/kv_cache/pool.py:68-78): K pages [page, nkv, page_size, D], V pages
// [page, nkv, D, page_size].  One block per (token, head).
//
// pairs8: the channels of every q and k head come in the order the fused
// few-rows product wants them (gemm.hip): the rotated channels in blocks of 16
// that hold channels 8b..8b+7 followed by their partners rot/2+8b..rot/2+8b+7,
// so that pair j sits at 16 (j / 8) + j % 8 and 8 further; then the rest.  Scores do not depend on the order of the
// channels as long as q and the cached k agree; v keeps its order.
// The float partial sums of a q/k/v product whose K was split over workgroups
// ([nparts][T][N], bias not yet added): the kernel below then reads its input
// from them instead of from qkv, which saves the product a kernel that only
// adds them up.
struct SplitProduct {
  const float* parts;            // or nullptr: the input is qkv itself
  int nparts;
  size_t stride;                 // T * N
  const float* bias;             // [N] or nullptr
};

__global__ void rope_store_kernel(act_t* __restrict__ qkv, const SplitProduct sp,
                                  const float* __restrict__ cosv,
                                  const float* __restrict__ sinv, const int* __restrict__ slots,
                                  act_t* __restrict__ kc, act_t* __restrict__ vc, int nh, int nkv,
                                  int D, int rot, int page, int pairs8, float qscale) {
  const int t = blockIdx.x, hd = blockIdx.y;
  const float qs = hd < nh ? qscale : 1.f;         // q heads leave multiplied by qscale
  const int half = rot / 2;
  const size_t row = ((size_t)t * (nh + 2 * nkv) + hd) * D;
  act_t* x = qkv + row;
  auto input = [&](int c) {
    if (sp.parts == nullptr) return to_f(x[c]);
    float v = sp.bias != nullptr ? sp.bias[hd * D + c] : 0.f;
    for (int j = 0; j < sp.nparts; ++j) v += sp.parts[j * sp.stride + row + c];
    return v;
  };
  if (hd < nh + nkv) {
    act_t* dst = nullptr;
    if (hd >= nh && kc != nullptr) {
      const int slot = slots[t];
      dst = kc + (((size_t)(slot / page) * nkv + (hd - nh)) * page + slot % page) * D;
    }
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
      const int p1 = pairs8 ? 16 * (j / 8) + j % 8 : j;
      const int p2 = pairs8 ? p1 + 8 : j + half;
      float x1 = input(p1), x2 = input(p2);
      if (cosv != nullptr) {
        const float c = cosv[(size_t)t * half + j], s = sinv[(size_t)t * half + j];
        const float r1 = x1 * c - x2 * s, r2 = x2 * c + x1 * s;
        x1 = r1;
        x2 = r2;
      }
      x1 *= qs;
      x2 *= qs;
      // in place: whatever changed; from partial sums: q (k lives on in the pages only)
      if (sp.parts != nullptr ? hd < nh : (cosv != nullptr || qs != 1.f)) {
        x[p1] = from_f<act_t>(x1);
        x[p2] = from_f<act_t>(x2);
      }
      if (dst != nullptr) {
        dst[p1] = from_f<act_t>(x1);
        dst[p2] = from_f<act_t>(x2);
      }
    }
    for (int c = rot + threadIdx.x; c < D; c += blockDim.x) {       // channels beyond the rotated ones pass
      const float v = input(c) * qs;
      if (hd < nh && (sp.parts != nullptr || qs != 1.f)) x[c] = from_f<act_t>(v);
      if (dst != nullptr) dst[c] = from_f<act_t>(v);
    }
  } else if (vc != nullptr) {
    const int slot = slots[t];
    act_t* dst = vc + ((size_t)(slot / page) * nkv + (hd - nh - nkv)) * D * page + slot % page;
    for (int d = threadIdx.x; d < D; d += blockDim.x) dst[(size_t)d * page] = from_f<act_t>(input(d));
  }
}

// The same work with 16-byte accesses, for head sizes that are multiples of 16
// (many-token steps: the per-pair kernel above needs one block of 64 threads
// per token and head and moves 2 bytes per access).  With few tokens, or with
// several partial sums to add, the per-pair kernel's many threads win (7B
// shape, graph-timed: 64 tokens 5.2 against 3.3 us, 256: 5.7 against 5.2, 512:
// 6.5 against 7.9, 2,048: 13.0 against 22.8; 512 tokens in 4 partial sums: 16.3
// against 12.8).
constexpr int VECTOR_MIN_TOKENS = 384;
struct __attribute__((aligned(16))) Act8 { act_t v[8]; };
struct __attribute__((aligned(16))) F4 { float v[4]; };

// q and k heads: a thread rotates 8 pairs (two 8-channel runs) of one head of
// one token and writes them back, k also to its cache row.  From partial sums
// (sp.parts): the 16 inputs are bias + the sums, q is written to qkv and k only
// to its cache row, as in the kernel above.
__device__ __forceinline__ void rope_store_qk_block(
    int t, int by, int gy, act_t* __restrict__ qkv, const SplitProduct& sp, const float* __restrict__ cosv,
    const float* __restrict__ sinv, const int* __restrict__ slots, act_t* __restrict__ kc, int nh,
    int nkv, int D, int rot, int page, int pairs8, float qscale) {
  const int half = rot / 2, chunks = D / 16, rotated = rot / 16;
  const int items = (nh + nkv) * chunks;
  for (int w = by * blockDim.x + threadIdx.x; w < items; w += gy * blockDim.x) {
    const int hd = w / chunks, c = w % chunks;
    // chunks below `rotated` hold 8 pairs; the others 16 channels that pass unrotated
    const bool turn = c < rotated;
    const int p1 = !turn || pairs8 ? 16 * c : 8 * c, p2 = !turn || pairs8 ? p1 + 8 : p1 + half;
    const size_t row = ((size_t)t * (nh + 2 * nkv) + hd) * D;
    act_t* x = qkv + row;
    float xa[8], xb[8];
    if (sp.parts == nullptr) {
      const Act8 a = *(const Act8*)(x + p1), b = *(const Act8*)(x + p2);
#pragma unroll
      for (int j = 0; j < 8; ++j) xa[j] = to_f(a.v[j]), xb[j] = to_f(b.v[j]);
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        F4 va{{0.f, 0.f, 0.f, 0.f}}, vb = va;
        if (sp.bias != nullptr) {
          va = *(const F4*)(sp.bias + hd * D + p1 + 4 * h);
          vb = *(const F4*)(sp.bias + hd * D + p2 + 4 * h);
        }
        for (int j = 0; j < sp.nparts; ++j) {
          const F4 pa = *(const F4*)(sp.parts + j * sp.stride + row + p1 + 4 * h);
          const F4 pb = *(const F4*)(sp.parts + j * sp.stride + row + p2 + 4 * h);
#pragma unroll
          for (int i = 0; i < 4; ++i) va.v[i] += pa.v[i], vb.v[i] += pb.v[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) xa[4 * h + i] = va.v[i], xb[4 * h + i] = vb.v[i];
      }
    }
    const float qs = hd < nh ? qscale : 1.f;
    const bool changed = (cosv != nullptr && turn) || qs != 1.f;
    if (changed) {
      F4 c0{{1.f, 1.f, 1.f, 1.f}}, c1 = c0, s0{{0.f, 0.f, 0.f, 0.f}}, s1 = s0;
      if (cosv != nullptr && turn) {
        const float* cp = cosv + (size_t)t * half + 8 * c;
        const float* sn = sinv + (size_t)t * half + 8 * c;
        c0 = *(const F4*)cp, c1 = *(const F4*)(cp + 4);
        s0 = *(const F4*)sn, s1 = *(const F4*)(sn + 4);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float cs = j < 4 ? c0.v[j] : c1.v[j - 4], sn = j < 4 ? s0.v[j] : s1.v[j - 4];
        const float x1 = xa[j], x2 = xb[j];
        xa[j] = (x1 * cs - x2 * sn) * qs;
        xb[j] = (x2 * cs + x1 * sn) * qs;
      }
    }
    Act8 a, b;
#pragma unroll
    for (int j = 0; j < 8; ++j) a.v[j] = from_f<act_t>(xa[j]), b.v[j] = from_f<act_t>(xb[j]);
    if (sp.parts != nullptr ? hd < nh : changed) {
      *(Act8*)(x + p1) = a;
      *(Act8*)(x + p2) = b;
    }
    if (hd >= nh && kc != nullptr) {
      const int slot = slots[t];
      act_t* dst = kc + (((size_t)(slot / page) * nkv + (hd - nh)) * page + slot % page) * D;
      *(Act8*)(dst + p1) = a;
      *(Act8*)(dst + p2) = b;
    }
  }
}

// v heads: a block takes 16 consecutive tokens of one kv head through LDS, so
// that neighbouring lanes write neighbouring slots of a channel's row (tokens
// of one request usually sit in consecutive slots of a page).
__device__ __forceinline__ void store_v_block(
    int t0, int kvh, const act_t* __restrict__ qkv, const SplitProduct& sp, const int* __restrict__ slots,
    act_t* __restrict__ vc, int T, int nh, int nkv, int D, int page) {
  __shared__ act_t tile[16][256 + 2];
  __shared__ int slot_of[16];
  const int nt = T - t0 < 16 ? T - t0 : 16;
  if (threadIdx.x < 16) slot_of[threadIdx.x] = threadIdx.x < nt ? slots[t0 + threadIdx.x] : 0;
  for (int idx = threadIdx.x; idx < nt * D; idx += blockDim.x) {
    const int i = idx / D, d = idx % D;
    const size_t at = ((size_t)(t0 + i) * (nh + 2 * nkv) + nh + nkv + kvh) * D + d;
    if (sp.parts == nullptr) {
      tile[i][d] = qkv[at];
    } else {
      float v = sp.bias != nullptr ? sp.bias[(nh + nkv + kvh) * D + d] : 0.f;
      for (int j = 0; j < sp.nparts; ++j) v += sp.parts[j * sp.stride + at];
      tile[i][d] = from_f<act_t>(v);
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < 16 * D; idx += blockDim.x) {
    const int i = idx % 16, d = idx / 16;
    if (i < nt) {
      const int slot = slot_of[i];
      vc[(((size_t)(slot / page) * nkv + kvh) * D + d) * page + slot % page] = tile[i][d];
    }
  }
}

// One launch for both: the first v_blocks workgroups take the v heads (16 tokens of one kv head
// each), the others the q and k heads (gy workgroups a token).  The two halves read and write
// different heads, so they run side by side instead of one launch after the other (2,048 tokens
// of the 7B shape: 14 + 7 us in two launches).
__global__ __launch_bounds__(256) void rope_store_vec_kernel(
    act_t* __restrict__ qkv, const SplitProduct sp, const float* __restrict__ cosv,
    const float* __restrict__ sinv, const int* __restrict__ slots, act_t* __restrict__ kc,
    act_t* __restrict__ vc, int T, int nh, int nkv, int D, int rot, int page, int pairs8, float qscale,
    int v_blocks, int gy) {
  const int b = blockIdx.x;
  if (b < v_blocks) {                                // (the same for the whole workgroup)
    const int groups = (T + 15) / 16;
    store_v_block(b % groups * 16, b / groups, qkv, sp, slots, vc, T, nh, nkv, D, page);
  } else {
    rope_store_qk_block((b - v_blocks) / gy, (b - v_blocks) % gy, gy, qkv, sp, cosv, sinv, slots, kc, nh, nkv, D, rot,
                        page, pairs8, qscale);
  }
}

// parts != nullptr: the input is the sum of nparts float partial products
// [nparts][T][N] plus bias; q is then written to qkv, k and v only to the pages.
// qscale: q heads are multiplied by it after the rotation and before their one
// rounding (an attention kernel that wants its scores in units of log 2 asks
// for scale * log2(e) here and then needs no multiply per score).
extern "C" const char* sl_rope_store(void* qkv, const float* cosv, const float* sinv,
                                     const int* slots, void* kc, void* vc, int T, int nh, int nkv,
                                     int D, int rot, int page, int pairs8, const float* parts,
                                     int nparts, const float* bias, float qscale, hipStream_t stream) {
  SL_CHECK(T >= 0 && nh > 0 && nkv > 0, "rope_store: sizes must be positive");
  SL_CHECK(D > 0 && rot >= 0 && rot <= D && rot % 2 == 0,
           "rope_store: the rotated width must be even and at most head_dim");
  SL_CHECK(cosv == nullptr || rot > 0, "rope_store: tables given but no channel is rotated");
  SL_CHECK(!pairs8 || rot % 16 == 0, "rope_store: the blocked pair order needs a rotated width % 16 == 0");
  SL_CHECK((cosv == nullptr) == (sinv == nullptr), "rope_store: cos and sin go together");
  SL_CHECK((kc == nullptr) == (vc == nullptr), "rope_store: k and v pages go together");
  SL_CHECK(kc == nullptr || (slots != nullptr && page > 0), "rope_store: pages need slots");
  SL_CHECK(parts == nullptr || nparts >= 1, "rope_store: partial products need their count");
  SL_CHECK(parts != nullptr || bias == nullptr, "rope_store: a bias comes with partial products only");
  const SplitProduct sp{parts, nparts, (size_t)T * (nh + 2 * nkv) * D, bias};
  if (T == 0) return nullptr;
  const int heads = kc != nullptr ? nh + 2 * nkv : nh + nkv;
  if (cosv == nullptr && kc == nullptr && parts == nullptr && qscale == 1.f) return nullptr;
  const bool aligned = ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)kc % 16) == 0 &&
                       ((uintptr_t)cosv % 16) == 0 && ((uintptr_t)sinv % 16) == 0;
  const bool sums_aligned = parts == nullptr || (((uintptr_t)parts % 16) == 0 && ((uintptr_t)bias % 16) == 0 &&
                                                  ((size_t)T * (nh + 2 * nkv) * D) % 4 == 0);
  if (T >= VECTOR_MIN_TOKENS && nparts <= 1 && D % 16 == 0 && rot % 16 == 0 && D <= 256 && aligned &&
      sums_aligned) {
    const int items = (nh + nkv) * (D / 16);
    const int gy = (items + 255) / 256 < 64 ? (items + 255) / 256 : 64;
    const long long v_blocks = vc != nullptr ? (long long)((T + 15) / 16) * nkv : 0;
    SL_CHECK(v_blocks + (long long)T * gy < (1ll << 31), "rope_store: too many tokens");
    rope_store_vec_kernel<<<(unsigned)(v_blocks + (long long)T * gy), 256, 0, stream>>>(
        (act_t*)qkv, sp, cosv, sinv, slots, (act_t*)kc, (act_t*)vc, T, nh, nkv, D, rot, page, pairs8, qscale,
        (int)v_blocks, gy);
    return sl_launch_status();
  }
  rope_store_kernel<<<dim3(T, heads), 64, 0, stream>>>((act_t*)qkv, sp, cosv, sinv, slots, (act_t*)kc,
                                                       (act_t*)vc, nh, nkv, D, rot, page, pairs8, qscale);
  return sl_launch_status();
}
