"""Plain torch versions of the kernel table, one function per kernel, written
from each kernel's contract (inputs, layouts, outputs).

Two uses: GPU tests compare each HIP kernel alone with the function of the same
name here; CPU tests plug this table into the engine so that everything above
the kernels (cache manager, block tables, batch packing, step function,
scheduler) runs without a GPU.  Nothing in ``servelab_amd`` imports this file.

Layouts: K pages [pages, nkv, page_size, D]; V pages [pages, nkv, D, page_size];
qkv rows [T, (nh + 2 nkv) D] with q first, then k, then v, head-major.
"""
import numpy as np
import torch


def _f(x):
    return x.float()


class EmulatedOps:
    def __init__(self, act_dtype=torch.float32):
        self.act_dtype = act_dtype

    # ------------------------------------------------------------ embedding
    def embed(self, ids, table):
        return _f(table[ids.long()])

    # ---------------------------------------------------------------- norms
    def add_rmsnorm(self, resid, delta, weight, eps, fuse=False):
        if delta is not None:
            resid += _f(delta)
        var = resid.pow(2).mean(-1, keepdim=True)
        return (resid * torch.rsqrt(var + eps) * weight).to(self.act_dtype)

    def rows_add_rmsnorm(self, resid, delta, rows, weight, eps, fuse=False):
        x = resid[rows.long()]
        if delta is not None:
            x = x + _f(delta[rows.long()])
        var = x.pow(2).mean(-1, keepdim=True)
        return (x * torch.rsqrt(var + eps) * weight).to(self.act_dtype)

    # --------------------------------------------------------------- linear
    def linear(self, x, w, bias, out_f32=False, defer=False):
        y = _f(x) @ _f(w).T
        if bias is not None:
            y = y + bias
        return y if out_f32 else y.to(self.act_dtype)

    def silu_mul(self, gate_up, block=None):
        """gate and up interleaved in blocks of ``block`` columns (default: halves)."""
        T, inter = gate_up.shape[0], gate_up.shape[1] // 2
        block = inter if block is None else block
        gu = _f(gate_up).view(T, inter // block, 2, block)
        g, u = gu[:, :, 0].reshape(T, inter), gu[:, :, 1].reshape(T, inter)
        return (g * torch.sigmoid(g) * u).to(self.act_dtype)

    def attend_and_project(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                           batch, scale, window, w_out, bias=None, defer=False):
        attn = self.paged_attention(qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                                    batch, scale, window)
        return self.linear(attn, w_out, bias, defer=defer)

    def gated_mlp(self, x, w_gate_up, block, w_down, defer=False):
        return self.linear(self.gated_linear(x, w_gate_up, block), w_down, None, defer=defer)

    def gated_linear(self, x, w, block):
        return self.silu_mul(self.linear(x, w, None), block)

    # ----------------------------------------------------------------- rope
    def rope_tables(self, positions, inv_freq):
        ang = positions.float()[:, None] * inv_freq[None, :]
        return torch.cos(ang), torch.sin(ang)

    def rope_store(self, qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                   pairs8=False, rot_dim=None):
        """Rotate the first ``rot_dim`` channels (default: all) of the q and k
        heads of ``qkv`` in place; write k and v to their pages.  ``pairs8``:
        the rotated channels come in blocks of 8 channels and their 8 partners
        (channel order [block][half][8]) instead of first half, second half."""
        T = qkv.shape[0]
        R = D if rot_dim is None else rot_dim
        half = R // 2
        qk = qkv[:, :(nh + nkv) * D].view(T, nh + nkv, D)
        if cos is not None:
            turned = qk[..., :R]
            if pairs8:
                std = turned.reshape(T, nh + nkv, half // 8, 2, 8).transpose(2, 3).reshape(T, nh + nkv, R)
            else:
                std = turned
            x1, x2 = _f(std[..., :half]), _f(std[..., half:])
            c, s = cos[:, None, :], sin[:, None, :]
            rot = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1).to(qkv.dtype)
            if pairs8:
                rot = rot.reshape(T, nh + nkv, 2, half // 8, 8).transpose(2, 3).reshape(T, nh + nkv, R)
            turned.copy_(rot)
        if k_cache is None:
            return
        k = qkv[:, nh * D:(nh + nkv) * D].view(T, nkv, D)
        v = qkv[:, (nh + nkv) * D:].view(T, nkv, D)
        page, off = (slots // page_size).long(), (slots % page_size).long()
        k_cache[page, :, off, :] = k.to(k_cache.dtype)
        v_cache[page, :, :, off] = v.to(v_cache.dtype)

    def qkv_rope_store(self, x, w, bias, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                       rot_dim=None):
        qkv = self.linear(x, w, bias)
        self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size, True, rot_dim)
        return qkv

    # --------------------------------------------- position encodings of a mixer
    def plan_rotation(self, head_dim, layout):
        """Channels stay as the checkpoint has them, except that an interleaved
        pairing is turned into halves (written independently of the kernel
        table's own: no blocks of 8 here)."""
        import types
        rot = 0 if layout is None else layout.rot_dim
        order = None
        if layout is not None and layout.pairing == "interleaved":
            order = torch.cat([torch.arange(0, rot, 2), torch.arange(1, rot, 2),
                               torch.arange(rot, head_dim)])
        return types.SimpleNamespace(order=order, rot_dim=rot, blocked=False)

    def project_qkv(self, x, w, bias, nh, nkv, D, plan, tables, slots, k_cache, v_cache, page_size,
                    q_scale=1.0):
        assert q_scale == 1.0                # (this table leaves the whole scale to paged_attention)
        qkv = self.linear(x, w, bias)
        cos, sin = (tables.cos, tables.sin) if tables is not None else (None, None)
        self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size, False,
                        plan.rot_dim)
        return qkv

    # ------------------------------------------------------------ attention
    def paged_attention(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                        batch, scale, window):
        T = qkv.shape[0]
        g = nh // nkv
        out = torch.empty(T, nh * D, dtype=self.act_dtype, device=qkv.device)
        cu = batch.cu_q.tolist()
        ctxs = batch.ctx_len.tolist()
        for s in range(batch.num_seqs):
            a, b = cu[s], cu[s + 1]
            ctx = ctxs[s]
            q = _f(qkv[a:b, :nh * D]).view(b - a, nh, D)
            q_pos = batch.positions[a:b].long()
            lo = 0
            if window is not None:
                lo = max(0, int(q_pos[0]) - window + 1)
            k_pos = torch.arange(lo, ctx)
            pages = block_tables[s].long()[k_pos // page_size]
            offs = k_pos % page_size
            k = _f(k_cache[pages, :, offs, :])                     # [ctx', nkv, D]
            v = _f(v_cache[pages, :, :, offs])                     # [ctx', nkv, D]
            k = k.repeat_interleave(g, dim=1)
            v = v.repeat_interleave(g, dim=1)
            scores = torch.einsum("qhd,rhd->hqr", q, k) * scale
            vis = k_pos[None, :] <= q_pos[:, None]
            if window is not None:
                vis &= k_pos[None, :] > q_pos[:, None] - window
            scores = scores.masked_fill(~vis[None], float("-inf"))
            o = torch.einsum("hqr,rhd->qhd", torch.softmax(scores, -1), v)
            out[a:b] = o.reshape(b - a, nh * D).to(self.act_dtype)
        return out

    # ------------------------------------------------------------- sampling
    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).to(torch.int32)

    def sample(self, logits, temperature, top_k, top_p, seeds, draws):
        """One token per row: the argmax where temperature is 0, else the largest
        of ``perturbed_scores`` among the logits the row's cut keeps."""
        out = []
        for r in range(logits.shape[0]):
            T = float(temperature[r])
            if T == 0.0:
                out.append(int(torch.argmax(logits[r])))
                continue
            k = int(top_k[r]) if top_k is not None else -1
            p = float(top_p[r]) if top_p is not None else 1.0
            scores = perturbed_scores(logits[r], T, int(seeds[r]), int(draws[r]))
            scores[~kept_by_cut(logits[r], T, k, p)] = -np.inf
            out.append(int(np.argmax(scores)))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)


def uniform01(seed: int, draw: int, n: int) -> np.ndarray:
    """u_i in (0, 1) for i in [0, n): a counter-based 64-bit mix of (seed, draw, i)
    whose top 23 bits become (bits + 0.5) / 2^23."""
    one = np.ones(n, dtype=np.uint64)
    i = np.arange(n, dtype=np.uint64)
    z = one * np.uint64(seed % (1 << 64)) + np.uint64(0x9E3779B97F4A7C15) * (
        one * np.uint64(draw) * np.uint64(0x100000001B3) + i + np.uint64(1))
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    z ^= z >> np.uint64(31)
    return ((z >> np.uint64(41)).astype(np.float64) + 0.5) / 8388608.0


def perturbed_scores(row, T: float, seed: int, draw: int) -> np.ndarray:
    """logit_i / max(T, 1e-6) + g_i with g_i = -ln(-ln u_i): the index of the
    largest one is an exact draw from softmax(logits / T) (Gumbel-max)."""
    x = row.detach().double().cpu().numpy() / max(T, 1e-6)
    u = uniform01(seed, draw, x.shape[0])
    return x - np.log(-np.log(u))


def kept_by_cut(row, T: float, top_k: int, top_p: float) -> np.ndarray:
    """Which logits a row's cut keeps: the top_k largest when top_k > 0 (top_p is
    then ignored); else the sorted prefix whose cumulative probability stays
    <= top_p, the first always kept (servelab/engine/sampler.py:30-44)."""
    x = row.detach().double().cpu().numpy() / max(T, 1e-6)
    keep = np.ones(x.shape[0], dtype=bool)
    if top_k > 0:
        keep[:] = False
        keep[np.argsort(-x, kind="stable")[:top_k]] = True
    elif top_p < 1.0:
        order = np.argsort(-x, kind="stable")
        probs = np.exp(x[order] - x[order[0]])
        cum = np.cumsum(probs / probs.sum())
        inside = cum <= top_p
        inside[0] = True
        keep[:] = False
        keep[order[inside]] = True
    return keep
