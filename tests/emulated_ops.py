"""Plain torch versions of the kernel table, one function per kernel, written
from each kernel's contract (inputs, layouts, outputs).

Two uses: GPU tests compare each HIP kernel alone with the function of the same
name here; CPU tests plug this table into the engine so that everything above
the kernels (cache manager, block tables, batch packing, step function,
scheduler) runs without a GPU.  Nothing in ``servelab_amd`` imports this file.

Layouts: K pages [pages, nkv, page_size, D]; V pages [pages, nkv, D, page_size];
qkv rows [T, (nh + 2 nkv) D] with q first, then k, then v, head-major.
"""
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
