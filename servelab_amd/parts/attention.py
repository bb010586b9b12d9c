"""Grouped-query attention over a paged cache.

Reference math: q/k/v projections with optional bias, head-major views
(servelab/parallel/tp_model.py:43-53); rotary on q and k before k is cached
(:128-129); per sequence scores * 1/sqrt(D), causal mask, softmax and PV in
float32 with kv head = head // g (:136-157).  The reference runs three GEMMs
and a Python loop over sequences; here q, k and v come from one GEMM over the
row-concatenated weight, the kernel table applies the position encoding (a
parameter this mixer never looks inside) and writes the pages, and one call
attends for all sequences of the batch through their block tables.  The
window (keys p - W < r <= p) is this build's own.
"""
import math

import torch

from .base import Mixer, PagedKVSpec, ParamSpec


class PagedAttention(Mixer):
    graph_safe = True
    takes_scaled_rows = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, position,
                 qkv_bias=True, window=None, scale=None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.position = position
        self.qkv_bias = bool(qkv_bias)
        self.window = None if not window else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)

    # ---- declarations
    def param_specs(self):
        h, d = self.hidden_size, self.head_dim
        specs = {
            "q_proj.weight": ParamSpec((self.num_heads * d, h)),
            "k_proj.weight": ParamSpec((self.num_kv_heads * d, h)),
            "v_proj.weight": ParamSpec((self.num_kv_heads * d, h)),
            "o_proj.weight": ParamSpec((h, self.num_heads * d)),
        }
        if self.qkv_bias:
            specs["q_proj.bias"] = ParamSpec((self.num_heads * d,))
            specs["k_proj.bias"] = ParamSpec((self.num_kv_heads * d,))
            specs["v_proj.bias"] = ParamSpec((self.num_kv_heads * d,))
        return specs

    def cache_spec(self):
        return PagedKVSpec(self.num_kv_heads, self.head_dim, self.window)

    def load(self, tensors, rt):
        self.rt = rt
        self.position.load(tensors, rt)
        # [Wq; Wk; Wv] -> one [(nh + 2 nkv) D, H] matrix, one GEMM.  The kernel table says in
        # which order it wants the channels of every q and k head for this position encoding
        # (q . k does not depend on the order as long as both agree); v keeps its own.
        self.rotation = rt.ops.plan_rotation(self.head_dim, self.position.layout())
        order = self.rotation.order

        def reorder(t, heads):
            if order is None:
                return t
            by_head = t.reshape(heads, self.head_dim, *t.shape[1:])
            return by_head[:, order.to(t.device)].reshape(t.shape)
        self.w_qkv = rt.linear_weight(torch.cat(
            [reorder(tensors("q_proj.weight"), self.num_heads),
             reorder(tensors("k_proj.weight"), self.num_kv_heads), tensors("v_proj.weight")], 0))
        self.b_qkv = None
        if self.qkv_bias:
            self.b_qkv = rt.vector(torch.cat(
                [reorder(tensors("q_proj.bias").float(), self.num_heads),
                 reorder(tensors("k_proj.bias").float(), self.num_kv_heads),
                 tensors("v_proj.bias").float()], 0))
        self.w_o = rt.linear_weight(tensors("o_proj.weight"), delta=True)
        # a kernel table may want part of the score scale applied to q where q is made
        split = getattr(rt.ops, "split_attention_scale", None)
        self.q_scale, self.score_scale = split(self.scale) if split is not None else (1.0, self.scale)

    # ---- compute
    def forward(self, x, batch, cache, shared):
        ops = self.rt.ops
        group = batch.groups[cache.group]
        slots, kc, vc = (group.slots, cache.k, cache.v) if cache.write else (None, None, None)
        qkv = ops.project_qkv(x, self.w_qkv, self.b_qkv, self.num_heads, self.num_kv_heads,
                              self.head_dim, self.rotation, self.position.tables(batch, shared),
                              slots, kc, vc, cache.page_size, q_scale=self.q_scale)
        return ops.attend_and_project(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, cache.k, cache.v,
            cache.page_size, group.block_tables, batch, self.score_scale, self.window,
            self.w_o, None, defer=True)
