"""Plain, slow implementation of the Qwen2 dense decoder.

Whole sequences, no cache, one function per part, float32 (or float64) torch on
the CPU.  It shares no code with ``servelab_amd``: it reads ``config.json`` and
``model.safetensors`` itself (through the ``safetensors`` package, which the
engine does not use) and is the oracle every engine test compares against.

Each function cites the reference lines (relative to the reference checkout)
whose formula it follows.  Bodies that the reference does not ship (RMSNorm,
apply_rope, the sliding window) follow the contracts its call sites and tests
pin; see the citations.
"""
import json
import math
import os

import torch


# --------------------------------------------------------------------- parts
def rms_norm(x, weight, eps):
    """y = x * rsqrt(mean(x^2) + eps) * w, all in the working precision.

    tests/test_triton_kernels.py:57-59 (the reference's own vector),
    servelab/attention/triton/paged_attention.py:86-91.
    """
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def rope_inv_freq(theta, head_dim, dtype=torch.float32):
    """inv_freq[j] = theta ** (-2j / D), j = 0 .. D/2-1.

    servelab/parallel/tp_model.py:94-96.
    """
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=dtype) / head_dim))


def apply_rope(x, positions, inv_freq):
    """Rotate-half rotary embedding on x [T, heads, D].

    Pairs are (j, j + D/2): x' = [x1 cos - x2 sin, x2 cos + x1 sin].
    Call contract servelab/parallel/tp_model.py:128 with inv_freq from :94-96;
    the rotate-half convention is stated in docs/architecture.md:69 and
    docs/knowledge_checklist.md:12-13.
    """
    half = x.shape[-1] // 2
    ang = positions.to(inv_freq.dtype)[:, None] * inv_freq[None, :]   # [T, D/2]
    cos = torch.cos(ang)[:, None, :].to(x.dtype)
    sin = torch.sin(ang)[:, None, :].to(x.dtype)
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)


def visibility_mask(q_positions, k_positions, window=None):
    """True where key r is visible to the query at p: r <= p, and with a window
    W also p - W < r.

    Causal part: servelab/parallel/tp_model.py:149-153 and
    servelab/engine/speculative.py:77-80 (mask where q_pos < k_pos).  The
    window is not in the reference; its rule (the last W positions, self
    included) is this build's own.
    """
    q = q_positions[:, None]
    k = k_positions[None, :]
    vis = k <= q
    if window is not None:
        vis = vis & (k > q - window)
    return vis


def attention(q, k, v, scale, q_positions, k_positions, window=None):
    """Grouped-query attention over whole sequences.

    q [Tq, nh, D], k/v [Tk, nkv, D].  kv head of query head h is h // g
    (servelab/attention/triton/paged_attention.py:41), expressed as
    repeat_interleave (servelab/parallel/tp_model.py:144-146); scores,
    softmax and PV as tp_model.py:147-155.
    """
    nh, nkv = q.shape[1], k.shape[1]
    g = nh // nkv
    if g > 1:
        k = k.repeat_interleave(g, dim=1)
        v = v.repeat_interleave(g, dim=1)
    scores = torch.einsum("qhd,rhd->hqr", q, k) * scale
    vis = visibility_mask(q_positions, k_positions, window)
    scores = scores.masked_fill(~vis[None], float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    return torch.einsum("hqr,rhd->qhd", probs, v)


def swiglu(x, w_gate, w_up, w_down):
    """down(silu(gate(x)) * up(x)), no biases.

    servelab/parallel/tp_model.py:67-68.
    """
    g = x @ w_gate.T
    return ((g * torch.sigmoid(g)) * (x @ w_up.T)) @ w_down.T


def layer_window(cfg, layer_index):
    """Window of a layer or None: windowed iff use_sliding_window and
    layer_index >= max_window_layers (this build's rule; the reference has no
    window)."""
    if cfg.get("use_sliding_window", False) and cfg.get("sliding_window") \
            and layer_index >= cfg.get("max_window_layers", 0):
        return int(cfg["sliding_window"])
    return None


def decoder_layer(cfg, w, i, h, positions):
    """Pre-norm block: h += Attn(Norm(h)); h += MLP(Norm(h)).

    servelab/parallel/tp_model.py:124-133 (order of ops), :48-53 (q/k/v with
    bias, head-major views), :41 (scale), :46 (o_proj without bias).
    """
    p = f"model.layers.{i}."
    nh = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads", nh)
    D = cfg.get("head_dim", cfg["hidden_size"] // nh)
    eps = cfg["rms_norm_eps"]
    T = h.shape[0]

    def project(name, heads):
        y = x @ w[p + f"self_attn.{name}.weight"].T
        if cfg.get("attention_bias", True):           # servelab/parallel/tp_model.py:48-50 (qkv_bias)
            y = y + w[p + f"self_attn.{name}.bias"]
        return y.view(T, heads, D)

    x = rms_norm(h, w[p + "input_layernorm.weight"], eps)
    q, k, v = project("q_proj", nh), project("k_proj", nkv), project("v_proj", nkv)
    inv_freq = rope_inv_freq(cfg.get("rope_theta", 1e6), D, dtype=h.dtype).to(h.device)
    q = apply_rope(q, positions, inv_freq)
    k = apply_rope(k, positions, inv_freq)
    o = attention(q, k, v, 1.0 / math.sqrt(D), positions, positions,
                  layer_window(cfg, i))
    h = h + o.reshape(T, nh * D) @ w[p + "self_attn.o_proj.weight"].T
    x2 = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
    h = h + swiglu(x2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                   w[p + "mlp.down_proj.weight"])
    return h


def forward(cfg, weights, token_ids, dtype=torch.float32, start_position=0):
    """Logits [T, V] for one whole sequence.

    Embedding servelab/parallel/tp_model.py:123; final norm :134; head with
    tied or untied weights :115-119; same as the reference's plain runner
    servelab/engine/speculative.py:53-87, which returns logits at every
    position.
    """
    w = {k: v.to(dtype) for k, v in weights.items()}
    device = w["model.embed_tokens.weight"].device
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
    positions = torch.arange(start_position, start_position + len(ids), device=device)
    h = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        h = decoder_layer(cfg, w, i, h, positions)
    z = rms_norm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) \
        else w["lm_head.weight"]
    return z @ head.T


def greedy_generate(cfg, weights, prompt, max_tokens, dtype=torch.float32):
    """Full recompute at every step; argmax takes the first maximal index
    (servelab/engine/sampler.py:23-24)."""
    toks = list(prompt)
    out = []
    for _ in range(max_tokens):
        logits = forward(cfg, weights, toks, dtype)
        nxt = int(torch.argmax(logits[-1]).item())
        out.append(nxt)
        toks.append(nxt)
    return out


# -------------------------------------------------------------------- folder
def load_folder(path):
    """(config dict, {checkpoint name: tensor}) read with the safetensors
    package; tensors are upcast by ``forward``."""
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json"), encoding="utf-8") as f:
        cfg = json.load(f)
    weights = load_file(os.path.join(path, "model.safetensors"))
    return cfg, weights
