"""Pins of the plain implementation: what fixes each formula besides the
reference's text (no GPU).  Each check fails for a plausible mistake: a wrong
sign or pairing in the rotation, a norm in the wrong place, a mask off by one,
a wrong head-to-kv-head mapping."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen2 as plain
from tiny_configs import TINY_A, TINY_B, make_folder

torch.manual_seed(0)


def test_rmsnorm_reference_vector_and_invariants():
    # the reference's own vector: tests/test_triton_kernels.py:57-59
    x, w = torch.randn(6, 40), torch.randn(40)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
    assert torch.allclose(plain.rms_norm(x, w, 1e-6), want, atol=0, rtol=0)
    assert torch.allclose(plain.rms_norm(x, w, 1e-6), F.rms_norm(x, (40,), w, 1e-6), atol=1e-6)
    y = plain.rms_norm(x, torch.ones(40), 1e-12)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(6), atol=1e-5)      # unit mean square
    assert torch.allclose(plain.rms_norm(3.0 * x, w, 1e-12), plain.rms_norm(x, w, 1e-12), atol=1e-5)
    # not LayerNorm: a constant offset is not removed
    assert not torch.allclose(plain.rms_norm(x + 5, w, 1e-6), plain.rms_norm(x, w, 1e-6), atol=1e-2)


def test_rope_properties():
    D = 16
    inv = plain.rope_inv_freq(10000.0, D)
    assert torch.allclose(inv, torch.tensor([10000.0 ** (-2 * j / D) for j in range(D // 2)]))
    x = torch.randn(5, 3, D)
    pos = torch.tensor([0, 1, 2, 7, 100])
    y = plain.apply_rope(x, pos, inv)
    assert torch.equal(y[0], x[0])                                          # position 0 is the identity
    half = D // 2
    n_in = x[..., :half] ** 2 + x[..., half:] ** 2                          # pairs are (j, j + D/2)
    n_out = y[..., :half] ** 2 + y[..., half:] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-5)
    n_wrong = y[..., 0::2] ** 2 + y[..., 1::2] ** 2                          # not (2j, 2j + 1)
    assert not torch.allclose(x[..., 0::2] ** 2 + x[..., 1::2] ** 2, n_wrong, atol=1e-3)
    # only distances count: shifting both positions leaves the score unchanged
    q, k = torch.randn(1, 1, D), torch.randn(1, 1, D)

    def score(m, n):
        return (plain.apply_rope(q, torch.tensor([m]), inv) *
                plain.apply_rope(k, torch.tensor([n]), inv)).sum()
    assert torch.allclose(score(5, 2), score(105, 102), atol=1e-4)
    assert not torch.allclose(score(5, 2), score(2, 5), atol=1e-3)           # sign of the rotation
    # the rotation goes the documented way: one pair, angle pos * inv_freq
    e = torch.zeros(1, 1, D)
    e[0, 0, 0] = 1.0
    r = plain.apply_rope(e, torch.tensor([1]), inv)
    assert torch.allclose(r[0, 0, 0], torch.cos(torch.tensor(1.0))) and \
        torch.allclose(r[0, 0, half], torch.sin(torch.tensor(1.0)))
    big = plain.apply_rope(x, pos, plain.rope_inv_freq(1e200, D, dtype=torch.float64).float())
    assert torch.allclose(big[..., 1:half], x[..., 1:half], atol=1e-3)       # theta -> inf: identity


def test_rope_is_a_complex_multiplication():
    """The rotation as a library routine: the pair (x[j], x[j + D/2]) read as the complex number
    x[j] + i x[j + D/2] is multiplied by exp(+i pos inv_freq[j]).  A flipped sign (the conjugate)
    or interleaved pairs (x[2j], x[2j + 1]) fail this."""
    D = 24
    inv = plain.rope_inv_freq(1e6, D)
    x = torch.randn(7, 3, D, dtype=torch.float64)
    pos = torch.tensor([0, 1, 3, 4, 50, 51, 64])        # float32 angles: small positions keep 1e-5
    z = torch.complex(x[..., :D // 2], x[..., D // 2:])
    angle = pos.double()[:, None, None] * inv.double()
    want = z * torch.polar(torch.ones_like(angle), angle)
    got = plain.apply_rope(x.float(), pos, inv)
    assert torch.allclose(got[..., :D // 2].double(), want.real, atol=1e-5)
    assert torch.allclose(got[..., D // 2:].double(), want.imag, atol=1e-5)
    flipped = z * torch.polar(torch.ones_like(angle), -angle)
    assert not torch.allclose(got[..., D // 2:].double(), flipped.imag, atol=1e-2)
    # hence q_m . k_n = Re(sum_j q_j conj(k_j) exp(i (m - n) theta_j)): distances only
    q, k = torch.randn(1, 1, D), torch.randn(1, 1, D)
    zq = torch.complex(q[..., :D // 2], q[..., D // 2:]).to(torch.complex128)
    zk = torch.complex(k[..., :D // 2], k[..., D // 2:]).to(torch.complex128)
    m, n = 40, 33
    want_score = (zq * zk.conj() * torch.polar(torch.ones(D // 2, dtype=torch.float64),
                                               (m - n) * inv.double())).real.sum()
    got_score = (plain.apply_rope(q, torch.tensor([m]), inv) *
                 plain.apply_rope(k, torch.tensor([n]), inv)).sum()
    assert abs(float(got_score) - float(want_score)) < 1e-4


def test_attention_reduces_to_the_library_routine():
    T, nh, nkv, D = 9, 4, 2, 8
    q, k, v = torch.randn(T, nh, D), torch.randn(T, nkv, D), torch.randn(T, nkv, D)
    pos = torch.arange(T)
    got = plain.attention(q, k, v, 1 / math.sqrt(D), pos, pos)
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1),
                                          vv.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-5)
    assert torch.allclose(got[0], vv[0], atol=1e-6)           # the first token sees only itself
    # kv head of head h is h // g, not h % nkv
    k2 = k.clone()
    k2[:, 1] += 1.0
    changed = (plain.attention(q, k2, v, 1.0, pos, pos) - plain.attention(q, k, v, 1.0, pos, pos)).abs().amax((0, 2))
    assert (changed[:2] == 0).all() and (changed[2:] > 0).all()
    # one head, one kv head: plain single-head attention
    g1 = plain.attention(q[:, :1], k[:, :1], v[:, :1], 0.5, pos, pos)
    s = (q[:, 0] @ k[:, 0].T) * 0.5
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(g1[:, 0], torch.softmax(s, -1) @ v[:, 0], atol=1e-5)


def test_decode_special_case_matches_the_reference_kernel_test():
    # tests/test_triton_kernels.py:38-45: one query against the whole context
    ctx, nh, nkv, D = 40, 8, 2, 16
    q, k, v = torch.randn(1, nh, D), torch.randn(ctx, nkv, D), torch.randn(ctx, nkv, D)
    scale = D ** -0.5
    kc, vc = k.repeat_interleave(4, 1), v.repeat_interleave(4, 1)
    p = torch.softmax(torch.einsum("hd,rhd->hr", q[0], kc) * scale, -1)
    want = torch.einsum("hr,rhd->hd", p, vc)
    got = plain.attention(q, k, v, scale, torch.tensor([ctx - 1]), torch.arange(ctx))
    assert torch.allclose(got[0], want, atol=1e-5)


def test_window():
    T, D = 30, 8
    q, k, v = torch.randn(T, 2, D), torch.randn(T, 1, D), torch.randn(T, 1, D)
    pos = torch.arange(T)
    full = plain.attention(q, k, v, 1.0, pos, pos)
    assert torch.allclose(plain.attention(q, k, v, 1.0, pos, pos, window=T), full)   # W >= ctx
    assert torch.allclose(plain.attention(q, k, v, 1.0, pos, pos, window=1),
                          v.expand(T, 2, D), atol=1e-6)                               # W = 1: own v
    w = plain.attention(q, k, v, 1.0, pos, pos, window=5)
    assert torch.allclose(w[:5], full[:5], atol=1e-6) and not torch.allclose(w[5:], full[5:], atol=1e-3)
    # locality: a key at distance >= W does not matter, one at distance W - 1 does
    k2, v2 = k.clone(), v.clone()
    k2[10] += 3.0
    v2[10] -= 2.0
    w2 = plain.attention(q, k2, v2, 1.0, pos, pos, window=5)
    assert torch.equal(w2[15:], w[15:]) and not torch.allclose(w2[14], w[14], atol=1e-4)
    vis = plain.visibility_mask(torch.tensor([20]), torch.arange(30), 16)[0]
    assert vis.nonzero().flatten().tolist() == list(range(5, 21))           # the last 16, self included


def test_swiglu():
    x = torch.randn(3, 10)
    wg, wu, wd = torch.randn(7, 10), torch.randn(7, 10), torch.randn(10, 7)
    want = (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    assert torch.allclose(plain.swiglu(x, wg, wu, wd), want, atol=1e-5)
    assert plain.swiglu(x, torch.zeros(7, 10), wu, wd).abs().max() == 0      # gate 0 => 0


def test_whole_model_options(tmp_path):
    fa = make_folder(tmp_path, "A", seed=2)
    cfg, w = plain.load_folder(fa)
    toks = torch.randint(0, 512, (40,)).tolist()
    logits = plain.forward(cfg, w, toks)
    assert logits.shape == (40, 512)
    # tied head: logits = z E^T; an untied model with lm_head := E agrees
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"]
    cfg2 = dict(cfg, tie_word_embeddings=False)
    assert torch.equal(plain.forward(cfg2, w2, toks), logits)
    # causality: a later token does not change earlier logits
    toks2 = toks[:30] + [(toks[30] + 1) % 512] + toks[31:]
    l2 = plain.forward(cfg, w, toks2)
    assert torch.equal(l2[:30], logits[:30]) and not torch.allclose(l2[30:], logits[30:], atol=1e-5)
    # biases matter (the reference's fixture has them zero)
    w3 = dict(w)
    w3["model.layers.0.self_attn.k_proj.bias"] = torch.zeros_like(w["model.layers.0.self_attn.k_proj.bias"])
    assert not torch.allclose(plain.forward(cfg, w3, toks), logits, atol=1e-5)
    # float64 agrees with float32 to rounding
    assert (plain.forward(cfg, w, toks, torch.float64).float() - logits).abs().max() < 1e-5

    fb = make_folder(tmp_path, "B", seed=2)
    cfg, w = plain.load_folder(fb)
    toks = torch.randint(0, 1000, (40,)).tolist()
    with_window = plain.forward(cfg, w, toks)
    without = plain.forward(dict(cfg, use_sliding_window=False), w, toks)
    assert torch.allclose(with_window[:16], without[:16], atol=1e-6)        # nothing is cut yet
    assert not torch.allclose(with_window[17:], without[17:], atol=1e-5)
    all_layers = plain.forward(dict(cfg, max_window_layers=0), w, toks)     # layers 0-1 stay full
    assert not torch.allclose(all_layers[17:], with_window[17:], atol=1e-5)
    assert plain.layer_window(cfg, 1) is None and plain.layer_window(cfg, 2) == 16


def test_greedy_generation_is_incremental(tmp_path):
    folder = make_folder(tmp_path, "A", seed=4)
    cfg, w = plain.load_folder(folder)
    out = plain.greedy_generate(cfg, w, [1, 2, 3, 4, 5], 6)
    assert len(out) == 6
    assert out[:3] == plain.greedy_generate(cfg, w, [1, 2, 3, 4, 5], 3)
