"""A Qwen2 model folder with hand-made weights whose logits say which keys every
position saw and how much weight each had.

Random weights hide a fault of the cache or of a mask: one wrongly visible key
among two hundred moves a logit by less than bfloat16 rounding does.  Here the
logits are (up to the final norm) weighted counts of the visible keys by token:

* the hidden state has a block of CODES dimensions for the token's own code, a
  block each for what layer 0 and layer 1 add, and a sign dimension: token t
  embeds as the unit vector of t % CODES plus u_t = +-1 in SIGN_DIM;
* q is a constant (its bias; the weight is zero) and k reads the sign, both in
  the pair of rotary channels with the lowest frequency (theta = 1e6: at
  position 1,000 they have turned by 0.002 rad), so the score of a key is
  +-GAMMA by its sign and the head's preference - even heads prefer u = +1, odd
  heads u = -1 - and a key read from a wrong cache row gets the wrong weight;
* v is the key's own code; o_proj adds GAIN times the two heads of a group into
  the layer's block; the feed-forward adds nothing (down_proj = 0);
* layer 0 sees all keys, layer 1 a window; logit t < CODES reads layer 0's
  block, logit CODES + t layer 1's, so a logit is (rescaled by the final norm)
  the weight that position gave to the visible keys that hold token t.  One key
  dropped or added changes its token's logit by its share among the visible
  keys of that token, about CODES / n of it, whatever the length n.

``tests/test_probe_model.py`` shows on the CPU that a window off by one, one
dropped far key or two swapped pages of keys move a logit by several times the bar the
GPU tests hold the engine to in bfloat16.
"""
import json
import os

import torch

from servelab_amd.weights.safetensors_io import write_safetensors

CODES = 64               # distinct codes (= v channels of all kv heads together)
SIGN_DIM = 200
GAMMA = 0.8              # score of a key: +-GAMMA
GAIN = 24.0

PROBE = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=2, hidden_size=256, num_attention_heads=4, num_key_value_heads=2,
    head_dim=32, intermediate_size=48, vocab_size=136, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, use_sliding_window=True,
    sliding_window=24, max_window_layers=1, max_position_embeddings=1024,
    torch_dtype="float32", eos_token_id=135)


def token_sign(t: int) -> float:
    return 1.0 if (t * 7 + t // 3) % 2 == 0 else -1.0


def probe_tensors(cfg=PROBE):
    H, V, L = cfg["hidden_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    nh, nkv, D, I = (cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                     cfg["intermediate_size"])
    assert nkv * D == CODES and nh == 2 * nkv and 3 * CODES <= SIGN_DIM < H and L == 2
    low = D // 2 - 1                                   # the rotary pair that turns slowest: (low, low + D/2)
    t = {}
    emb = torch.zeros(V, H)
    for tok in range(V):
        emb[tok, tok % CODES] = 1.0
        emb[tok, SIGN_DIM] = token_sign(tok)
    t["model.embed_tokens.weight"] = emb
    head = torch.zeros(V, H)
    for tok in range(V):                               # logits beyond 2 * CODES read nothing
        if tok < 2 * CODES:
            head[tok, CODES + tok] = 1.0
    t["lm_head.weight"] = head
    t["model.norm.weight"] = torch.ones(H)
    gen = torch.Generator().manual_seed(1)
    for i in range(L):
        p = f"model.layers.{i}."
        t[p + "input_layernorm.weight"] = torch.ones(H)
        t[p + "post_attention_layernorm.weight"] = torch.ones(H)
        t[p + "self_attn.q_proj.weight"] = torch.zeros(nh * D, H)
        bq = torch.zeros(nh, D)
        for h in range(nh):
            bq[h, low] = 4.0 if h % 2 == 0 else -4.0
        t[p + "self_attn.q_proj.bias"] = bq.reshape(-1)
        # the normed sign entry is +-sqrt(H / 2) in layer 0 (two entries of size 1 among H); the
        # score is q k / sqrt(D), so this weight makes it +-GAMMA there
        wk = torch.zeros(nkv, D, H)
        wk[:, low, SIGN_DIM] = GAMMA * (D ** 0.5) / 4.0 / (H / 2) ** 0.5
        t[p + "self_attn.k_proj.weight"] = wk.reshape(nkv * D, H)
        t[p + "self_attn.k_proj.bias"] = torch.zeros(nkv * D)
        wv = torch.zeros(nkv * D, H)
        wv[torch.arange(CODES), torch.arange(CODES)] = 1.0
        t[p + "self_attn.v_proj.weight"] = wv
        t[p + "self_attn.v_proj.bias"] = torch.zeros(nkv * D)
        wo = torch.zeros(H, nh, D)
        for g in range(nkv):
            for c in range(D):
                wo[(i + 1) * CODES + g * D + c, 2 * g, c] = GAIN / (H / 2) ** 0.5
                wo[(i + 1) * CODES + g * D + c, 2 * g + 1, c] = GAIN / (H / 2) ** 0.5
        t[p + "self_attn.o_proj.weight"] = wo.reshape(H, nh * D)
        t[p + "mlp.gate_proj.weight"] = torch.randn(I, H, generator=gen) * 0.05
        t[p + "mlp.up_proj.weight"] = torch.randn(I, H, generator=gen) * 0.05
        t[p + "mlp.down_proj.weight"] = torch.zeros(H, I)
    return t


def write_probe_model(folder, **overrides):
    cfg = dict(PROBE)
    cfg.update(overrides)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), probe_tensors(cfg),
                      metadata={"format": "pt"})
    return folder
