"""More toy parts, defined here in the test and plugged into the framework
without touching its files: a feed-forward that routes every token to one of a
few small experts (router logits in float32), a position encoding that rotates
by interpolated positions, and one that rotates only the first channels of a
head, in interleaved pairs.  They sit in a model whose three layers have
different position encodings, feed-forwards and windows.  It is no model of
anyone's; it only exercises the part interfaces."""
import math
from dataclasses import dataclass

import pytest
import torch

import plain_qwen2 as plain
from servelab_amd import load_config, register_architecture, write_random_model
from servelab_amd.engine import ModelRunner, StepEntry
from servelab_amd.engine.session import load_model_on_device
from servelab_amd.parts import (FeedForward, GatedMLP, LayerCall, ModelSpec, NoPosition, OutputHead,
                                PagedAttention, ParamSpec, PositionEncoding, PreNormBlock, RMSNorm,
                                RotaryLayout, RotaryTables, TokenEmbedding)

pytestmark = pytest.mark.gpu


class TopOneExperts(FeedForward):
    """y_t = expert_{e(t)}(x_t), e(t) = argmax_e (x_t . r_e) with the router in
    float32; an expert is silu(x G^T) * (x U^T) D^T."""

    def __init__(self, hidden_size, intermediate_size, num_experts):
        self.h, self.i, self.n = hidden_size, intermediate_size, num_experts

    def param_specs(self):
        specs = {"router.weight": ParamSpec((self.n, self.h))}
        for e in range(self.n):
            specs[f"experts.{e}.gate.weight"] = ParamSpec((self.i, self.h))
            specs[f"experts.{e}.up.weight"] = ParamSpec((self.i, self.h))
            specs[f"experts.{e}.down.weight"] = ParamSpec((self.h, self.i))
        return specs

    def load(self, tensors, rt):
        self.rt = rt
        self.router = tensors("router.weight").to(rt.device, torch.float32)
        self.gate_up = [rt.linear_weight(torch.cat([tensors(f"experts.{e}.gate.weight"),
                                                    tensors(f"experts.{e}.up.weight")]))
                        for e in range(self.n)]
        self.down = [rt.linear_weight(tensors(f"experts.{e}.down.weight")) for e in range(self.n)]

    def forward(self, x):
        ops = self.rt.ops
        choice = torch.argmax(x.float() @ self.router.T, -1)
        y = torch.zeros_like(x)
        for e in range(self.n):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel():
                act = ops.silu_mul(ops.linear(x[rows].contiguous(), self.gate_up[e], None))
                y[rows] = ops.linear(act, self.down[e], None)
        return y


class InterpolatedRotary(PositionEncoding):
    """Rotary angles of positions scaled by a factor: position p rotates as p * factor."""

    def __init__(self, head_dim, theta, factor):
        self.head_dim, self.theta, self.factor = head_dim, theta, factor

    def layout(self):
        return RotaryLayout(self.head_dim)

    def load(self, tensors, rt):
        self.inv_freq = plain.rope_inv_freq(self.theta, self.head_dim).to(rt.device)

    def tables(self, batch, shared):
        ang = batch.positions.float()[:, None] * self.factor * self.inv_freq[None, :]
        return RotaryTables(torch.cos(ang), torch.sin(ang))


class PartialInterleavedRotary(PositionEncoding):
    """Only the first ``rot`` channels of a head turn, in pairs (2j, 2j + 1) by
    the angle p * theta^(-2j / rot); the other channels carry no position."""

    def __init__(self, rot, theta):
        self.rot, self.theta = rot, theta

    def layout(self):
        return RotaryLayout(self.rot, "interleaved")

    def load(self, tensors, rt):
        self.inv_freq = plain.rope_inv_freq(self.theta, self.rot).to(rt.device)

    def tables(self, batch, shared):
        ang = batch.positions.float()[:, None] * self.inv_freq[None, :]
        return RotaryTables(torch.cos(ang), torch.sin(ang))


@dataclass
class ToyPartsConfig:
    hidden_size: int = 64
    vocab_size: int = 157
    factor: float = 0.25
    head_dim: int = 16
    rot: int = 8
    dtype: str = "float32"
    architecture: str = "ToyRoutedForCausalLM"
    path: str = ""

    @classmethod
    def from_hf(cls, raw, path=""):
        return cls(raw["hidden_size"], raw["vocab_size"], raw["factor"], raw["head_dim"], raw["rot"],
                   raw.get("torch_dtype", "float32"), path=path)

    def to_hf(self):
        return {"architectures": [self.architecture], "hidden_size": self.hidden_size,
                "vocab_size": self.vocab_size, "factor": self.factor, "head_dim": self.head_dim,
                "rot": self.rot, "torch_dtype": self.dtype}


NH, NKV, W, EXPERTS, INTER = 4, 2, 8, 3, 40


def build_toy(cfg):
    h, D = cfg.hidden_size, cfg.head_dim
    first = PreNormBlock(RMSNorm(h, 1e-5),
                         PagedAttention(h, NH, NKV, D, InterpolatedRotary(D, 100.0, cfg.factor), qkv_bias=True),
                         RMSNorm(h, 1e-5), TopOneExperts(h, INTER, EXPERTS))
    second = PreNormBlock(RMSNorm(h, 1e-5),
                          PagedAttention(h, NH, NKV, D, NoPosition(), qkv_bias=False, window=W),
                          RMSNorm(h, 1e-5), GatedMLP(h, 72))
    third = PreNormBlock(RMSNorm(h, 1e-5),
                         PagedAttention(h, NH, NKV, D, PartialInterleavedRotary(cfg.rot, 50.0), qkv_bias=True),
                         RMSNorm(h, 1e-5), GatedMLP(h, 56))
    return ModelSpec(("tok.", TokenEmbedding(cfg.vocab_size, h)),
                     [("layers.0.", first), ("layers.1.", second), ("layers.2.", third)],
                     [LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2)], ("final_norm.", RMSNorm(h, 1e-5)),
                     ("out.", OutputHead(cfg.vocab_size, h)), cfg.vocab_size, h, eos_token_id=-1,
                     max_position_embeddings=4096)


def plain_toy(cfg, w, toks):
    T, h, D = len(toks), cfg.hidden_size, cfg.head_dim
    pos = torch.arange(T)
    x = w["tok.weight"][toks]
    p = "layers.0."
    n = plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
    ang = pos.float()[:, None] * cfg.factor * plain.rope_inv_freq(100.0, D)[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def rotate(t):
        a, b = t[..., :D // 2], t[..., D // 2:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
    q = rotate((n @ w[p + "self_attn.q_proj.weight"].T + w[p + "self_attn.q_proj.bias"]).view(T, NH, D))
    k = rotate((n @ w[p + "self_attn.k_proj.weight"].T + w[p + "self_attn.k_proj.bias"]).view(T, NKV, D))
    v = (n @ w[p + "self_attn.v_proj.weight"].T + w[p + "self_attn.v_proj.bias"]).view(T, NKV, D)
    x = x + plain.attention(q, k, v, 1 / math.sqrt(D), pos, pos).reshape(T, NH * D) @ w[p + "self_attn.o_proj.weight"].T
    n = plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
    choice = torch.argmax(n @ w[p + "mlp.router.weight"].T, -1)
    y = torch.zeros_like(n)
    for e in range(EXPERTS):
        rows = choice == e
        y[rows] = plain.swiglu(n[rows], w[p + f"mlp.experts.{e}.gate.weight"], w[p + f"mlp.experts.{e}.up.weight"],
                               w[p + f"mlp.experts.{e}.down.weight"])
    x = x + y
    p = "layers.1."
    n = plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
    q = (n @ w[p + "self_attn.q_proj.weight"].T).view(T, NH, D)
    k = (n @ w[p + "self_attn.k_proj.weight"].T).view(T, NKV, D)
    v = (n @ w[p + "self_attn.v_proj.weight"].T).view(T, NKV, D)
    x = x + plain.attention(q, k, v, 1 / math.sqrt(D), pos, pos, window=W).reshape(T, NH * D) @ w[p + "self_attn.o_proj.weight"].T
    x = x + plain.swiglu(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5), w[p + "mlp.gate_proj.weight"],
                         w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    p = "layers.2."
    n = plain.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5)
    ang = pos.float()[:, None] * plain.rope_inv_freq(50.0, cfg.rot)[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def turn(t):                                  # pairs (2j, 2j + 1) of the first rot channels
        a, b = t[..., 0:cfg.rot:2], t[..., 1:cfg.rot:2]
        out = t.clone()
        out[..., 0:cfg.rot:2], out[..., 1:cfg.rot:2] = a * cos - b * sin, b * cos + a * sin
        return out
    q = turn((n @ w[p + "self_attn.q_proj.weight"].T + w[p + "self_attn.q_proj.bias"]).view(T, NH, D))
    k = turn((n @ w[p + "self_attn.k_proj.weight"].T + w[p + "self_attn.k_proj.bias"]).view(T, NKV, D))
    v = (n @ w[p + "self_attn.v_proj.weight"].T + w[p + "self_attn.v_proj.bias"]).view(T, NKV, D)
    x = x + plain.attention(q, k, v, 1 / math.sqrt(D), pos, pos).reshape(T, NH * D) @ w[p + "self_attn.o_proj.weight"].T
    x = x + plain.swiglu(plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5), w[p + "mlp.gate_proj.weight"],
                         w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return plain.rms_norm(x, w["final_norm.weight"], 1e-5) @ w["out.weight"].T, choice


@pytest.mark.parametrize("head_dim,rot", [(16, 8), (32, 16), (48, 32)])
def test_routed_feed_forward_and_other_position_encodings(tmp_path, head_dim, rot):
    """(16, 8): the rotated width is no multiple of 16, so the kernel table leaves the channels in
    halves; (32, 16) and (48, 32): it lays them out in blocks of 8 and their partners."""
    register_architecture("ToyRoutedForCausalLM", ToyPartsConfig.from_hf, build_toy)
    folder = write_random_model(ToyPartsConfig(head_dim=head_dim, rot=rot), str(tmp_path / "toy"),
                                seed=5, std=0.15)
    cfg = load_config(folder)
    _, model = load_model_on_device(folder, "float32")
    runner = ModelRunner(model, num_pages=12, page_size=16, max_num_seqs=4)
    assert len(runner.manager.page_groups) == 2         # all keys for layers 0 and 2, a window of them for layer 1
    from safetensors.torch import load_file
    w = {k: v.float() for k, v in load_file(folder + "/model.safetensors").items()}
    gen = torch.Generator().manual_seed(1)
    seqs = {r: torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for r, n in (("a", 50), ("b", 37))}
    ref = {}
    for r, t in seqs.items():
        ref[r], choice = plain_toy(cfg, w, t)
        assert len(set(choice.tolist())) == EXPERTS     # every expert gets tokens
    plan = [[("a", 0, 17), ("b", 0, 2)], [("a", 17, 18), ("b", 2, 30)], [("a", 18, 50), ("b", 30, 31)],
            [("b", 31, 37)]]
    worst = 0.0
    for step in plan:
        out = runner.step([StepEntry(r, seqs[r][a:b], list(range(b - a))) for r, a, b in step])
        row = 0
        for r, a, b in step:
            worst = max(worst, (out[row:row + b - a].cpu() - ref[r][a:b]).abs().max().item())
            row += b - a
    assert worst < 1e-4, worst
    runner.manager.check()
