"""Each part alone on the GPU against the plain functions, at sizes other than
the tiny models', in float32 and bfloat16; and a model whose run list names a
layer twice and lets a layer read another layer's cache."""
import math

import pytest
import torch

import plain_qwen2 as plain
from servelab_amd.cache import CacheManager, CachePool
from servelab_amd.engine import ModelRunner, StepEntry
from servelab_amd.engine.batch import pack_batch
from servelab_amd.engine.session import make_runtime
from servelab_amd.parts import (DecoderModel, GatedMLP, LayerCall, ModelSpec, NoPosition,
                                OutputHead, PagedAttention, PreNormBlock, RMSNorm,
                                RotaryPosition, TokenEmbedding)

pytestmark = pytest.mark.gpu
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def rt(request):
    return make_runtime(DTYPES[request.param]), request.param


def rand(*shape, scale=1.0, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def load(part, tensors, runtime):
    """Give a part its tensors (rounded to the activation dtype first, so that
    the plain side computes with the very same values)."""
    rounded = {n: t.to(runtime.act_dtype).float() if t.dim() > 1 else t for n, t in tensors.items()}
    part.load(rounded.__getitem__, runtime)
    return rounded


def rel(got, ref):
    return ((got.float().cpu() - ref).abs().max() / ref.abs().max()).item()


def test_rmsnorm_part(rt):
    runtime, name = rt
    norm = RMSNorm(200, 1e-5)
    assert norm.param_specs()["weight"].shape == (200,) and norm.param_specs()["weight"].init == "gain"
    w = load(norm, {"weight": 1 + 0.1 * rand(200)}, runtime)
    resid, delta = rand(9, 200, seed=1), rand(9, 200, seed=2).to(runtime.act_dtype)
    r = resid.cuda()
    got = norm.forward(r, delta.cuda())
    ref = plain.rms_norm(resid + delta.float(), w["weight"], 1e-5)
    assert rel(got, ref) < TOL[name] and rel(r, resid + delta.float()) < 1e-6
    rows = torch.tensor([8, 2], dtype=torch.int32).cuda()
    assert rel(norm.forward_rows(r, None, rows), plain.rms_norm(r.cpu()[[8, 2]], w["weight"], 1e-5)) < TOL[name]


def test_rotary_part(rt):
    runtime, _ = rt
    pos_part = RotaryPosition(48, 5000.0)
    pos_part.load(None, runtime)
    batch = type("B", (), {"positions": torch.tensor([0, 3, 77, 1000], dtype=torch.int32).cuda()})
    shared = {}
    tables = pos_part.tables(batch, shared)
    cos, sin = tables.cos, tables.sin
    ang = batch.positions.cpu().float()[:, None] * plain.rope_inv_freq(5000.0, 48)[None, :]
    assert (cos.cpu() - torch.cos(ang)).abs().max() < 1e-5 and (sin.cpu() - torch.sin(ang)).abs().max() < 1e-5
    assert pos_part.tables(batch, shared) is tables          # prepared once per step
    assert NoPosition().tables(batch, shared) is None
    with pytest.raises(ValueError):
        RotaryPosition(15, 1e4)


def test_gated_mlp_part(rt):
    runtime, name = rt
    ffn = GatedMLP(96, 200)
    t = load(ffn, {"gate_proj.weight": rand(200, 96, scale=0.1, seed=1),
                   "up_proj.weight": rand(200, 96, scale=0.1, seed=2),
                   "down_proj.weight": rand(96, 200, scale=0.1, seed=3)}, runtime)
    for rows in (3, 70):
        x = rand(rows, 96, seed=4).to(runtime.act_dtype)
        ref = plain.swiglu(x.float(), t["gate_proj.weight"], t["up_proj.weight"], t["down_proj.weight"])
        assert rel(runtime.ops.materialize(ffn.forward(x.cuda())), ref) < TOL[name]
    with pytest.raises(ValueError):
        GatedMLP(96, 200, activation="gelu")


def test_embedding_and_head_parts(rt):
    runtime, name = rt
    emb = TokenEmbedding(1000, 72)
    t = load(emb, {"weight": rand(1000, 72, seed=1)}, runtime)
    ids = torch.tensor([0, 999, 5], dtype=torch.int32).cuda()
    import types
    assert torch.equal(emb.forward(types.SimpleNamespace(ids=ids)).cpu(), t["weight"][[0, 999, 5]])
    x = rand(4, 72, seed=2).to(runtime.act_dtype)
    tied = OutputHead(1000, 72, tied_to=emb)
    assert tied.param_specs() == {}
    tied.load(None, runtime)
    got = tied.forward(x.cuda())
    assert got.dtype == torch.float32 and rel(got, x.float() @ t["weight"].T) < TOL[name]
    untied = OutputHead(1000, 72)
    u = load(untied, {"weight": rand(1000, 72, seed=3)}, runtime)
    assert rel(untied.forward(x.cuda()), x.float() @ u["weight"].T) < TOL[name]


def attention_tensors(nh, nkv, D, H, bias, seed=0):
    t = {"q_proj.weight": rand(nh * D, H, scale=0.1, seed=seed), "k_proj.weight": rand(nkv * D, H, scale=0.1, seed=seed + 1),
         "v_proj.weight": rand(nkv * D, H, scale=0.1, seed=seed + 2), "o_proj.weight": rand(H, nh * D, scale=0.1, seed=seed + 3)}
    if bias:
        t.update({"q_proj.bias": rand(nh * D, scale=0.1, seed=seed + 4), "k_proj.bias": rand(nkv * D, scale=0.1, seed=seed + 5),
                  "v_proj.bias": rand(nkv * D, scale=0.1, seed=seed + 6)})
    return t


def plain_attention_layer(x, t, nh, nkv, D, theta, window, scale):
    T = x.shape[0]
    zero = torch.zeros(1)
    q = (x @ t["q_proj.weight"].T + t.get("q_proj.bias", zero)).view(T, nh, D)
    k = (x @ t["k_proj.weight"].T + t.get("k_proj.bias", zero)).view(T, nkv, D)
    v = (x @ t["v_proj.weight"].T + t.get("v_proj.bias", zero)).view(T, nkv, D)
    pos = torch.arange(T)
    if theta is not None:
        inv = plain.rope_inv_freq(theta, D)
        q, k = plain.apply_rope(q, pos, inv), plain.apply_rope(k, pos, inv)
    o = plain.attention(q, k, v, scale, pos, pos, window)
    return o.reshape(T, nh * D) @ t["o_proj.weight"].T


@pytest.mark.parametrize("nh,nkv,D,bias,theta,window", [
    (6, 2, 48, True, 1e4, None), (5, 5, 32, False, 1e6, 24), (8, 1, 64, True, None, None),
    (3, 1, 16, True, 500.0, 7)])
def test_attention_part_in_portions(rt, nh, nkv, D, bias, theta, window):
    """The mixer alone over its own cache stream: a sequence fed in portions
    (position encoding rotary or none, with and without bias and window)."""
    runtime, name = rt
    H, T = 72, 75
    position = RotaryPosition(D, theta) if theta is not None else NoPosition()
    mixer = PagedAttention(H, nh, nkv, D, position, qkv_bias=bias, window=window, scale=0.3)
    t = load(mixer, attention_tensors(nh, nkv, D, H, bias), runtime)
    assert mixer.cache_spec().window == window and (("q_proj.bias" in mixer.param_specs()) == bias)
    manager = CacheManager({0: mixer.cache_spec()}, num_pages=8, page_size=16)
    pool = CachePool(manager, runtime.device, runtime.act_dtype)
    binding = pool.binding(0, True)
    x = rand(T, H, seed=9).to(runtime.act_dtype)
    ref = plain_attention_layer(x.float(), t, nh, nkv, D, theta, window, 0.3)
    manager.open("r")
    got, start = [], 0
    for n in (20, 1, 33, 2, 19):
        manager.grow("r", start + n)
        batch = pack_batch([StepEntry("r", [0] * n, [])], [start], [], manager, runtime.device)
        got.append(runtime.ops.materialize(
            mixer.forward(x[start:start + n].cuda().contiguous(), batch, binding, {})))
        manager.commit("r", start + n)
        start += n
    assert rel(torch.cat(got), ref) < TOL[name]


def test_block_part(rt):
    runtime, name = rt
    H, nh, nkv, D, I, T = 80, 4, 2, 32, 136, 40
    block = PreNormBlock(RMSNorm(H, 1e-6), PagedAttention(H, nh, nkv, D, RotaryPosition(D, 1e4)),
                         RMSNorm(H, 1e-6), GatedMLP(H, I))
    tensors = {"input_layernorm.weight": 1 + 0.1 * rand(H, seed=1), "post_attention_layernorm.weight": 1 + 0.1 * rand(H, seed=2)}
    tensors.update({"self_attn." + n: v for n, v in attention_tensors(nh, nkv, D, H, True, seed=3).items()})
    tensors.update({"mlp.gate_proj.weight": rand(I, H, scale=0.1, seed=11), "mlp.up_proj.weight": rand(I, H, scale=0.1, seed=12),
                    "mlp.down_proj.weight": rand(H, I, scale=0.1, seed=13)})
    assert set(block.param_specs()) == set(tensors)
    t = load(block, tensors, runtime)
    manager = CacheManager({0: block.cache_specs()[0]}, num_pages=4, page_size=16)
    pool = CachePool(manager, runtime.device, runtime.act_dtype)
    manager.open("r")
    manager.grow("r", T)
    batch = pack_batch([StepEntry("r", [0] * T, [])], [0], [], manager, runtime.device)
    h = rand(T, H, seed=20)
    pending = rand(T, H, scale=0.1, seed=21).to(runtime.act_dtype)
    resid = h.cuda()
    delta = runtime.ops.materialize(block.forward(resid, pending.cuda(), batch, [pool.binding(0, True)], {}))
    h0 = h + pending.float()
    att = {n[len("self_attn."):]: v for n, v in t.items() if n.startswith("self_attn.")}
    h1 = h0 + plain_attention_layer(plain.rms_norm(h0, t["input_layernorm.weight"], 1e-6), att,
                                    nh, nkv, D, 1e4, None, 1 / math.sqrt(D))
    ffn = plain.swiglu(plain.rms_norm(h1, t["post_attention_layernorm.weight"], 1e-6),
                       t["mlp.gate_proj.weight"], t["mlp.up_proj.weight"], t["mlp.down_proj.weight"])
    assert rel(resid, h1) < TOL[name]               # the stream after the mixer's add
    assert rel(delta, ffn) < TOL[name] * 2           # the feed-forward output, pending


def test_run_list_names_a_layer_twice_and_shares_a_cache(rt):
    """Order of layers as data: block 0 runs twice (two cache streams of its
    own), block 1 reads the stream that the first call of block 0 wrote."""
    runtime, name = rt
    H, nh, nkv, D, I, V, T = 64, 4, 2, 16, 96, 300, 45
    emb = TokenEmbedding(V, H)

    def block():
        return PreNormBlock(RMSNorm(H, 1e-6), PagedAttention(H, nh, nkv, D, RotaryPosition(D, 1e4)),
                            RMSNorm(H, 1e-6), GatedMLP(H, I))
    spec = ModelSpec(("emb.", emb), [("b0.", block()), ("b1.", block())],
                     [LayerCall(0, 0), LayerCall(1, 0, write=False), LayerCall(0, 1)],
                     ("norm.", RMSNorm(H, 1e-6)), ("head.", OutputHead(V, H, tied_to=emb)), V, H)
    assert sorted(spec.stream_specs()) == [0, 1]
    from servelab_amd.weights import random_tensors
    tensors = random_tensors(spec.param_specs(), seed=5, std=0.1)
    tensors = {n: (v.to(runtime.act_dtype).float() if v.dim() > 1 else v) for n, v in tensors.items()}
    model = DecoderModel(spec, runtime)
    model.load(tensors)
    runner = ModelRunner(model, num_pages=8, page_size=16)
    toks = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(1)).tolist()
    got = torch.cat([runner.step([StepEntry("r", toks[a:b], list(range(b - a)))])
                     for a, b in ((0, 17), (17, 18), (18, 45))])

    def layer(h, p, kv_from=None):
        x = plain.rms_norm(h, tensors[p + "input_layernorm.weight"], 1e-6)
        pos = torch.arange(T)
        inv = plain.rope_inv_freq(1e4, D)
        proj = lambda n, src: (src @ tensors[p + f"self_attn.{n}_proj.weight"].T
                               + tensors[p + f"self_attn.{n}_proj.bias"])
        q = plain.apply_rope(proj("q", x).view(T, nh, D), pos, inv)
        if kv_from is None:
            k = plain.apply_rope(proj("k", x).view(T, nkv, D), pos, inv)
            v = proj("v", x).view(T, nkv, D)
        else:
            k, v = kv_from
        o = plain.attention(q, k, v, 1 / math.sqrt(D), pos, pos)
        h = h + o.reshape(T, nh * D) @ tensors[p + "self_attn.o_proj.weight"].T
        x2 = plain.rms_norm(h, tensors[p + "post_attention_layernorm.weight"], 1e-6)
        h = h + plain.swiglu(x2, tensors[p + "mlp.gate_proj.weight"], tensors[p + "mlp.up_proj.weight"],
                             tensors[p + "mlp.down_proj.weight"])
        return h, (k, v)
    h = tensors["emb.weight"][toks]
    h, kv0 = layer(h, "b0.")
    h, _ = layer(h, "b1.", kv_from=kv0)
    h, _ = layer(h, "b0.")
    ref = plain.rms_norm(h, tensors["norm.weight"], 1e-6) @ tensors["emb.weight"].T
    assert rel(got, ref) < TOL[name] * 2
    with pytest.raises(ValueError, match="written by two"):
        ModelSpec(("emb.", emb), [("b0.", block())], [LayerCall(0, 0), LayerCall(0, 0)],
                  ("norm.", RMSNorm(H, 1e-6)), ("head.", OutputHead(V, H)), V, H).stream_specs()
