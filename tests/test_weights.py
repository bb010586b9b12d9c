"""Safetensors reading and writing, kept dtypes, the one error for a checkpoint
that does not match, random-weights folders (no GPU)."""
import json
import os

import pytest
import torch

import plain_qwen2 as plain
from servelab_amd import Qwen2Config, WeightError, load_config, load_model, write_random_model
from servelab_amd.parts import DecoderModel, Runtime, build_model_spec
from servelab_amd.weights import (Checkpoint, SafetensorsFile, check_tensors, keep_dtype,
                                  write_safetensors)
from emulated_ops import EmulatedOps
from tiny_configs import TINY, TINY_A, TINY_B, make_folder


def test_container_round_trip_and_foreign_reader(tmp_path):
    tensors = {"a": torch.randn(3, 5), "b": torch.arange(7, dtype=torch.int64),
               "c": torch.randn(4, 4).to(torch.bfloat16), "d": torch.randn(2).to(torch.float16),
               "e": torch.zeros(0, 3)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors, metadata={"k": "v"})
    f = SafetensorsFile(path)
    assert f.metadata == {"k": "v"} and set(f.names()) == set(tensors)
    for n, t in tensors.items():
        assert f.tensor(n).dtype == t.dtype and torch.equal(f.tensor(n), t)
    from safetensors.torch import load_file, save_file       # the package reads our file
    theirs = load_file(path)
    assert all(torch.equal(theirs[n], t) for n, t in tensors.items())
    save_file({n: t.contiguous() for n, t in tensors.items() if t.numel()},
              str(tmp_path / "y.safetensors"))                # and we read the package's file
    g = SafetensorsFile(str(tmp_path / "y.safetensors"))
    assert all(torch.equal(g.tensor(n), tensors[n]) for n in g.names())


def test_kept_dtypes():
    assert keep_dtype(torch.zeros(2, dtype=torch.bfloat16)).dtype == torch.bfloat16
    assert keep_dtype(torch.zeros(2, dtype=torch.float16)).dtype == torch.bfloat16
    assert keep_dtype(torch.zeros(2, dtype=torch.float32)).dtype == torch.float32
    assert keep_dtype(torch.zeros(2, dtype=torch.int64)).dtype == torch.int32


def test_truncated_file_is_refused(tmp_path):
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, {"a": torch.randn(8, 8)})
    data = open(path, "rb").read()
    open(path, "wb").write(data[:-16])
    with pytest.raises(ValueError, match="byte range|file size"):
        SafetensorsFile(path)


def test_random_folder_is_reproducible_and_loads(tmp_path):
    f1 = make_folder(tmp_path / "1", "B", seed=7)
    f2 = make_folder(tmp_path / "2", "B", seed=7)
    f3 = make_folder(tmp_path / "3", "B", seed=8)
    a, b, c = Checkpoint(f1).state_dict(), Checkpoint(f2).state_dict(), Checkpoint(f3).state_dict()
    assert set(a) == set(b) and all(torch.equal(a[n], b[n]) for n in a)
    assert any(not torch.equal(a[n], c[n]) for n in a)
    cfg, state = load_model(f1)
    assert isinstance(cfg, Qwen2Config) and cfg.path == f1
    assert state["model.layers.2.self_attn.q_proj.bias"].abs().max() > 0        # biases are not zero
    gains = state["model.norm.weight"]
    assert abs(gains.mean().item() - 1) < 0.05 and gains.std().item() > 0.01
    assert abs(state["model.embed_tokens.weight"].std().item() - 0.02) < 0.002
    assert "lm_head.weight" in state
    tied = Checkpoint(make_folder(tmp_path / "4", "A", seed=1)).shapes()
    assert "lm_head.weight" not in tied
    assert json.load(open(os.path.join(f1, "config.json")))["sliding_window"] == 16
    assert load_config(f1) == Qwen2Config.from_hf(TINY_B, path=f1)


def test_bfloat16_folder_keeps_bfloat16(tmp_path):
    folder = make_folder(tmp_path, "A", seed=1, torch_dtype="bfloat16")
    state = Checkpoint(folder).state_dict()
    assert all(t.dtype == torch.bfloat16 for t in state.values())


def _model(which):
    cfg = Qwen2Config.from_hf(TINY[which])
    return DecoderModel(build_model_spec(cfg), Runtime(EmulatedOps(), "cpu", torch.float32))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_folder(tmp_path, "B", seed=3)
    state = Checkpoint(folder).state_dict()
    del state["model.layers.1.mlp.up_proj.weight"]
    del state["model.norm.weight"]
    state["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(4)
    state["model.layers.2.self_attn.k_proj.bias"] = torch.zeros(33)
    state["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)     # ignorable
    with pytest.raises(WeightError) as e:
        _model("B").load(state)
    msg = str(e.value)
    assert "missing (2)" in msg and "model.layers.1.mlp.up_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected (1)" in msg and "q_norm" in msg and "inv_freq" not in msg
    assert "wrong shape (1)" in msg and "expected [32] found [33]" in msg


def test_tied_head_ignores_a_stray_lm_head_but_untied_needs_it(tmp_path):
    folder = make_folder(tmp_path, "A", seed=3)
    state = Checkpoint(folder).state_dict()
    state["lm_head.weight"] = torch.zeros(512, 64)
    _model("A").load(state)                                   # servelab/parallel/tp_model.py:112-113
    state_b = Checkpoint(make_folder(tmp_path, "B", seed=3)).state_dict()
    del state_b["lm_head.weight"]
    with pytest.raises(WeightError, match="lm_head.weight"):
        _model("B").load(state_b)


def test_missing_files(tmp_path):
    with pytest.raises(WeightError, match="config.json"):
        load_config(str(tmp_path))
    folder = make_folder(tmp_path, "A")
    os.remove(os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError, match="model.safetensors"):
        Checkpoint(folder)


def test_sharded_checkpoint(tmp_path):
    folder = make_folder(tmp_path, "A", seed=5)
    state = Checkpoint(folder).state_dict()
    names = list(state)
    half = len(names) // 2
    shards = {"model-1.safetensors": names[:half], "model-2.safetensors": names[half:]}
    for fname, ns in shards.items():
        write_safetensors(os.path.join(folder, fname), {n: state[n] for n in ns})
    os.remove(os.path.join(folder, "model.safetensors"))
    json.dump({"weight_map": {n: f for f, ns in shards.items() for n in ns}},
              open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    again = Checkpoint(folder).state_dict()
    assert all(torch.equal(again[n], state[n]) for n in state)
