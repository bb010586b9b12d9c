"""Configuration and registry (no GPU)."""
import pytest

from servelab_amd import ConfigError, Qwen2Config
from servelab_amd.config import (CacheConfig, SchedulerConfig, register_architecture,
                                 registered_architectures, resolve_architecture)
from tiny_configs import TINY_A, TINY_B


def test_reads_every_key():
    c = Qwen2Config.from_hf(TINY_B, path="/x")
    assert (c.num_layers, c.hidden_size, c.num_heads, c.num_kv_heads, c.head_dim) == (3, 128, 4, 1, 32)
    assert (c.intermediate_size, c.vocab_size) == (352, 1000)
    assert c.rope_theta == 1e6 and c.rms_norm_eps == 1e-5
    assert c.tie_word_embeddings is False and c.max_position_embeddings == 512
    assert c.use_sliding_window and c.sliding_window == 16 and c.max_window_layers == 2
    assert c.eos_token_id == 999 and c.dtype == "float32" and c.path == "/x"
    assert c.num_query_groups == 4
    assert [c.layer_window(i) for i in range(3)] == [None, None, 16]
    a = Qwen2Config.from_hf(TINY_A)
    assert [a.layer_window(i) for i in range(2)] == [None, None]


def test_defaults_follow_the_reference():
    # servelab/config.py:55-72
    raw = {k: TINY_A[k] for k in ("hidden_size", "num_hidden_layers", "num_attention_heads",
                                  "intermediate_size", "vocab_size", "rms_norm_eps")}
    c = Qwen2Config.from_hf(raw)
    assert c.num_kv_heads == c.num_heads == 4
    assert c.head_dim == 64 // 4
    assert c.rope_theta == 1e6 and c.max_position_embeddings == 4096
    assert c.tie_word_embeddings is False and c.dtype == "float16" and c.eos_token_id == 0
    assert c.use_sliding_window is False and c.attention_bias is True


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "intermediate_size", "vocab_size", "rms_norm_eps"])
def test_missing_required_key_is_named(key):
    raw = dict(TINY_A)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        Qwen2Config.from_hf(raw)


@pytest.mark.parametrize("change,word", [
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"torch_dtype": "int8"}, "torch_dtype"), ({"vocab_size": "many"}, "vocab_size"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0,
                       "original_max_position_embeddings": 32768}}, "rope_scaling"),
    ({"rope_scaling": {"rope_type": "linear", "factor": 2.0}}, "rope_scaling"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, r"layer_types\[1\]"),
    ({"layer_types": ["full_attention"]}, "layer_types must list 2"),
    ({"layer_types": ["full_attention", "chunked_attention"]}, "chunked_attention"),
    ({"head_dim": 320}, "head_dim 320 is more than the attention kernels take")])
def test_impossible_values_are_refused(change, word):
    raw = dict(TINY_A)
    raw.update(change)
    with pytest.raises(ConfigError, match=word):
        Qwen2Config.from_hf(raw)


def test_keys_that_ask_for_what_is_computed_pass():
    raw = dict(TINY_B, rope_scaling=None,
               layer_types=["full_attention", "full_attention", "sliding_attention"])
    assert Qwen2Config.from_hf(raw) == Qwen2Config.from_hf(TINY_B)
    raw = dict(TINY_A, rope_scaling={"rope_type": "default"},
               layer_types=["full_attention", "full_attention"])
    assert Qwen2Config.from_hf(raw) == Qwen2Config.from_hf(TINY_A)
    # a window that use_sliding_window switches off is no window, whatever sliding_window says
    raw = dict(TINY_B, use_sliding_window=False, layer_types=["full_attention"] * 3)
    assert [Qwen2Config.from_hf(raw).layer_window(i) for i in range(3)] == [None] * 3
    with pytest.raises(ConfigError, match="contradicts"):
        Qwen2Config.from_hf(dict(TINY_B, layer_types=["full_attention"] * 3))


def test_round_trip_and_param_count():
    c = Qwen2Config.from_hf(TINY_B)
    assert Qwen2Config.from_hf(c.to_hf()) == c
    # tiny B: 785,856 parameters; tiny A (tied): 131,648
    assert c.num_params() == 785856
    assert Qwen2Config.from_hf(TINY_A).num_params() == 131648


def test_registry():
    assert "Qwen2ForCausalLM" in registered_architectures()
    assert resolve_architecture({"architectures": ["Qwen2ForCausalLM"]}).name == "Qwen2ForCausalLM"
    assert resolve_architecture({"model_type": "qwen2"}).name == "Qwen2ForCausalLM"
    with pytest.raises(ValueError, match="Qwen2ForCausalLM"):      # lists what is registered
        resolve_architecture({"architectures": ["MambaForCausalLM"]})
    with pytest.raises(ValueError, match="unsupported"):
        resolve_architecture({"model_type": "gpt2"})
    register_architecture("ToyForTest", lambda raw, path: raw, lambda cfg: None)
    assert resolve_architecture({"architectures": ["ToyForTest"]}).name == "ToyForTest"


def test_engine_configs_validate():
    assert CacheConfig().block_size == 16 and SchedulerConfig().max_num_batched_tokens == 2048
    with pytest.raises(ValueError):
        CacheConfig(block_size=24)
    with pytest.raises(ValueError):
        SchedulerConfig(policy="shortest")
    assert SchedulerConfig(policy="sjf-predicted").policy == "sjf-predicted"     # (servelab/config.py:93)
    with pytest.raises(ValueError):
        SchedulerConfig(max_num_seqs=0)
