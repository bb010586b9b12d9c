"""The two tiny Qwen2 configurations every test uses.  They differ in every
size and option: layers, width, heads and groups, head size, intermediate size
(neither a multiple of 128), vocabulary (1000 is no power of two), rope base,
eps, tied or untied head, window."""
import os

from servelab_amd import Qwen2Config, write_random_model

TINY_A = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
    head_dim=16, intermediate_size=192, vocab_size=512, rope_theta=10000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=True, use_sliding_window=False,
    max_position_embeddings=256, torch_dtype="float32", eos_token_id=511)

TINY_B = dict(
    architectures=["Qwen2ForCausalLM"], model_type="qwen2",
    num_hidden_layers=3, hidden_size=128, num_attention_heads=4, num_key_value_heads=1,
    head_dim=32, intermediate_size=352, vocab_size=1000, rope_theta=1000000.0,
    rms_norm_eps=1e-5, tie_word_embeddings=False, use_sliding_window=True,
    sliding_window=16, max_window_layers=2, max_position_embeddings=512,
    torch_dtype="float32", eos_token_id=999)

TINY = {"A": TINY_A, "B": TINY_B}


def make_folder(tmp_path, which="A", seed=0, **overrides):
    raw = dict(TINY[which])
    raw.update(overrides)
    cfg = Qwen2Config.from_hf(raw)
    folder = os.path.join(str(tmp_path), f"tiny_{which}_{seed}")
    write_random_model(cfg, folder, seed=seed)
    return folder
