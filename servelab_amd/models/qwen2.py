"""Qwen2 dense decoder, assembled from parts.

Reference: ``TPDecoderModel`` with world size 1
(servelab/parallel/tp_model.py:80-134): embedding, L pre-norm blocks of
(RMSNorm, GQA attention with q/k/v bias and rotary positions, RMSNorm, SwiGLU),
final RMSNorm, tied or untied head.  Checkpoint names are the reference's
(tests/helpers_tiny_model.py:34-50).  Layers at or above max_window_layers get
a sliding window when use_sliding_window is set (this build's rule).
"""
from ..config import Qwen2Config, register_architecture
from ..parts.attention import PagedAttention
from ..parts.block import PreNormBlock
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.feedforward import GatedMLP
from ..parts.model import LayerCall, ModelSpec
from ..parts.norm import RMSNorm
from ..parts.position import RotaryPosition


def build_qwen2(cfg: Qwen2Config) -> ModelSpec:
    embedding = TokenEmbedding(cfg.vocab_size, cfg.hidden_size)
    layers = []
    for i in range(cfg.num_layers):
        block = PreNormBlock(
            RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
            PagedAttention(cfg.hidden_size, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim,
                           RotaryPosition(cfg.head_dim, cfg.rope_theta),
                           qkv_bias=cfg.attention_bias, window=cfg.layer_window(i)),
            RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
            GatedMLP(cfg.hidden_size, cfg.intermediate_size, cfg.hidden_act))
        layers.append((f"model.layers.{i}.", block))
    head = OutputHead(cfg.vocab_size, cfg.hidden_size,
                      tied_to=embedding if cfg.tie_word_embeddings else None)
    return ModelSpec(
        embedding=("model.embed_tokens.", embedding),
        layers=layers,
        run=[LayerCall(i, i) for i in range(cfg.num_layers)],
        final_norm=("model.norm.", RMSNorm(cfg.hidden_size, cfg.rms_norm_eps)),
        head=("lm_head.", head),
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        eos_token_id=cfg.eos_token_id,
        max_position_embeddings=cfg.max_position_embeddings,
        optional_tensors=("lm_head.weight",) if cfg.tie_word_embeddings else (),
    )


register_architecture("Qwen2ForCausalLM", Qwen2Config.from_hf, build_qwen2, model_type="qwen2")
