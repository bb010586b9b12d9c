from .base import (Block, Embedding, FeedForward, Mixer, Norm, PagedKVSpec, ParamSpec, Part,
                   PositionEncoding, RotaryLayout, RotaryTables, Runtime, StateSpec, prefixed)
from .norm import RMSNorm
from .position import NoPosition, RotaryPosition
from .attention import PagedAttention
from .feedforward import GatedMLP
from .block import PreNormBlock
from .embedding import OutputHead, TokenEmbedding
from .model import DecoderModel, LayerCall, ModelSpec, build_model_spec
