from .base import (Part, Mixer, FeedForward, Norm, LazyNorm, ProjectionStep, Segment, StepContext, Workspace, lookup,
                   register_norm, register_position, register_mixer, register_feed_forward, register_block,
                   register_embedding, register_head, register_projection_step)
from . import norm, rotary, attention, mlp, embedding, block  # noqa: F401  (registers the built-in parts)
from .norm import RMSNorm
from .rotary import Rotary, rope_frequencies
from .attention import Attention
from .mlp import GatedMLP
from .embedding import Embedding, Head
from .block import PreNormBlock
