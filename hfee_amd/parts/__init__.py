from .base import (Part, Mixer, FeedForward, Norm, LazyNorm, ProjectionStep, Segment, StepContext, Workspace, lookup,
                   register_norm, register_position, register_mixer, register_feed_forward, register_block,
                   register_embedding, register_head, register_projection_step)
from . import (norm, rotary, attention, kv_attention, mix_attention, recurrent, mlp, moe, embedding,  # noqa: F401
               block, paired)       # (registers the built-in parts)
from .norm import LayerNorm, RMSNorm
from .rotary import Rotary, rope_frequencies
from .attention import Attention
from .mlp import DenseMLP, GatedMLP
from .kv_attention import KvAttention, LatentAttention, SigmoidAttention, WindowAttention
from .embedding import Embedding, Head
from .mix_attention import MixedAttention
from .recurrent import GatedDelta, GatedLinearAttention, RealGatedRecurrentUnit, Retention, StateSpace
from .paired import SideBySide
from .moe import RoutedMoE, TableMoE
from .block import ParallelBlock, PreNormBlock, SandwichBlock
