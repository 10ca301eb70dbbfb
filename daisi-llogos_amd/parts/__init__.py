"""Parts a layer is put together from; importing the package registers the built-in ones."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, OTHER_PARTS, POSITIONS, Block, FeedForward, GroupView, KVSpec, LayerCache,
                   Mixer, Norm, NormedRows, Part, PositionEncoding, Residual, Runtime, StateSpec, StepContext, TensorSpec, make,
                   register_block, register_feed_forward, register_mixer, register_norm, register_part, register_position)
from .linear import Linear
from .norm import LayerNorm, RMSNorm
from .rope import Rotary
from .attention import Attention
from .conv import CausalConv
from .wkv import WKV
from .latent_attention import LatentAttention
from .mlp import ActivatedMLP, SwiGLU
from .capped_attention import CappedAttention
from .moe import RoutedMoE, TableMoE
from .loop import LoopEntry
from .rglru import RGLRU
from .diff_attention import DiffAttention
from .block import OutputNormBlock, ParallelBlock, PostNormBlock, PreNormBlock, SandwichBlock
