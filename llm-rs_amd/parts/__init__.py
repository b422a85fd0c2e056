from .base import (BLOCKS, FAMILIES, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Block, FeedForward, Mixer, Norm, Part,
                   PositionEncoding, TensorSpec, build_block, build_feed_forward, build_mixer, build_norm, build_part,
                   build_position, place, register_block, register_feed_forward, register_mixer, register_norm,
                   register_part_family, register_position)
from . import attention, block, hyper, latent, linear, mlp, norm, recurrent, rope  # noqa: F401  (register the built-in kinds)
from .attention import Attention
from .latent import LatentAttention
from .block import ParallelBlock, PreNormBlock, SandwichBlock
from .linear import MLSTM, DeltaRule, Lightning, Parallel
from .mlp import ClampedGLU, PlainFF, RoutedFF, SwiGLU
from .hyper import HyperBlock, HyperConnection
from .norm import DynamicTanh, GroupRMSNorm, LayerNorm, RMSNorm
from .recurrent import Mamba1, MinGRU
from .rope import RotaryEncoding, rope_inv_freq
