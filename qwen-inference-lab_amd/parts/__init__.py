"""Parts that models are assembled from."""
from .base import (ParamSpec, KVNeed, PagedNeed, StateNeed, CompoundNeed, Part, Norm, PositionEncoding, Rotation,
                   Mixer, FeedForward, Block)
from .norm import RMSNorm, LayerNorm
from .rotary import Rotary, RotaryFrequencies
from .attention import Attention
from .latent_attention import LatentAttention
from .recurrent import MatrixMemory
from .mlp import GatedMLP, PlainMLP
from .conv import ShortConvolution
from .moe import RoutedExperts
from .ssm import SelectiveScan
from .parallel import ParallelMixers
from .block import PreNormBlock, SandwichBlock, PostNormBlock
from .embedding import Embedding, LMHead
from .model import CausalLM, ScheduleEntry

__all__ = ['ParamSpec', 'KVNeed', 'PagedNeed', 'StateNeed', 'CompoundNeed', 'Part', 'Norm', 'PositionEncoding', 'Rotation', 'Mixer',
           'FeedForward', 'Block', 'RMSNorm', 'LayerNorm', 'Rotary', 'RotaryFrequencies', 'Attention',
           'LatentAttention', 'MatrixMemory', 'GatedMLP', 'PlainMLP', 'ShortConvolution', 'RoutedExperts', 'SelectiveScan', 'ParallelMixers', 'PreNormBlock',
           'SandwichBlock', 'PostNormBlock',
           'Embedding', 'LMHead', 'CausalLM', 'ScheduleEntry']
