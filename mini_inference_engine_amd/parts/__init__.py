from .attention import Attention
from .base import (BLOCKS, CombinedCache, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheBinding, CacheRequirement, DecoderSpec,
                   FeedForward, FixedState, LayerCall, Mixer, Norm, PagedKV, ParamSpec, Part, PositionEncoding,
                   Source, WEIGHT_TRANSFORMS, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding, register_weight_transform)
from .block import BranchNormBlock, ParallelBlock, PreNormBlock, SandwichBlock
from .delta_rule import DeltaRule
from .dense_ff import DenseFF
from .embedding import Embedding, LMHead
from .gla import GatedLinearAttention
from .input_conv import ConvTail, ResidualConv
from .latent_attention import LatentAttention, PagedLatent
from .layernorm import LayerNorm
from .rglru import RGLRU, RecurrentState
from .rmsnorm import RMSNorm
from .rope import NoPosition, RotaryHalfAngles, RotaryHalfSplit, RotaryInterleaved, rotary_tables
from .routed_experts import RoutedExperts
from .side_by_side import SideBySide
from .sigmoid_attention import SigmoidAttention
from .softmax_attention import SoftmaxAttention
from .summed_ff import SummedFF
from .swiglu import SwiGLU
