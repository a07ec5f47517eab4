"""Parts a layer is put together from.  Importing this package registers the built-in kinds."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward, Mixer, Norm, Part,
                   PartSpec, PositionEncoding, Registry, ResidualStream, Runtime, StepContext, WeightSpec, Workspace)
from .linear import Linear
from .norm import LayerNorm, RMSNorm
from .rope import Llama3RotaryEncoding, LongRotaryEncoding, RotaryEncoding, YarnRotaryEncoding
from .attention import GeneralAttention, GQAAttention, InfLLMv2Attention
from .latent_attention import LatentAttention
from .ssm import Mamba2Mixer
from .mlstm import MLSTMMixer
from .diff_attention import DifferentialAttention
from .delta import GatedDeltaMixer
from .parallel import ParallelMixer
from .linear_attention import DecayLinearAttention
from .ffn import GatedFFN, PolyNormFFN, RoutedExpertsFFN
from .block import HyperConnectionBlock, ParallelGatedBlock, ParallelScaledBlock, PreNormBlock, SandwichNormBlock
from .embedding import LMHead, TokenEmbedding
