from .attention import PagedAttention
from .base import Block, FeedForward, Mixer, Norm, Part, PositionEncoding
from .block import DepthMix, OutputNormBlock, PreNormBlock
from .embedding import LMHead, PairHashEmbedding, TokenEmbedding
from .latent_attention import LatentAttention
from .mlp import DenseMLP, GatedMLP
from .norm import RMSNorm
from .recurrent import MinGRU
from .rotary import RotaryEmbedding
