from .attention import PagedAttention
from .base import Block, FeedForward, Mixer, Norm, Part, PositionEncoding
from .block import DepthMix, OutputNormBlock, ParallelBlock, PassEntry, PreNormBlock, ResultGate
from .embedding import LMHead, PairHashEmbedding, TokenEmbedding
from .latent_attention import LatentAttention
from .mlp import DenseMLP, GatedMLP, MoEMLP
from .norm import RMSNorm
from .recurrent import ChannelDelta, HeadDelta, MinGRU, MLSTM, TimeMix
from .rotary import RotaryEmbedding
from .side_by_side import SideBySide
