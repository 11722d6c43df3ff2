"""Registration of the parts that ship with the engine."""
from .base import register_part
from .norm import LayerNorm
from .position import LearnedPositions, NoPositions
from .embedding import TokenEmbedding, LMHead
from .feed_forward import DenseFeedForward
from .attention import PagedAttention
from .arrangement import PreNorm, PostNorm

register_part("norm", "layer_norm", LayerNorm)
register_part("position", "learned", LearnedPositions)
register_part("position", "none", NoPositions)
register_part("embedding", "token", TokenEmbedding)
register_part("head", "linear", LMHead)
register_part("feed_forward", "dense", DenseFeedForward)
register_part("mixer", "paged_attention", PagedAttention)
register_part("arrangement", "pre_norm", PreNorm)
register_part("arrangement", "post_norm", PostNorm)
