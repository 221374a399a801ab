"""MI355X-native sliding-window 2-simplicial attention (gfx950 HIP kernels behind the
Python API of lucidrains/simplicial-attention for that one path)."""
from .naive import naive_two_simplicial_attend, nth_order_attend, signed_determinant
from .simplicial_mha import HigherOrderAttention, TwoSimplicialMHA
from .two_simplicial_attention import (
    SlidingTwoSimplicialAttention,
    SlidingWindowTwoSimplicialMHA,
    sliding_two_simplicial_attn,
)

__all__ = [
    'naive_two_simplicial_attend',
    'nth_order_attend',
    'signed_determinant',
    'HigherOrderAttention',
    'TwoSimplicialMHA',
    'SlidingTwoSimplicialAttention',
    'SlidingWindowTwoSimplicialMHA',
    'sliding_two_simplicial_attn',
]
