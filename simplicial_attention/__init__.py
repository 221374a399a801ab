"""Import paths of lucidrains/simplicial-attention, served by the MI355X-native build.

``from simplicial_attention.triton_two_simplicial_attention import SlidingWindowTwoSimplicialMHA``
(the reference's README usage) resolves to the gfx950 implementation in
``simplicial_attention_amd``; nothing here contains code of its own.  The reference's
``__init__`` also exports the n-directional attends (simplicial_attention/__init__.py:1-15);
those operators are not part of the sliding-window path and are not provided.
"""
from simplicial_attention_amd import (
    HigherOrderAttention,
    TwoSimplicialMHA,
    naive_two_simplicial_attend,
    nth_order_attend,
    signed_determinant,
)

__all__ = ['naive_two_simplicial_attend', 'nth_order_attend', 'signed_determinant', 'TwoSimplicialMHA', 'HigherOrderAttention']
