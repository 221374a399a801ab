"""Module name of the reference kept for drop-in imports; no Triton inside."""
from simplicial_attention_amd.two_simplicial_attention import (  # noqa: F401
    SlidingTwoSimplicialAttention,
    SlidingWindowTwoSimplicialMHA,
    _sliding_two_simplicial_attn,
    sliding_two_simplicial_attn,
)
