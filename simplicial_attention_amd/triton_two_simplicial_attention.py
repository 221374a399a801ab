"""Import-path alias: the reference exposes this operator as
``simplicial_attention.triton_two_simplicial_attention`` (README.md:19 there).
Nothing in this package uses Triton; the names below are the HIP implementation."""
from .two_simplicial_attention import (  # noqa: F401
    SlidingTwoSimplicialAttention,
    SlidingWindowTwoSimplicialMHA,
    _sliding_two_simplicial_attn,
    sliding_two_simplicial_attn,
)
