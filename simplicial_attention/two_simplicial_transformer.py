from simplicial_attention_amd.two_simplicial_transformer import (  # noqa: F401
    Attention,
    FeedForward,
    TwoSimplicialTransformer,
)
