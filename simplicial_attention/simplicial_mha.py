from simplicial_attention_amd.simplicial_mha import HigherOrderAttention, TwoSimplicialMHA  # noqa: F401
