from simplicial_attention_amd.naive import naive_two_simplicial_attend  # noqa: F401
