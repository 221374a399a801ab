from simplicial_attention_amd.naive import naive_two_simplicial_attend, nth_order_attend, signed_determinant  # noqa: F401
