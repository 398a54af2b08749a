"""Lets a test say `from naive_implementation import attention`, as the reference's tests do
(reference tests/test_fused_attn.py:6).  The function is this repository's own CPU checker,
evaluated in float32; like the reference function (reference tests/naive_implementation.py:4-18,
every operation in the dtype of its inputs) it returns the dtype it was given, so that
`torch.testing.assert_close(actual, expected)` compares like with like."""
from oracle.naive_attention import attention as _attention_fp32


def attention(queries, keys, values, head_dim):
    return _attention_fp32(queries, keys, values, head_dim).to(queries.dtype)
