"""Lets a test say `from naive_implementation import attention`, as the reference's tests do
(reference tests/test_fused_attn.py:6); the function is this repository's own CPU checker."""
from oracle.naive_attention import attention  # noqa: F401
