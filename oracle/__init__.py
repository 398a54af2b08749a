"""CPU oracle for the fused attention forward.  TEST INFRASTRUCTURE ONLY.

Nothing under this directory is part of the product: only tests/, the smoke() of
__graft_entry__.py and the cpu_baseline leg of bench.py may import it, and only as the checker
(or as the timed CPU baseline), never as the thing that computes a result handed to a user.
The product path (fused_attention_amd, module fused_attn) never falls back to it.
"""
from .naive_attention import (attention, attention_f64, attention_lse, attention_per_head,  # noqa: F401
                              causal_mask)
from .qkv_projection import qkv_projection, rope_tables, rotate_half  # noqa: F401
