"""MI355X (gfx950) fused multi-head attention forward.

Two ways in, both ending in the same hand-written HIP kernel:

* ``fused_attn.attention_forward(head_dim, chunk_size, queries, keys, values, mask=None)`` --
  the compiled torch binding, a drop-in for the reference's extension module (reference
  src/fused_attn_extention.cu:119-129).  ``attention_forward`` is re-exported here.
* ``fused_attention_amd.capi`` -- a ctypes view of the C ABI declared in include/fused_attn.h,
  for callers that hold raw device pointers or a strided ``[B, R, L, H]`` tensor.

There is no CPU or eager fallback: if the kernel library or the binding has not been built
(``python -m fused_attention_amd.build``), importing the entry points raises.
"""
from . import capi  # noqa: F401


def attention_forward(head_dim, chunk_size, queries, keys, values, mask=None):
    """Fused multihead attention; see the module `fused_attn` (the compiled binding)."""
    import fused_attn  # the compiled extension built in-tree at the repository root

    return fused_attn.attention_forward(head_dim, chunk_size, queries, keys, values, mask)
