"""CPU restatement of the fused QKV projection front end.  TEST INFRASTRUCTURE ONLY.

The reference has no code for this step: it lists "QKV projection" among the things not done
(reference README.md:137) and its kernel takes queries, keys and values as three separate
[B, L, R*H] tensors (reference src/fused_attn_extention.cu:15-22, tests/naive_implementation.py:8-10
splits each into heads).  What is restated here is therefore the textbook operation a caller would
place in front of that kernel: one linear map from the hidden state to the concatenation of q, k and
v, and the rotary position encoding of q and k in its rotate-half form.

What pins each function (tests/test_oracle.py):
  qkv_projection  the linear part against torch.nn.functional.linear (a library routine) and a
                  numpy float64 einsum; identity weights return the input three times; one-hot
                  weight columns select input features; the bias lands on its slice.
  rotate_half     against multiplication by exp(i theta) of the complex number y[i] + 1j y[i + H/2]
                  (an independent formulation); cos = 1, sin = 0 is the identity; norms are kept;
                  the product of a rotated q and a rotated k depends on the positions only through
                  their difference.
  rope_tables     position 0 gives cos = 1, sin = 0; angles are pos * base^(-2 i / H).
"""
import torch


def rope_tables(seq_len, head_dim, base=10000.0):
    """cos and sin of pos * base^(-2 i / head_dim), float32 [seq_len, head_dim / 2] each."""
    i = torch.arange(head_dim // 2, dtype=torch.float64)
    inv_freq = base ** (-2.0 * i / head_dim)
    angle = torch.arange(seq_len, dtype=torch.float64)[:, None] * inv_freq[None, :]
    return torch.cos(angle).to(torch.float32), torch.sin(angle).to(torch.float32)


def rotate_half(y, cos, sin):
    """Rotary encoding of head vectors y [..., L, H] with tables [L, H / 2]:
    out[..., :H/2] = y1 cos - y2 sin, out[..., H/2:] = y2 cos + y1 sin, (y1, y2) the two halves of y."""
    half = y.shape[-1] // 2
    y1, y2 = y[..., :half], y[..., half:]
    return torch.cat([y1 * cos - y2 * sin, y2 * cos + y1 * sin], dim=-1)


def qkv_projection(x, w, bias, num_heads, head_dim, rope_cos=None, rope_sin=None):
    """x [B, L, F_in] times w [F_in, 3 F] (+ bias [3 F]) in float32 -> [B, L, 3, F], F = num_heads *
    head_dim, with the rotary encoding applied to every head of the q and k slices when tables
    (float32 [L, head_dim / 2]) are given."""
    B, L, _ = x.shape
    F = num_heads * head_dim
    y = x.to(torch.float32) @ w.to(torch.float32)
    if bias is not None:
        y = y + bias.to(torch.float32)
    y = y.view(B, L, 3, num_heads, head_dim)
    if rope_cos is not None:
        cos = rope_cos.view(1, L, 1, 1, head_dim // 2)
        sin = rope_sin.view(1, L, 1, 1, head_dim // 2)
        y = torch.cat([rotate_half(y[:, :, :2], cos, sin), y[:, :, 2:]], dim=2)
    return y.reshape(B, L, 3, F)
