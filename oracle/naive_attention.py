"""CPU restatement of the reference's naive multi-head attention.  TEST INFRASTRUCTURE ONLY.

Restates reference tests/naive_implementation.py:4-18:
    split the feature axis into heads   (view(B, L, R, H).transpose(1, 2), :8-10)
    scores = (Q @ K^T) / sqrt(head_dim)                                   (:12)
    scores = softmax(scores, dim=-1)                                      (:13)
    output = scores @ V                                                   (:14)
    merge the heads back to [B, L, R*H]                                   (:16)
The reference function is dtype/device agnostic; the checker evaluates it in float32 on the
host (the fp16 inputs are upcast exactly), which is what the 5e-3 tolerance is quoted against.

What pins each function (none of it is "this file compared with itself"):
  attention           against torch.nn.functional.scaled_dot_product_attention (a library routine
                      with the same mathematical definition), against attention_f64 and against
                      oracle/attention_ref.c (an independent plain-C double-precision triple
                      loop) on seeded inputs, and against closed forms: Q = 0 gives the column
                      mean of V, constant V is returned unchanged, L = 1 returns V, one-hot
                      retrieval returns the selected row, permutation / shift / duplication
                      invariances.  See tests/test_oracle.py.
  attention_per_head  bit-for-bit identical arithmetic per (batch, head); pinned against
                      attention on shapes where both fit.
  attention_f64       numpy float64 brute force with explicit loops over (batch, head); pinned by
                      the same closed forms and by the C restatement.
The reference ships no golden vectors for this path (its tests draw inputs from the device RNG
at run time, reference tests/test_fused_attn.py:13,23-25), so there is no reference-held fixture
to check against; the reference's CUDA kernel cannot be built in an image without nvcc.
"""
import math

import numpy as np
import torch


def attention(queries, keys, values, head_dim, mask=None):
    """softmax(Q K^T / sqrt(head_dim) [+ mask]) V with heads packed along the last axis.

    queries, keys, values: [B, L, R*head_dim] tensors of any float dtype; evaluated in float32.
    mask: optional additive [B, L, L] tensor shared by all heads (reference README.md:88-89).
    Returns float32 [B, L, R*head_dim].  Same name and argument order as the reference function
    (reference tests/naive_implementation.py:4) so a test can import either.
    """
    batch_size, sequence_len, num_features = queries.shape
    num_heads = num_features // head_dim

    def split(x):
        return x.to(torch.float32).view(batch_size, sequence_len, num_heads, head_dim).transpose(1, 2)

    q, k, v = split(queries), split(keys), split(values)
    scores = (q @ k.mT) / (head_dim ** 0.5)
    if mask is not None:
        scores = scores + mask.to(torch.float32).view(batch_size, 1, sequence_len, sequence_len)
    scores = torch.softmax(scores, dim=-1)
    output = scores @ v
    return output.transpose(1, 2).contiguous().view(batch_size, sequence_len, num_features)


def attention_lse(queries, keys, head_dim, mask=None):
    """log(sum_j exp(score_ij)) of the scaled (and masked) scores, float32 [B, R, L].

    The row statistic a backward pass needs; the reference's kernel does not produce it
    (reference README.md:138-139 lists the backward pass as not done).  Pinned in
    tests/test_oracle.py by closed forms: zero queries give log(L), and exp(score - lse) are the
    softmax weights that reproduce `attention`.
    """
    batch_size, sequence_len, num_features = queries.shape
    num_heads = num_features // head_dim
    q = queries.to(torch.float32).view(batch_size, sequence_len, num_heads, head_dim).transpose(1, 2)
    k = keys.to(torch.float32).view(batch_size, sequence_len, num_heads, head_dim).transpose(1, 2)
    scores = (q @ k.mT) / (head_dim ** 0.5)
    if mask is not None:
        scores = scores + mask.to(torch.float32).view(batch_size, 1, sequence_len, sequence_len)
    return torch.logsumexp(scores, dim=-1)


def causal_mask(batch_size, sequence_len):
    """Additive [B, L, L] mask of a causal model: 0 where key <= query, -inf above the diagonal."""
    m = torch.full((sequence_len, sequence_len), float("-inf")).triu(1)
    return m.expand(batch_size, sequence_len, sequence_len).contiguous()


def attention_per_head(queries, keys, values, head_dim, heads=None, rows=None):
    """Same arithmetic as `attention`, one (batch, head) at a time.

    The one-shot form materialises two float32 [B, R, L, L] tensors (2 x 4 GiB at B=4, R=16,
    L=4096; 2 x 32 GiB at R=32, L=16384).  This form needs 2 x 4 L^2 bytes at a time.
    heads: optional iterable of (batch, head) pairs to evaluate; the others are left as NaN.
    rows: optional 1-D index tensor of query positions to evaluate (all keys are always used);
    the other rows are left as NaN.  Pinned against `attention` in tests/test_oracle.py.
    """
    batch_size, sequence_len, num_features = queries.shape
    num_heads = num_features // head_dim
    out = torch.full((batch_size, sequence_len, num_features), float("nan"), dtype=torch.float32)
    pairs = heads if heads is not None else [(b, h) for b in range(batch_size) for h in range(num_heads)]
    inv = 1.0 / (head_dim ** 0.5)
    for b, h in pairs:
        cols = slice(h * head_dim, (h + 1) * head_dim)
        q = queries[b, :, cols].to(torch.float32)
        k = keys[b, :, cols].to(torch.float32)
        v = values[b, :, cols].to(torch.float32)
        if rows is not None:
            q = q[rows]
        scores = torch.softmax((q @ k.mT) * inv, dim=-1)
        if rows is not None:
            out[b, rows, cols] = scores @ v
        else:
            out[b, :, cols] = scores @ v
    return out


def attention_f64(queries, keys, values, head_dim, mask=None):
    """numpy float64 brute force with explicit (batch, head) loops; for small shapes."""
    q = np.asarray(queries, dtype=np.float64)
    k = np.asarray(keys, dtype=np.float64)
    v = np.asarray(values, dtype=np.float64)
    batch_size, sequence_len, num_features = q.shape
    num_heads = num_features // head_dim
    out = np.empty_like(q)
    for b in range(batch_size):
        for h in range(num_heads):
            c0 = h * head_dim
            qh, kh, vh = q[b, :, c0:c0 + head_dim], k[b, :, c0:c0 + head_dim], v[b, :, c0:c0 + head_dim]
            s = qh @ kh.T / math.sqrt(head_dim)
            if mask is not None:
                s = s + np.asarray(mask, dtype=np.float64)[b]
            s = s - s.max(axis=1, keepdims=True)
            p = np.exp(s)
            out[b, :, c0:c0 + head_dim] = (p @ vh) / p.sum(axis=1, keepdims=True)
    return out
