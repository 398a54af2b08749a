"""Synthetic workloads of the fused attention forward: the five benchmark configurations.

Inputs are drawn on the host from a seeded torch.Generator in float32 and rounded to fp16, so
a host-side checker and the GPU see identical bits.  The logical tensor is [B, R, L, H]; the
drop-in entry point takes the [B, L, R*H] rearrangement (heads packed along the feature axis,
reference src/fused_attn_extention.cu:50-52 and include/fused_attn.cuh:683-690).
"""
from collections import namedtuple

import torch

Workload = namedtuple("Workload", "name B R L H q_std k_std v_std seed note")

# The seed base echoes the reference's test seed (reference tests/test_fused_attn.py:13).
WORKLOADS = {
    "c1": Workload("c1", 1, 4, 256, 64, 1.0, 1.0, 1.0, 179, "smoke"),
    "c2": Workload("c2", 8, 12, 1024, 64, 1.0, 1.0, 1.0, 180, "BERT-base-like"),
    "c3": Workload("c3", 4, 16, 4096, 64, 1.0, 1.0, 1.0, 181, "long sequence (headline)"),
    "c4": Workload("c4", 1, 32, 16384, 128, 0.5, 0.5, 0.5, 182, "LLaMA-7B-like head shape"),
    "c5a": Workload("c5a", 2, 8, 1000, 64, 3.0, 3.0, 1.0, 183, "ragged + large scores"),
    "c5b": Workload("c5b", 2, 8, 3073, 64, 3.0, 3.0, 1.0, 184, "ragged + large scores"),
    # the configuration of the reference's own benchmark (reference tests/benchmark_fused_attn.py:9-15)
    "readme": Workload("readme", 4, 40, 2048, 128, 1.0, 1.0, 1.0, 185, "reference benchmark shape"),
}


def flops(w):
    """Algorithmic work of one forward: two GEMMs of 2*L*L*H flop per (batch, head)."""
    return 4.0 * w.B * w.R * w.L * w.L * w.H


def io_bytes(w):
    """Algorithmic HBM traffic: Q, K, V read once and O written once, fp16."""
    return 4 * w.B * w.R * w.L * w.H * 2


def make_inputs(w, device="cpu"):
    """Returns (q, k, v) as fp16 [B, L, R*H] tensors on `device`, from distinct seeded streams."""
    out = []
    for i, std in enumerate((w.q_std, w.k_std, w.v_std)):
        gen = torch.Generator().manual_seed(w.seed * 1000 + i)
        x = torch.randn(w.B, w.R, w.L, w.H, generator=gen, dtype=torch.float32)
        if std != 1.0:
            x = x * std
        x = x.to(torch.float16).transpose(1, 2).reshape(w.B, w.L, w.R * w.H).contiguous()
        out.append(x.to(device))
    return tuple(out)


def to_bhld(x, head_dim):
    """[B, L, R*H] -> contiguous [B, R, L, H]."""
    B, L, F = x.shape
    return x.view(B, L, F // head_dim, head_dim).transpose(1, 2).contiguous()
