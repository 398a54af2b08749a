"""Pins the CPU oracle (oracle/) before anything is compared against it.  No GPU needed.

Each check is chosen so that a plausible mistake in the restatement fails it: a wrong head split
(columns of head h), a wrong scale (1/H instead of 1/sqrt(H)), softmax over the wrong axis, a
transposed operand, a mask applied to the wrong axis.
"""
import ctypes
import math
import os

import numpy as np
import pytest
import torch

from oracle import (attention, attention_f64, attention_lse, attention_per_head, causal_mask, qkv_projection,
                    rope_tables, rotate_half)

ORACLE_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")


def _rand(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(torch.float16)


def _c_oracle():
    path = os.path.join(ORACLE_DIR, "libattention_ref.so")
    if not os.path.exists(path):
        pytest.skip("oracle/libattention_ref.so not built (make -C oracle)")
    lib = ctypes.CDLL(path)
    fp = ctypes.POINTER(ctypes.c_float)
    lib.attention_ref_f64.argtypes = [fp, fp, fp, fp, ctypes.POINTER(ctypes.c_double)] + [ctypes.c_int64] * 4
    lib.attention_ref_f64.restype = ctypes.c_int
    return lib


def _run_c(q, k, v, head_dim, mask=None):
    lib = _c_oracle()
    B, L, F = q.shape
    arrs = [np.ascontiguousarray(t.float().numpy()) for t in (q, k, v)]
    fp = ctypes.POINTER(ctypes.c_float)
    m = np.ascontiguousarray(mask.float().numpy()) if mask is not None else None
    out = np.empty((B, L, F), dtype=np.float64)
    rc = lib.attention_ref_f64(*[a.ctypes.data_as(fp) for a in arrs],
                               m.ctypes.data_as(fp) if m is not None else None,
                               out.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), B, L, F // head_dim, head_dim)
    assert rc == 0
    return out


@pytest.mark.parametrize("B,R,L,H", [(1, 2, 32, 16), (2, 3, 77, 32), (1, 4, 256, 64), (1, 2, 130, 128)])
def test_against_plain_c_and_numpy_f64(B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 10 + i) for i in range(3))
    got = attention(q, k, v, H).double().numpy()
    ref_c = _run_c(q, k, v, H)
    ref_np = attention_f64(q.float().numpy(), k.float().numpy(), v.float().numpy(), H)
    np.testing.assert_allclose(ref_np, ref_c, rtol=0, atol=1e-12)
    np.testing.assert_allclose(got, ref_c, rtol=0, atol=2e-6)


@pytest.mark.parametrize("B,R,L,H", [(2, 4, 100, 64), (1, 3, 513, 32)])
def test_against_library_sdpa(B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 20 + i) for i in range(3))

    def split(x):
        return x.float().view(B, L, R, H).transpose(1, 2)

    lib = torch.nn.functional.scaled_dot_product_attention(split(q), split(k), split(v))
    lib = lib.transpose(1, 2).reshape(B, L, R * H)
    torch.testing.assert_close(attention(q, k, v, H), lib, rtol=0, atol=2e-6)


def test_per_head_form_is_the_same_arithmetic():
    B, R, L, H = 2, 3, 150, 64
    q, k, v = (_rand((B, L, R * H), 30 + i) for i in range(3))
    torch.testing.assert_close(attention_per_head(q, k, v, H), attention(q, k, v, H), rtol=0, atol=1e-6)
    part = attention_per_head(q, k, v, H, heads=[(1, 2)])
    assert torch.isnan(part[0]).all() and torch.isnan(part[1, :, : 2 * H]).all()
    torch.testing.assert_close(part[1, :, 2 * H:], attention(q, k, v, H)[1, :, 2 * H:], rtol=0, atol=1e-6)
    # a subset of the query rows: the same rows of the full answer, the others untouched
    rows = torch.tensor([0, 7, 64, 149])
    some = attention_per_head(q, k, v, H, heads=[(0, 1)], rows=rows)
    torch.testing.assert_close(some[0, rows, H:2 * H], attention(q, k, v, H)[0, rows, H:2 * H], rtol=0, atol=1e-6)
    assert torch.isnan(some).sum().item() == some.numel() - rows.numel() * H


def test_head_h_is_columns_hH_to_hH_plus_H():
    # V of head h is the constant h + 1: whatever the weights, head h's output columns equal h + 1.
    B, R, L, H = 1, 4, 19, 16
    q, k = _rand((B, L, R * H), 40), _rand((B, L, R * H), 41)
    v = torch.arange(1, R + 1, dtype=torch.float16).repeat_interleave(H).expand(B, L, R * H).contiguous()
    out = attention(q, k, v, H)
    want = torch.arange(1, R + 1, dtype=torch.float32).repeat_interleave(H).expand(B, L, R * H)
    torch.testing.assert_close(out, want, rtol=0, atol=1e-5)


def test_heads_and_batches_do_not_mix():
    B, R, L, H = 2, 3, 40, 32
    q, k, v = (_rand((B, L, R * H), 50 + i) for i in range(3))
    base = attention(q, k, v, H)
    q2, k2, v2 = q.clone(), k.clone(), v.clone()
    for t in (q2, k2, v2):
        t[0, :, H:2 * H] += 1.0   # disturb head 1 of batch 0 only
    out = attention(q2, k2, v2, H)
    assert torch.equal(out[0, :, :H], base[0, :, :H]) and torch.equal(out[0, :, 2 * H:], base[0, :, 2 * H:])
    assert torch.equal(out[1], base[1])
    assert not torch.equal(out[0, :, H:2 * H], base[0, :, H:2 * H])


@pytest.mark.parametrize("H", [16, 64])
def test_scale_is_one_over_sqrt_head_dim(H):
    # Two keys; q.k0 = a*b, q.k1 = 0  =>  weight on key 0 is sigmoid(a*b/sqrt(H)).
    a, b = 3.0, 2.0
    q = torch.zeros(1, 2, H, dtype=torch.float16)
    k = torch.zeros(1, 2, H, dtype=torch.float16)
    v = torch.zeros(1, 2, H, dtype=torch.float16)
    q[0, :, 0] = a
    k[0, 0, 0] = b
    v[0, 0, :] = 1.0
    v[0, 1, :] = -1.0
    w = 1.0 / (1.0 + math.exp(-a * b / math.sqrt(H)))
    out = attention(q, k, v, H)
    torch.testing.assert_close(out, torch.full_like(out, 2 * w - 1), rtol=0, atol=1e-6)


def test_zero_queries_give_the_column_mean_of_values():
    B, R, L, H = 2, 2, 333, 32
    k, v = _rand((B, L, R * H), 60), _rand((B, L, R * H), 61)
    out = attention(torch.zeros_like(k), k, v, H)
    want = v.float().mean(dim=1, keepdim=True).expand_as(out)
    torch.testing.assert_close(out, want, rtol=0, atol=1e-5)


def test_single_key_returns_values():
    q, k, v = (_rand((3, 1, 128), 70 + i) for i in range(3))
    assert torch.equal(attention(q, k, v, 64), v.float())


def test_one_hot_retrieval():
    # Keys are scaled basis vectors, query i is a large multiple of key pi(i): row i returns V[pi(i)].
    H = L = 32
    k = (torch.eye(L) * 8.0).to(torch.float16).view(1, L, H)
    perm = torch.randperm(L, generator=torch.Generator().manual_seed(5))
    q = (k[0, perm] * 4.0).view(1, L, H)            # score of the matching key: 256/sqrt(32) = 45
    v = _rand((1, L, H), 80)
    out = attention(q, k, v, H)
    torch.testing.assert_close(out[0], v[0, perm].float(), rtol=0, atol=1e-6)


def test_invariances_permutation_shift_duplication():
    B, R, L, H = 1, 2, 96, 32
    q, k, v = (_rand((B, L, R * H), 90 + i) for i in range(3))
    base = attention(q, k, v, H)
    perm = torch.randperm(L, generator=torch.Generator().manual_seed(6))
    torch.testing.assert_close(attention(q, k[:, perm], v[:, perm], H), base, rtol=0, atol=2e-6)
    # adding one vector to every key shifts each score row by a constant
    delta = _rand((1, 1, R * H), 93)
    torch.testing.assert_close(attention(q, (k.float() + delta.float()), v, H), base, rtol=0, atol=2e-5)
    # concatenating (K, V) with itself leaves the weighted mean unchanged
    dup = attention(q.repeat(1, 2, 1), k.repeat(1, 2, 1), v.repeat(1, 2, 1), H)
    torch.testing.assert_close(dup[:, :L], base, rtol=0, atol=2e-6)


def test_additive_mask_removes_keys():
    B, R, L, H = 2, 2, 50, 32
    q, k, v = (_rand((B, L, R * H), 100 + i) for i in range(3))
    keep = 17
    mask = torch.zeros(B, L, L, dtype=torch.float16)
    mask[:, :, keep:] = float("-inf")
    masked = attention(q, k, v, H, mask=mask)
    # the first `keep` query rows of the masked call see exactly the shortened problem
    short = attention(*(t[:, :keep].contiguous() for t in (q, k, v)), H)
    torch.testing.assert_close(masked[:, :keep], short, rtol=0, atol=2e-6)
    np.testing.assert_allclose(masked.double().numpy(), _run_c(q, k, v, H, mask=mask), rtol=0, atol=2e-6)


def test_lse_closed_forms():
    B, R, L, H = 2, 2, 37, 32
    q, k, v = (_rand((B, L, R * H), 110 + i) for i in range(3))
    # zero queries: every score is 0, so lse = log(L)
    lse0 = attention_lse(torch.zeros_like(q), k, H)
    torch.testing.assert_close(lse0, torch.full((B, R, L), math.log(L)), rtol=0, atol=1e-6)
    # exp(score - lse) are the softmax weights: they reproduce the attention output
    lse = attention_lse(q, k, H)
    qh = q.float().view(B, L, R, H).transpose(1, 2)
    kh = k.float().view(B, L, R, H).transpose(1, 2)
    vh = v.float().view(B, L, R, H).transpose(1, 2)
    w = torch.exp((qh @ kh.mT) / math.sqrt(H) - lse.unsqueeze(-1))
    torch.testing.assert_close(w.sum(-1), torch.ones(B, R, L), rtol=0, atol=1e-5)
    out = (w @ vh).transpose(1, 2).reshape(B, L, R * H)
    torch.testing.assert_close(out, attention(q, k, v, H), rtol=0, atol=1e-5)


def test_causal_mask_means_prefix_attention():
    # row i of the causal result equals the last row of the unmasked problem cut to i + 1 tokens
    B, R, L, H = 1, 2, 21, 16
    q, k, v = (_rand((B, L, R * H), 120 + i) for i in range(3))
    causal = attention(q, k, v, H, mask=causal_mask(B, L))
    for i in (0, 1, 7, L - 1):
        prefix = attention(*(t[:, :i + 1].contiguous() for t in (q, k, v)), H)
        torch.testing.assert_close(causal[:, i], prefix[:, i], rtol=0, atol=2e-6)


# ---- the rounding model of the kernels' probabilities, on the host ------------------------------

def _rtz_fp16(x):
    """float32 -> fp16 rounded toward zero (what v_cvt_pkrtz_f16_f32 does), for x >= 0."""
    h = x.to(torch.float16)
    up = h.float() > x
    bits = h.view(torch.int16) - up.to(torch.int16)
    return bits.view(torch.float16)


def _kernel_bias_log2(L):
    """The launcher's choice (fused_attn_capi.hip): 11 - ceil(log2 L), clamped to the limits the
    kernel header states."""
    import os
    import re

    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(here, "fused_attention_amd", "csrc", "fused_attn_kernel.hpp")).read()
    lo = float(re.search(r"constexpr float kBiasMin = (-?[0-9.]+)f;", text).group(1))
    hi = float(re.search(r"constexpr float kBiasMax = (-?[0-9.]+)f;", text).group(1))
    launcher = open(os.path.join(here, "fused_attention_amd", "csrc", "fused_attn_capi.hip")).read()
    assert "const float bias = 11.0f - (float)log2_len;" in launcher
    return min(hi, max(lo, 11.0 - math.ceil(math.log2(L))))


def test_rounding_model_of_small_weights():
    # The kernels round p = exp2(score - reference - bias) toward zero to fp16 before the second
    # product.  fp16 has normal numbers down to 2^-14 and subnormals down to 2^-24, so keys more
    # than 24 - bias log2 units below the reference vanish and keys in the ten units above that
    # are truncated.  Worst case over the gap: one dominant key and L - 1 keys `gap` below it; the
    # lost share of the row is at most (L - 1) 2^-(24 - bias).  With the bias the launcher picks
    # for a sequence length, that stays inside half the 5e-3 bound for values of magnitude 4 at
    # every length; a fixed bias of +6 (reference 64 times above the maximum) would not.
    def worst_error(L, bias, vmag=4.0):
        worst = 0.0
        for gap in torch.arange(8.0, 30.0, 0.25):
            p_tail = _rtz_fp16(torch.exp2(-gap - bias).reshape(1)).float().item()
            p_top = _rtz_fp16(torch.exp2(torch.tensor([-bias]))).float().item()
            got = (p_top * vmag - (L - 1) * p_tail * vmag) / (p_top + (L - 1) * p_tail)
            w = (L - 1) * 2.0 ** -gap.item()
            want = (vmag - w * vmag) / (1.0 + w)
            worst = max(worst, abs(got - want))
        return worst

    assert [_kernel_bias_log2(L) for L in (1, 64, 1000, 3073, 4096, 16384, 65536, 2 ** 22)] == [6, 5, 1, -1, -1, -3, -5, -8]
    for L in (64, 1000, 4096, 16384, 65536, 2 ** 19):
        assert worst_error(L, _kernel_bias_log2(L)) <= 2.5e-3
    assert worst_error(16384, 6.0) > 0.1          # what the bound protects against
    assert _rtz_fp16(torch.tensor([1.0 + 2.0 ** -11, 3.9999, 2.0 ** -25])).tolist() == [1.0, 3.998046875, 0.0]


# ---- the QKV projection front end and the rotary encoding ----------------------------------------

def test_projection_is_the_library_linear_map_and_its_slices_are_q_k_v():
    B, L, Fin, R, H = 2, 37, 96, 3, 32
    F = R * H
    x, w, b = _rand((B, L, Fin), 900), _rand((Fin, 3 * F), 901, 0.1), _rand((3 * F,), 902)
    got = qkv_projection(x, w, b, R, H)
    assert got.shape == (B, L, 3, F) and got.dtype == torch.float32
    lib = torch.nn.functional.linear(x.float(), w.float().T, b.float()).view(B, L, 3, F)
    torch.testing.assert_close(got, lib, rtol=1e-5, atol=1e-5)
    ref64 = (np.einsum("blk,kn->bln", x.double().numpy(), w.double().numpy()) + b.double().numpy()).reshape(B, L, 3, F)
    assert np.abs(got.numpy() - ref64).max() < 1e-4
    # slice s of the output uses columns [s F, (s + 1) F) of w
    for s in range(3):
        only = qkv_projection(x, w[:, s * F:(s + 1) * F].repeat(1, 3), None, R, H)
        torch.testing.assert_close(only[:, :, 0], got[:, :, s] - b.float()[s * F:(s + 1) * F], rtol=1e-5, atol=1e-5)


def test_projection_closed_forms():
    B, L, R, H = 1, 9, 2, 32
    F = R * H
    x = _rand((B, L, F), 910)
    eye3 = torch.eye(F).repeat(1, 3).half()
    out = qkv_projection(x, eye3, None, R, H)                      # identity weights: the input three times
    for s in range(3):
        assert torch.equal(out[:, :, s], x.float())
    w = torch.zeros(F, 3 * F)
    w[5, 0], w[7, F + 1], w[11, 2 * F + 2] = 1.0, 2.0, -1.0        # one-hot columns pick input features
    out = qkv_projection(x, w.half(), None, R, H)
    assert torch.equal(out[0, :, 0, 0], x[0, :, 5].float())
    assert torch.equal(out[0, :, 1, 1], 2.0 * x[0, :, 7].float())
    assert torch.equal(out[0, :, 2, 2], -x[0, :, 11].float())
    assert out.abs().sum() == out[0, :, 0, 0].abs().sum() + out[0, :, 1, 1].abs().sum() + out[0, :, 2, 2].abs().sum()


def test_rotary_encoding_is_a_rotation_of_feature_pairs():
    L, H = 50, 64
    cos, sin = rope_tables(L, H)
    assert torch.equal(cos[0], torch.ones(H // 2)) and torch.equal(sin[0], torch.zeros(H // 2))
    inv = 10000.0 ** (-2.0 * torch.arange(H // 2, dtype=torch.float64) / H)
    torch.testing.assert_close(cos[7].double(), torch.cos(7 * inv), rtol=0, atol=1e-6)
    y = _rand((3, L, H), 920).float()
    out = rotate_half(y, cos, sin)
    # an independent formulation: (y[i], y[i + H/2]) as a complex number, multiplied by exp(i theta)
    z = torch.complex(y[..., :H // 2].double(), y[..., H // 2:].double()) * torch.polar(
        torch.ones(L, H // 2, dtype=torch.float64), torch.atan2(sin.double(), cos.double()))
    torch.testing.assert_close(out.double(), torch.cat([z.real, z.imag], dim=-1), rtol=0, atol=1e-5)
    torch.testing.assert_close(out.norm(dim=-1), y.norm(dim=-1), rtol=1e-5, atol=1e-5)        # rotations keep norms
    assert torch.equal(rotate_half(y, torch.ones_like(cos), torch.zeros_like(sin)), y)
    # q at position m times k at position n depends on m - n only
    q, k = _rand((H,), 921).float(), _rand((H,), 922).float()

    def score(m, n):
        return (rotate_half(q, cos[m], sin[m]) * rotate_half(k, cos[n], sin[n])).sum()

    assert abs(score(9, 4) - score(25, 20)) < 1e-3 and abs(score(9, 4) - score(4, 9)) > 1e-3


def test_projection_rotates_q_and_k_heads_only():
    B, L, Fin, R, H = 2, 21, 64, 3, 16
    F = R * H
    x, w, b = _rand((B, L, Fin), 930), _rand((Fin, 3 * F), 931, 0.2), _rand((3 * F,), 932)
    cos, sin = rope_tables(L, H)
    plain = qkv_projection(x, w, b, R, H)
    rot = qkv_projection(x, w, b, R, H, cos, sin)
    assert torch.equal(rot[:, :, 2], plain[:, :, 2])                                        # v untouched
    torch.testing.assert_close(rot[:, 0], plain[:, 0], rtol=0, atol=1e-6)                   # position 0: no rotation
    for s in range(2):
        for h in range(R):
            want = rotate_half(plain[:, :, s, h * H:(h + 1) * H], cos.view(1, L, H // 2), sin.view(1, L, H // 2))
            torch.testing.assert_close(rot[:, :, s, h * H:(h + 1) * H], want, rtol=0, atol=1e-6)
