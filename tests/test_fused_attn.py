"""GPU parity of the fused attention forward against the CPU oracle.

Mirrors the reference's test strategy (reference tests/test_fused_attn.py:12-67: one case per
legal (head_dim, chunk_size), B=1, two heads, two chunks, seed 179, N(0,1) inputs) and adds what
the reference never tested: batch > 1, more than two heads, many key tiles, sequence lengths that
are not tile multiples, large-magnitude scores, closed-form answers and the strided C-ABI entry.

Tolerance: max |fused.float() - oracle_fp32| <= 5e-3 and every output finite.  The reference's
own bound (rtol = atol = 1e-2, tests/test_fused_attn.py:30) is checked as well in the drop-in cases.
"""
import math

import pytest
import torch

from fused_attention_amd import capi, workloads
from oracle import attention, attention_lse, attention_per_head, causal_mask

pytestmark = pytest.mark.gpu

TOL = 5e-3


def _max_err(got, want):
    got = got.float().cpu()
    assert torch.isfinite(got).all(), "non-finite output"
    return (got - want).abs().max().item()


def _rand(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(torch.float16)


# ---- the reference's 12 (head_dim, chunk_size) cases, through the torch binding ---------------

LEGAL = [(16, 16), (16, 32), (32, 16), (32, 32), (32, 64), (64, 16), (64, 32), (64, 64), (64, 128),
         (128, 32), (128, 64), (128, 128)]


@pytest.mark.parametrize("head_dim,chunk_size", LEGAL)
def test_simple(gpu, head_dim, chunk_size):
    import fused_attn

    torch.random.manual_seed(179)
    batch_size, num_heads, num_chunks = 1, 2, 2
    num_features = num_heads * head_dim
    sequence_len = num_chunks * chunk_size
    queries, keys, values = (torch.randn(batch_size, sequence_len, num_features).half() for _ in range(3))

    expected = attention(queries, keys, values, head_dim)
    actual = fused_attn.attention_forward(head_dim, chunk_size, queries.to(gpu), keys.to(gpu), values.to(gpu))

    assert actual.shape == queries.shape and actual.dtype == torch.float16 and actual.device.type == "cuda"
    torch.testing.assert_close(actual.float().cpu(), expected, rtol=0.01, atol=0.01)
    assert _max_err(actual, expected) <= TOL


def test_reference_test_body_through_the_shim(gpu):
    # The body of the reference's run_simple_test (reference tests/test_fused_attn.py:12-30) with
    # its own imports: `import fused_attn`, `from naive_implementation import attention`, and
    # assert_close on the two fp16 tensors as they come.
    import os
    import sys

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    try:
        from naive_implementation import attention as shim_attention
    finally:
        sys.path.pop(0)
    import fused_attn

    head_dim, chunk_size = 64, 64
    torch.random.manual_seed(179)
    queries, keys, values = (torch.randn(1, 2 * chunk_size, 2 * head_dim).half().to(gpu) for _ in range(3))
    expected = shim_attention(queries.cpu(), keys.cpu(), values.cpu(), head_dim)
    actual = fused_attn.attention_forward(head_dim, chunk_size, queries, keys, values)
    assert expected.dtype == actual.dtype == torch.float16
    torch.testing.assert_close(actual.cpu(), expected, rtol=0.01, atol=0.01)


# ---- benchmark configurations -------------------------------------------------------------------

@pytest.mark.parametrize("name", ["c1", "c2", "c5a", "c5b"])
def test_config_full_tensor(gpu, name):
    import fused_attn

    w = workloads.WORKLOADS[name]
    q, k, v = workloads.make_inputs(w)
    want = attention_per_head(q, k, v, w.H)
    got = fused_attn.attention_forward(w.H, 64, q.to(gpu), k.to(gpu), v.to(gpu))
    assert _max_err(got, want) <= TOL
    if name.startswith("c5"):
        # the stress inputs really do reach large scores
        s = (q[0, :, :w.H].float() @ k[0, :, :w.H].float().T) / math.sqrt(w.H)
        assert s.abs().max() > 20


def test_config_c3_headline(gpu):
    import fused_attn

    w = workloads.WORKLOADS["c3"]
    q, k, v = workloads.make_inputs(w)
    got = fused_attn.attention_forward(w.H, 64, q.to(gpu), k.to(gpu), v.to(gpu)).float().cpu()
    assert torch.isfinite(got).all()
    # every row of a third of the (batch, head) pairs, spread over batches and heads
    pairs = [(b, h) for b in range(w.B) for h in range(w.R) if (b * w.R + h) % 3 == 0]
    want = attention_per_head(q, k, v, w.H, heads=pairs)
    sel = ~torch.isnan(want)
    assert (got[sel] - want[sel]).abs().max().item() <= TOL
    # size-independent property on the whole tensor: a convex combination stays inside the range of V
    vmax = v.float().view(w.B, w.L, w.R, w.H).abs().amax(dim=1, keepdim=True).expand(w.B, w.L, w.R, w.H)
    assert (got.view(w.B, w.L, w.R, w.H).abs() <= vmax + 1e-3).all()


def _sample_rows(L, n, seed):
    """Query positions to check: the first and last rows of the sequence (first and last query
    tiles, wave boundaries) and a seeded sample of the rest."""
    g = torch.Generator().manual_seed(seed)
    edge = torch.cat([torch.arange(0, min(L, 96)), torch.arange(max(0, L - 96), L)])
    rand = torch.randperm(L, generator=g)[:n]
    return torch.unique(torch.cat([edge, rand]))


def _check_whole_tensor_without_an_oracle(forward, q, k, v, w, got, gpu):
    """Two checks that touch every (batch, head, row): a convex combination stays inside the range
    of the head's values, and zero queries return the mean of the head's values."""
    vh = v.float().view(w.B, w.L, w.R, w.H)
    vmax = vh.abs().amax(dim=1, keepdim=True).expand(w.B, w.L, w.R, w.H)
    assert (got.view(w.B, w.L, w.R, w.H).abs() <= vmax + 1e-3).all()
    flat = forward(torch.zeros_like(q).to(gpu), k.to(gpu), v.to(gpu)).float().cpu()
    mean = vh.mean(dim=1, keepdim=True).expand(w.B, w.L, w.R, w.H)
    assert (flat.view(w.B, w.L, w.R, w.H) - mean).abs().max().item() <= 2e-3


def test_config_c4_sampled_heads(gpu):
    import fused_attn

    w = workloads.WORKLOADS["c4"]
    q, k, v = workloads.make_inputs(w)

    def forward(q, k, v):
        return fused_attn.attention_forward(w.H, 128, q, k, v)

    got = forward(q.to(gpu), k.to(gpu), v.to(gpu)).float().cpu()
    assert torch.isfinite(got).all()
    # Eight heads, one per residue modulo 8 (the kernel renumbers workgroups per XCD, so a mistake
    # there would depend on the head): ~2200 rows of each, every key.
    pairs = [(0, h) for h in (0, 5, 10, 15, 16, 21, 26, 31)]
    rows = _sample_rows(w.L, 2048, 4)
    want = attention_per_head(q, k, v, w.H, heads=pairs, rows=rows)
    sel = ~torch.isnan(want)
    assert sel.sum().item() == len(pairs) * rows.numel() * w.H
    assert (got[sel] - want[sel]).abs().max().item() <= TOL
    _check_whole_tensor_without_an_oracle(forward, q, k, v, w, got, gpu)


def test_config_reference_benchmark_shape(gpu):
    # The shape of the reference's own benchmark (reference tests/benchmark_fused_attn.py:9-15:
    # batch 4, 40 heads, sequence 2048, head_dim 128, chunk 128), which the reference times but
    # never checks.
    import fused_attn

    w = workloads.WORKLOADS["readme"]
    q, k, v = workloads.make_inputs(w)

    def forward(q, k, v):
        return fused_attn.attention_forward(w.H, 128, q, k, v)

    got = forward(q.to(gpu), k.to(gpu), v.to(gpu)).float().cpu()
    assert torch.isfinite(got).all()
    pairs = [(b, h) for b in range(w.B) for h in range(w.R) if (b * w.R + h) % 9 == 0]   # 18 of 160, every residue mod 8
    want = attention_per_head(q, k, v, w.H, heads=pairs)
    sel = ~torch.isnan(want)
    assert (got[sel] - want[sel]).abs().max().item() <= TOL
    _check_whole_tensor_without_an_oracle(forward, q, k, v, w, got, gpu)


def test_full_size_properties_without_an_oracle(gpu):
    # Size-independent properties at the headline size: the output is linear in V, and a constant
    # shift of all values shifts the output by the same constant (the weights of a row sum to one).
    import fused_attn

    w = workloads.WORKLOADS["c3"]
    q, k, v = (t.to(gpu) for t in workloads.make_inputs(w))
    g = torch.Generator().manual_seed(97)
    v2 = (torch.randn(v.shape, generator=g) * 0.5).to(torch.float16).to(gpu)
    o1 = fused_attn.attention_forward(w.H, 64, q, k, v).float()
    o2 = fused_attn.attention_forward(w.H, 64, q, k, v2).float()
    vsum = (v.float() + 2.0 * v2.float()).half()
    o12 = fused_attn.attention_forward(w.H, 64, q, k, vsum).float()
    # fp16 rounding of the summed values and of the three outputs: a few 1e-3
    assert (o12 - (o1 + 2.0 * o2)).abs().max().item() <= TOL
    shifted = fused_attn.attention_forward(w.H, 64, q, k, (v.float() + 1.0).half()).float()
    assert (shifted - (o1 + 1.0)).abs().max().item() <= TOL


def test_duplicated_keys_at_long_sequence(gpu):
    # Concatenating (K, V) with itself leaves the output unchanged: 8192 -> 16384 keys at head_dim
    # 128 crosses from one launch shape to another and doubles the number of key tiles.
    B, R, L, H = 1, 32, 8192, 128
    q, k, v = (_rand((B, L, R * H), 5100 + i, std=0.5).to(gpu) for i in range(3))
    once = capi.forward(q, k, v, H).float()
    q2 = torch.cat([q, q], dim=1)
    twice = capi.forward(q2, torch.cat([k, k], dim=1), torch.cat([v, v], dim=1), H).float()
    assert (twice[:, :L] - once).abs().max().item() <= 2e-3
    assert (twice[:, L:] - once).abs().max().item() <= 2e-3


# ---- shapes the reference never exercised ---------------------------------------------------------

@pytest.mark.parametrize("B,R,L,H", [
    (1, 1, 1, 64), (1, 1, 2, 16), (2, 3, 31, 32), (1, 2, 33, 64), (3, 5, 63, 64), (2, 2, 65, 128),
    (1, 3, 255, 64), (2, 2, 257, 64), (1, 2, 511, 32), (2, 7, 300, 16), (1, 1, 1025, 128), (1, 40, 129, 128),
])
def test_ragged_and_odd_shapes(gpu, B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 1000 + L + i) for i in range(3))
    want = attention(q, k, v, H)
    out = torch.full_like(q, float("nan"), device=gpu)
    capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, out=out)
    assert _max_err(out, want) <= TOL


def test_native_bhld_layout_matches_packed_layout(gpu):
    B, R, L, H = 2, 3, 200, 64
    q, k, v = (_rand((B, L, R * H), 2000 + i).to(gpu) for i in range(3))
    packed = capi.forward(q, k, v, H)
    qb, kb, vb = (workloads.to_bhld(t, H) for t in (q, k, v))
    native = capi.forward(qb, kb, vb, H, layout="bhld")
    assert torch.equal(native.transpose(1, 2).reshape(B, L, R * H), packed)


@pytest.mark.parametrize("B,R,L,H,mode", [
    (2, 3, 200, 64, "plain"), (1, 2, 333, 128, "plain"), (2, 4, 130, 16, "plain"), (3, 2, 257, 32, "causal"),
    (1, 2, 200, 64, "mask"), (4, 16, 2048, 64, "plain"), (1, 32, 2048, 128, "causal"), (2, 80, 512, 64, "plain"),
    (1, 40, 2048, 128, "causal"),
])
def test_views_into_a_packed_qkv_tensor(gpu, B, R, L, H, mode):
    """q, k, v as slices of one [B, L, 3, R*H] projection output and a dense output of its own
    strides: bitwise the result of the same call on contiguous copies, and the packed tensor's
    other bytes (and the padding around a strided output) stay untouched."""
    F = R * H
    qkv = _rand((B, L, 3, F), 77 + L).to(gpu)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    assert not q.is_contiguous()
    mask = None
    if mode == "mask":
        mask = (_rand((B, L, L), 5) * 2).to(gpu)
    kw = dict(mask=mask, causal=(mode == "causal"), return_lse=True)
    want, want_lse = capi.forward(q.contiguous(), k.contiguous(), v.contiguous(), H, **kw)
    before = qkv.clone()
    got, got_lse = capi.forward(q, k, v, H, **kw)
    assert got.is_contiguous() and torch.equal(got, want) and torch.equal(got_lse, want_lse)
    assert torch.equal(qkv, before)
    # the output as a view as well: every second row slot of a padded buffer
    pad = torch.full((B, L, 2, F + 8), 7.0, dtype=torch.float16, device=gpu)
    view = pad[:, :, 1, 8:]
    capi.forward(q, k, v, H, out=view, mask=mask, causal=(mode == "causal"))
    assert torch.equal(view, want)
    assert (pad[:, :, 0] == 7.0).all() and (pad[:, :, 1, :8] == 7.0).all()
    if L <= 400:
        omask = causal_mask(B, L) if mode == "causal" else (mask.cpu() if mask is not None else None)
        assert _max_err(got, attention(*(t.contiguous().cpu() for t in (q, k, v)), H, mask=omask)) <= TOL


def test_views_in_the_bhld_layout_and_mismatched_strides(gpu):
    B, R, L, H = 2, 3, 150, 64
    big = _rand((3, B, R, L + 10, H), 9).to(gpu)          # [3][B, R, L+10, H]: rows beyond L are padding
    q, k, v = (big[i, :, :, :L] for i in range(3))
    want = capi.forward(q.contiguous(), k.contiguous(), v.contiguous(), H, layout="bhld")
    assert torch.equal(capi.forward(q, k, v, H, layout="bhld"), want)
    with pytest.raises(ValueError, match="same strides"):
        capi.forward(q, k.contiguous(), v, H, layout="bhld")
    with pytest.raises(ValueError, match="last dimension"):
        capi.forward(q.transpose(2, 3).contiguous().transpose(2, 3), k, v, H, layout="bhld")


@pytest.mark.parametrize("R,L,H", [(2, 70, 64), (160, 600, 64), (80, 600, 128)])
def test_row_pitch_at_the_limit(gpu, R, L, H):
    """stride_l = 2^24 elements, the largest the library accepts (32 MiB between sequence
    positions): q, k, v are column ranges of one [L, 2^24] buffer.  Bitwise the result of the
    same call on contiguous copies, through the four-wave and the eight-wave kernel."""
    F = R * H
    pitch = 1 << 24
    buf = torch.empty((L, pitch), dtype=torch.float16, device=gpu)      # 2.3 GB / 20 GB, mostly untouched
    buf[:, :3 * F] = _rand((L, 3 * F), 4100 + L).to(gpu)
    q, k, v = (buf[:, i * F:(i + 1) * F].unsqueeze(0) for i in range(3))
    assert q.stride()[1:] == (pitch, 1)
    want, want_lse = capi.forward(q.contiguous(), k.contiguous(), v.contiguous(), H, return_lse=True)
    got, got_lse = capi.forward(q, k, v, H, return_lse=True)
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    assert torch.equal(capi.forward(q, k, v, H, causal=True),
                       capi.forward(q.contiguous(), k.contiguous(), v.contiguous(), H, causal=True))
    _check_pairs(got.cpu(), q.contiguous().cpu(), k.contiguous().cpu(), v.contiguous().cpu(), H, [(0, 0), (0, R - 1)])
    # one element more is rejected
    with pytest.raises(capi.FusedAttnError, match="index range"):
        status = capi.load_library().fa_fwd_strided(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), None, got.data_ptr(), None, 1, R, L, H,
            L * pitch, H, pitch + 8, L * F, H, F, 0.125, 0, None)
        capi._check(status)
    del buf


def test_runs_on_the_current_stream_and_is_deterministic(gpu):
    import fused_attn

    w = workloads.WORKLOADS["c1"]
    q, k, v = (t.to(gpu) for t in workloads.make_inputs(w))
    first = fused_attn.attention_forward(w.H, 64, q, k, v)
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(side):
        second = fused_attn.attention_forward(w.H, 64, q, k, v)
    side.synchronize()
    assert torch.equal(first, second)


def test_concurrent_calls_from_host_threads(gpu):
    """The library keeps no state between calls except a mutex-guarded list of kernels whose LDS
    limit it has raised: four host threads launching different shapes on streams of their own
    get the results of the same calls made one after the other."""
    from concurrent.futures import ThreadPoolExecutor

    shapes = [(2, 3, 300, 64, False), (4, 16, 2048, 64, False), (2, 40, 1024, 128, True), (1, 24, 777, 32, False)]
    inputs = [tuple(_rand((B, L, R * H), 4300 + L + i).to(gpu) for i in range(3)) for B, R, L, H, _ in shapes]
    serial = [capi.forward(*inputs[i], shapes[i][3], causal=shapes[i][4]) for i in range(len(shapes))]
    torch.cuda.synchronize()

    def work(i):
        stream = torch.cuda.Stream(device=gpu)
        outs = []
        with torch.cuda.stream(stream):
            for _ in range(20):
                outs.append(capi.forward(*inputs[i], shapes[i][3], causal=shapes[i][4]))
        stream.synchronize()
        return all(torch.equal(o, serial[i]) for o in outs)

    with ThreadPoolExecutor(max_workers=4) as pool:
        assert all(pool.map(work, range(len(shapes))))


# ---- closed forms (no oracle involved) ---------------------------------------------------------------

@pytest.mark.parametrize("L", [1000, 3073])
def test_zero_queries_return_the_mean_over_the_true_keys(gpu, L):
    # Catches tail-padding leakage: padded keys would enter the mean.
    B, R, H = 1, 2, 64
    k, v = _rand((B, L, R * H), 3000, 3.0), _rand((B, L, R * H), 3001)
    out = capi.forward(torch.zeros_like(k).to(gpu), k.to(gpu), v.to(gpu), H)
    want = v.double().mean(dim=1, keepdim=True).float().expand(B, L, R * H)
    assert _max_err(out, want) <= 1e-3


def test_constant_values_are_returned(gpu):
    B, R, L, H = 2, 2, 777, 64
    q, k = _rand((B, L, R * H), 3100, 3.0), _rand((B, L, R * H), 3101, 3.0)
    v = torch.full((B, L, R * H), 1.5, dtype=torch.float16)
    out = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H)
    assert _max_err(out, v.float()) <= 1e-3


def test_one_hot_retrieval_with_huge_scores(gpu):
    # Orthogonal keys (scaled Hadamard-like sign codes); query i points at key pi(i) with score 90+.
    H, L = 64, 64
    had = torch.tensor([[1.0]])
    while had.shape[0] < H:
        had = torch.cat([torch.cat([had, had], 1), torch.cat([had, -had], 1)], 0)
    k = (had * 3.0).to(torch.float16).view(1, L, H)
    perm = torch.randperm(L, generator=torch.Generator().manual_seed(7))
    q = (k[0, perm] * 1.5).contiguous().view(1, L, H)    # matching score 4.5*3*64/8 = 108, others 0
    v = _rand((1, L, H), 3200)
    out = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H)
    assert _max_err(out, v[0, perm].float().view(1, L, H)) <= 1e-3


def test_shift_and_duplication_invariance(gpu):
    B, R, L, H = 1, 2, 320, 64
    q, k, v = (_rand((B, L, R * H), 3300 + i) for i in range(3))
    base = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H).float().cpu()
    # a constant added to every key shifts each score row by q.delta/sqrt(H): the running max moves
    # by a large amount while the weights stay the same
    delta = torch.zeros(1, 1, R * H, dtype=torch.float16)
    delta[..., ::2] = 4.0
    shifted = capi.forward(q.to(gpu), (k + delta).to(gpu), v.to(gpu), H).float().cpu()
    assert (shifted - base).abs().max().item() <= 3e-3
    dup = capi.forward(q.repeat(1, 2, 1).to(gpu), k.repeat(1, 2, 1).to(gpu), v.repeat(1, 2, 1).to(gpu), H)
    assert (dup.float().cpu()[:, :L] - base).abs().max().item() <= 2e-3


def test_heads_and_batches_are_independent_bitwise(gpu):
    B, R, L, H = 2, 3, 130, 64
    q, k, v = (_rand((B, L, R * H), 3400 + i) for i in range(3))
    base = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H).cpu()
    q2, k2, v2 = q.clone(), k.clone(), v.clone()
    for t in (q2, k2, v2):
        t[0, :, H:2 * H] = t[0, :, H:2 * H] * 0.5 + 1.0
    out = capi.forward(q2.to(gpu), k2.to(gpu), v2.to(gpu), H).cpu()
    assert torch.equal(out[1], base[1])
    assert torch.equal(out[0, :, :H], base[0, :, :H]) and torch.equal(out[0, :, 2 * H:], base[0, :, 2 * H:])
    assert not torch.equal(out[0, :, H:2 * H], base[0, :, H:2 * H])


@pytest.mark.parametrize("B,R,L,H,causal", [
    (2, 16, 1024, 64, False),       # the four-wave kernel
    (4, 16, 2048, 64, False),       # the 16 x 16 kernel, one whole round
    (2, 64, 1024, 128, False),      # ... at head_dim 128
    (16, 16, 1024, 64, True),       # ... causal, a pair of tiles per workgroup
    (2, 40, 2048, 128, True),       # ... causal, tiles dealt out to a resident grid
])
def test_launch_can_be_captured_in_a_graph_and_replayed(gpu, B, R, L, H, causal):
    # The library allocates nothing and clears nothing at launch time, so a launch on a capturing
    # stream is recorded as a single kernel node.  Replays must follow the contents of the (static)
    # input buffers and agree bitwise with eager launches, with eager work between the replays.
    import fused_attn

    forward = lambda a, b_, c: fused_attn.attention_forward_ex(a, b_, c, H, causal=causal)
    q, k, v = (_rand((B, L, R * H), 2400 + i).to(gpu) for i in range(3))
    eager0 = forward(q, k, v)        # also the warm-up launch
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = forward(q, k, v)
    for rep in range(4):
        if rep:
            q.copy_(_rand((B, L, R * H), 2410 + rep))            # new inputs in the captured buffers
        eager = forward(q, k, v)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        if rep == 0:
            assert torch.equal(out, eager0)
    pairs = [(0, 0), (B - 1, R // 2), (B - 1, R - 1)]
    _check_pairs(out, q.cpu(), k.cpu(), v.cpu(), H, pairs, mask=causal_mask(B, L) if causal else None)


def _random_cases(n, seed):
    import random

    rng = random.Random(seed)
    cases = []
    for i in range(n):
        H = rng.choice([16, 32, 64, 128])
        L = rng.choice([rng.randint(1, 96), rng.randint(97, 700), rng.randint(701, 2600)])
        heads = rng.choice([1, 3, 8, 24, 96, 300])
        B = rng.choice([1, 2, 3])
        R = max(1, heads // B)
        if B * R * L * H > 40_000_000:
            R = max(1, 40_000_000 // (B * L * H))
        mode = rng.choice(["plain", "plain", "causal", "mask"])
        cases.append((i, B, R, L, H, mode))
    return cases


def _random_big_cases(n, seed):
    # grids of several hundred workgroups and more: the eight-wave kernel in all its variants
    import random

    rng = random.Random(seed)
    cases = []
    for i in range(n):
        H = rng.choice([16, 32, 64, 64, 128, 128])
        L = rng.choice([rng.randint(520, 1100), rng.randint(1101, 2600), 8 * rng.randint(70, 300)])
        B = rng.choice([1, 2, 4])
        R = max(1, min(rng.choice([96, 200, 320, 512]) // B, 36_000_000 // (B * L * H)))
        cases.append((100 + i, B, R, L, H, ["plain", "causal", "mask"][i % 3]))
    return cases


@pytest.mark.parametrize("i,B,R,L,H,mode", _random_cases(28, 20261125) + _random_big_cases(18, 20261126))
def test_seeded_random_shapes(gpu, i, B, R, L, H, mode):
    # shapes drawn once from a fixed seed: odd lengths, every head_dim, grids from one workgroup to
    # several rounds of the chip, all three modes
    q, k, v = (_rand((B, L, R * H), 6000 + 3 * i + j) for j in range(3))
    mask = None
    dev_mask = None
    if mode == "causal":
        mask = causal_mask(B, L)
    elif mode == "mask":
        g = torch.Generator().manual_seed(6100 + i)
        mask = torch.where(torch.rand(B, L, L, generator=g) < 0.25, float("-inf"), 0.0)
        mask = (mask + torch.randn(B, L, L, generator=g) * 0.5).to(torch.float16)
        mask[:, :, 0] = 0
        dev_mask = mask.to(gpu)
        mask = mask.float()
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=dev_mask, causal=(mode == "causal"),
                            return_lse=True)
    assert torch.isfinite(got.float()).all()
    pairs = sorted({(0, 0), (B - 1, R // 2), (B - 1, R - 1)})
    _check_pairs(got, q, k, v, H, pairs, mask=mask)
    for b, h in pairs:
        sl = slice(h * H, (h + 1) * H)
        want = attention_lse(q[b:b + 1, :, sl], k[b:b + 1, :, sl], H, mask=None if mask is None else mask[b:b + 1])[0, 0]
        assert ((lse[b, h].cpu() - want).abs() / (1 + want.abs())).max().item() <= 1e-3


# ---- additive mask ---------------------------------------------------------------------------------

@pytest.mark.parametrize("L,H,offset", [(64, 64, 0), (200, 32, 0), (300, 128, 0), (203, 64, 0), (97, 16, 0),
                                        (200, 64, 1)])
def test_additive_mask_on_every_key_tile(gpu, L, H, offset):
    # L % 4 != 0 or a mask that starts `offset` elements into its allocation (2-byte aligned only)
    # take the element-wise mask loads instead of the 8-byte ones
    import fused_attn

    B, R = 2, 2
    q, k, v = (_rand((B, L, R * H), 3500 + i) for i in range(3))
    g = torch.Generator().manual_seed(3510)
    mask = torch.where(torch.rand(B, L, L, generator=g) < 0.3, float("-inf"), 0.0)
    mask = (mask + torch.randn(B, L, L, generator=g) * 0.5).to(torch.float16)
    mask[:, :, 0] = 0                                   # keep at least one key per row
    want = attention(q, k, v, H, mask=mask)
    flat = torch.empty(B * L * L + offset, dtype=torch.float16, device=gpu)
    dev_mask = flat[offset:].view(B, L, L)
    dev_mask.copy_(mask)
    assert dev_mask.is_contiguous() and dev_mask.data_ptr() % 8 == (2 * offset) % 8
    got = fused_attn.attention_forward(H, 32, q.to(gpu), k.to(gpu), v.to(gpu), dev_mask)
    assert _max_err(got, want) <= TOL


@pytest.mark.parametrize("B,R,L,H", [(2, 2, 200, 64), (4, 16, 2048, 64), (2, 40, 1024, 128)])
def test_mask_of_finite_minimum_values(gpu, B, R, L, H):
    """Masks as libraries commonly build them: the most negative fp16 number (-65504) instead of
    -inf, here above the diagonal and on the padded keys at the end of the last batch entry."""
    q, k, v = (_rand((B, L, R * H), 3650 + L + i) for i in range(3))
    lowest = torch.finfo(torch.float16).min
    mask = torch.full((L, L), lowest).triu(1).expand(B, L, L).clone()
    mask[B - 1, :, L - 37:] = lowest
    mask = mask.to(torch.float16)
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=mask.to(gpu))
    assert torch.isfinite(got.float()).all()
    # the oracle with -inf in the same places: every row keeps at least key 0
    hard = torch.where(mask == lowest, float("-inf"), 0.0)
    _check_pairs(got, q, k, v, H, [(0, 0), (B - 1, R - 1)], mask=hard)


@pytest.mark.parametrize("B,R,L,H", [(2, 2, 200, 64), (4, 16, 2048, 64), (2, 40, 1024, 128)])
def test_subnormal_inputs(gpu, B, R, L, H):
    """fp16 subnormals (below 6.1e-5) are operands like any other: values of that size come out
    as their weighted mean, not as zero, and subnormal queries and keys give uniform weights."""
    q, k, v = (_rand((B, L, R * H), 3680 + L + i) for i in range(3))
    tiny_v = (v.float() * 2e-5).to(torch.float16)
    assert (tiny_v.float().abs() < 6.1e-5).float().mean() > 0.9
    got = capi.forward(q.to(gpu), k.to(gpu), tiny_v.to(gpu), H).float().cpu()
    for b, h in [(0, 0), (B - 1, R - 1)]:
        sl = slice(h * H, (h + 1) * H)
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], tiny_v[b:b + 1, :, sl], H)
        # compared in units of the values' own size; the output has fp16 subnormal spacing 6e-8
        assert ((got[b:b + 1, :, sl] - want).abs().max().item()) / 2e-5 <= TOL + 6e-8 / 2e-5
        assert got[b, :, sl].abs().max().item() > 0
    tiny_q = (q.float() * 1e-5).to(torch.float16)
    tiny_k = (k.float() * 1e-5).to(torch.float16)
    flat = capi.forward(tiny_q.to(gpu), tiny_k.to(gpu), v.to(gpu), H)
    assert _max_err(flat, v.float().mean(dim=1, keepdim=True).expand(B, L, R * H)) <= 1e-3


def test_fully_masked_rows_give_zeros_not_nan(gpu):
    B, R, L, H = 1, 2, 100, 64
    q, k, v = (_rand((B, L, R * H), 3600 + i) for i in range(3))
    mask = torch.zeros(B, L, L, dtype=torch.float16)
    mask[0, 5] = float("-inf")
    mask[0, 77] = float("-inf")
    out = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=mask.to(gpu)).float().cpu()
    assert torch.isfinite(out).all()
    assert (out[0, 5] == 0).all() and (out[0, 77] == 0).all()
    want = attention(q, k, v, H)
    keep = [i for i in range(L) if i not in (5, 77)]
    assert (out[0, keep] - want[0, keep]).abs().max().item() <= TOL


# ---- causal flag and row log-sum-exp (extensions of the C ABI) -------------------------------------

@pytest.mark.parametrize("B,R,L,H", [(1, 2, 64, 64), (2, 3, 200, 32), (1, 2, 777, 64), (2, 2, 300, 128),
                                     (1, 12, 1024, 64), (1, 2, 33, 16)])
def test_causal_matches_the_masked_oracle(gpu, B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 3700 + L + i) for i in range(3))
    want = attention(q, k, v, H, mask=causal_mask(B, L))
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=True)
    assert _max_err(got, want) <= TOL
    # the first row sees one key only: it returns V[0] exactly (after fp16 rounding of an fp16 value)
    assert torch.equal(got[:, 0].cpu(), v[:, 0])


@pytest.mark.parametrize("name,causal", [("c1", False), ("c2", False), ("c5a", False), ("c5a", True), ("c1", True)])
def test_row_logsumexp(gpu, name, causal):
    w = workloads.WORKLOADS[name]
    q, k, v = workloads.make_inputs(w)
    if w.B * w.R > 16:
        q, k, v = (t[:1, :, : 4 * w.H].contiguous() for t in (q, k, v))
    B, L, F = q.shape
    mask = causal_mask(B, L) if causal else None
    want_lse = attention_lse(q, k, w.H, mask=mask)
    want_out = attention(q, k, v, w.H, mask=mask)
    out, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), w.H, causal=causal, return_lse=True)
    assert lse.shape == (B, F // w.H, L) and lse.dtype == torch.float32
    assert _max_err(out, want_out) <= TOL
    # lse is an f32 quantity of magnitude up to ~40 on the stress inputs: compare relatively
    assert ((lse.cpu() - want_lse).abs() / (1 + want_lse.abs())).max().item() <= 1e-3


def test_lse_of_the_pingpong_kernel(gpu):
    # enough workgroups to select the eight-wave kernel; zero queries give lse = log(L) exactly
    B, R, L, H = 4, 16, 2048, 64
    k, v = _rand((B, L, R * H), 3800), _rand((B, L, R * H), 3801)
    out, lse = capi.forward(torch.zeros_like(k).to(gpu), k.to(gpu), v.to(gpu), H, return_lse=True)
    assert (lse.cpu() - math.log(L)).abs().max().item() <= 1e-4
    want = v.double().mean(dim=1, keepdim=True).float().expand(B, L, R * H)
    assert _max_err(out, want) <= 1e-3


@pytest.mark.parametrize("R,H,causal", [(48, 64, False), (24, 128, False), (24, 64, True)])
def test_very_long_ragged_sequence(gpu, R, H, causal):
    """L = 65537: 1025 key tiles with a single key in the last one, 129 (257) query tiles with a
    single query in the last one.  One head against the oracle on sampled query rows (the full
    L x L scores of one head would be 17 GB), every head against closed forms."""
    B, L = 1, 65537
    q, k, v = (_rand((B, L, R * H), 6500 + H + i) for i in range(3))
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=causal, return_lse=True)
    got, lse = got.float().cpu(), lse.cpu()
    assert torch.isfinite(got).all() and torch.isfinite(lse).all()
    rows = torch.tensor([0, 1, 31, 32, 255, 256, 511, 512, 4095, 32768, 65023, 65024, 65535, 65536])
    h = R - 1
    sl = slice(h * H, (h + 1) * H)
    scores = (q[0, rows, sl].float() @ k[0, :, sl].float().T) / math.sqrt(H)
    if causal:
        scores = scores.masked_fill(torch.arange(L)[None, :] > rows[:, None], float("-inf"))
    want = torch.softmax(scores, dim=-1) @ v[0, :, sl].float()
    assert (got[0, rows, sl] - want).abs().max().item() <= TOL
    assert (lse[0, h, rows] - torch.logsumexp(scores, dim=-1)).abs().max().item() <= 1e-3 * math.log(L)
    # outputs are convex combinations of the value rows
    assert (got.abs().amax(dim=1) <= v.float().abs().amax(dim=1) + 1e-3).all()
    if not causal:
        zero = capi.forward(torch.zeros_like(q).to(gpu), k.to(gpu), v.to(gpu), H).float().cpu()
        mean = v.float().mean(dim=1, keepdim=True)
        assert (zero - mean).abs().max().item() <= 1e-3


@pytest.mark.parametrize("B,R,L,H", [(1, 3, 300, 64), (4, 16, 2048, 64), (2, 64, 1024, 128)])
def test_non_finite_inputs_stay_where_the_oracle_puts_them(gpu, B, R, L, H):
    """A NaN in one query row and an inf in one key row: the call returns, the rows the oracle
    leaves finite match it, the rows it makes NaN are NaN, and the other heads do not change a bit."""
    q, k, v = (_rand((B, L, R * H), 8800 + L + i) for i in range(3))
    clean = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H).cpu()
    q2, k2 = q.clone(), k.clone()
    q2[0, 5, 3] = float("nan")                       # head 0, query 5
    k2[B - 1, L - 2, H + 1] = float("inf")           # head 1 of the last batch, key L - 2
    got = capi.forward(q2.to(gpu), k2.to(gpu), v.to(gpu), H).cpu()
    # heads and batches that hold no non-finite input: bitwise unchanged
    touched = torch.zeros(B, R, dtype=torch.bool)
    touched[0, 0] = True
    touched[B - 1, 1] = True
    for b in range(B):
        for h in range(R):
            if not touched[b, h]:
                assert torch.equal(got[b, :, h * H:(h + 1) * H], clean[b, :, h * H:(h + 1) * H]), (b, h)
    for b, h in ((0, 0), (B - 1, 1)):
        sl = slice(h * H, (h + 1) * H)
        want = attention(q2[b:b + 1, :, sl], k2[b:b + 1, :, sl], v[b:b + 1, :, sl], H)[0]
        mine = got[b, :, sl].float()
        bad = ~torch.isfinite(want).all(dim=-1)
        assert bad.any()
        assert (~torch.isfinite(mine[bad])).any(dim=-1).all()
        assert torch.isfinite(mine[~bad]).all()
        assert (mine[~bad] - want[~bad]).abs().max().item() <= TOL


@pytest.mark.parametrize("B,R,L,H", [(2, 3, 300, 64), (4, 16, 2048, 64), (2, 64, 1024, 128)])
def test_scale_argument(gpu, B, R, L, H):
    """The C ABI takes the softmax scale as an argument (the reference fixes it at 1/sqrt(head_dim)):
    a tiny one gives the mean of the value rows, any other value equals the default scale on
    queries multiplied by scale * sqrt(head_dim) (done in fp32 on the oracle's side)."""
    q, k, v = (_rand((B, L, R * H), 9100 + L + i) for i in range(3))
    dq, dk, dv = q.to(gpu), k.to(gpu), v.to(gpu)
    flat = capi.forward(dq, dk, dv, H, scale=1e-9)
    assert _max_err(flat, v.float().mean(dim=1, keepdim=True).expand(B, L, R * H)) <= 1e-3
    for scale in (1.0 / H, 0.3, 1.0):
        got, lse = capi.forward(dq, dk, dv, H, scale=scale, return_lse=True)
        qs = q.float() * (scale * math.sqrt(H))
        pairs = [(0, 0), (B - 1, R - 1)]
        for b, h in pairs:
            sl = slice(h * H, (h + 1) * H)
            want = attention(qs[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H)
            assert _max_err(got[b:b + 1, :, sl], want) <= TOL, (scale, b, h)
            want_lse = attention_lse(qs[b:b + 1, :, sl], k[b:b + 1, :, sl], H)[0, 0]
            assert (lse[b, h].cpu() - want_lse).abs().max().item() <= 2e-3, (scale, b, h)
    for bad in (0.0, -1.0, float("nan"), float("inf")):
        with pytest.raises(capi.FusedAttnError):
            capi.forward(dq, dk, dv, H, scale=bad)


# ---- every launch shape, plain and masked -------------------------------------------------------------

def _check_pairs_tol(got, q, k, v, H, pairs, mask, tol):
    for b, h in pairs:
        sl = slice(h * H, (h + 1) * H)
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H, mask=mask[b:b + 1])
        assert _max_err(got[b:b + 1, :, sl], want) <= tol, (b, h)


def _check_pairs(got, q, k, v, H, pairs, mask=None):
    """Compares the listed (batch, head) slices of a full-tensor result against the oracle."""
    for b, h in pairs:
        sl = slice(h * H, (h + 1) * H)
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H,
                         mask=None if mask is None else mask[b:b + 1])
        assert _max_err(got[b:b + 1, :, sl], want) <= TOL, (b, h)


@pytest.mark.parametrize("B,R,L,H", [
    (1, 20, 4096, 64),      # eight-wave workgroups filling part of one round of the chip
    (1, 40, 4096, 64),      # a poorly filled second round: eight 32-row waves, two workgroups per CU
    (1, 500, 256, 64),      # ... on short sequences
    (2, 8, 3073, 64),       # ... with ragged tiles, less than one workgroup per CU
    (1, 40, 2100, 32), (3, 20, 1111, 16),   # ... at the smaller head dims
    (1, 400, 40, 64), (2, 200, 7, 32),      # ... with sequences far shorter than a workgroup's 256 rows
    (1, 32, 1024, 64),      # too few of those: four-wave workgroups
    (4, 16, 2112, 64),      # many workgroups, ragged last key tile and last query tile
    (1, 20, 2048, 128),     # head_dim 128, eight-wave workgroups in a part-filled round
    (1, 40, 2048, 128),     # head_dim 128, four-wave workgroups
    (2, 160, 1088, 128),    # head_dim 128, many workgroups, ragged tiles
])
def test_launch_shapes_plain(gpu, B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 3900 + L + i) for i in range(3))
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H)
    assert torch.isfinite(got.float()).all()
    _check_pairs(got, q, k, v, H, [(0, 0), (B - 1, R // 2), (B - 1, R - 1)])


@pytest.mark.parametrize("B,R,L", [
    (4, 16, 2048),      # one whole round of 512-query workgroups
    (8, 32, 1000),      # two rounds, ragged last key tile and second query tile
    (4, 64, 1500),      # three rounds, three tiles per head, the last a quarter full
    (2, 60, 2048),      # a last round seven eighths full
    (1, 16, 16384),     # long rows: 256 key tiles per workgroup
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kernel_with_16_row_matrix_tiles(gpu, B, R, L, dtype):
    # Plain launches at head_dim 64 whose workgroups fill whole rounds of the chip take the kernel
    # written on 16 x 16 x 32 products; here with row log-sum-exps, in both layouts.
    H = 64
    assert capi.launch_plan(B, R, L, H)["matrix_tile"] == 16
    q, k, v = (_rand((B, L, R * H), 4000 + L + i).to(dtype) for i in range(3))
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, return_lse=True)
    assert torch.isfinite(got.float()).all()
    tol = TOL if dtype == torch.float16 else BF16_TOL
    pairs = [(0, 0), (B // 2, R // 3), (B - 1, R // 2), (B - 1, R - 1)]
    for b, h in pairs:
        sl = slice(h * H, (h + 1) * H)
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H)
        assert _max_err(got[b:b + 1, :, sl], want) <= tol, (b, h)
        want = attention_lse(q[b:b + 1, :, sl], k[b:b + 1, :, sl], H)[0, 0]
        assert ((lse[b, h].cpu() - want).abs() / (1 + want.abs())).max().item() <= 1e-3, (b, h)
    heads = lambda t: t.view(B, L, R, H).permute(0, 2, 1, 3).contiguous().to(gpu)
    same = capi.forward(heads(q), heads(k), heads(v), H, layout="bhld")
    assert torch.equal(same.permute(0, 2, 1, 3).reshape(B, L, R * H), got)


@pytest.mark.parametrize("B,R,L,causal", [
    (2, 64, 1024, False),    # 512 workgroups of 256 queries: two whole rounds
    (4, 40, 2048, False),    # the reference's benchmark shape: five rounds
    (4, 64, 1250, False),    # five tiles per head, ragged end (1280 workgroups)
    (1, 28, 2048, False),    # a single round seven eighths full
    (1, 8, 16384, False),    # 256 key tiles per workgroup
    (2, 64, 1024, True),     # causal: two pairs per head
    (1, 32, 16384, True),    # ... 32 pairs per head
    (4, 64, 1250, True),     # ... five tiles per head, ragged end, dealt out to a resident grid
    (5, 17, 1250, True),     # ... in pairs with the middle one alone
    (2, 40, 2048, True),     # ... tiles dealt out to a resident grid
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kernel_with_16_row_matrix_tiles_at_head_dim_128(gpu, B, R, L, causal, dtype):
    # The 16 x 16 kernel with 32-row waves (two blocks of 16 queries, dealt w and 15 - w under the causal flag)
    H = 128
    assert capi.launch_plan(B, R, L, H, causal=causal)["matrix_tile"] == 16
    q, k, v = (_rand((B, L, R * H), 4080 + L + i).to(dtype) for i in range(3))
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=causal, return_lse=True)
    assert torch.isfinite(got.float()).all()
    tol = TOL if dtype == torch.float16 else BF16_TOL
    mask = causal_mask(1, L) if causal else None
    for b, h in [(0, 0), (B // 2, R // 3), (B - 1, R - 1)]:
        sl = slice(h * H, (h + 1) * H)
        rows = slice(None) if L <= 4096 else torch.cat([torch.arange(0, 600), torch.arange(L - 600, L), torch.arange(600, L - 600, 97)])
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H, mask=mask)
        assert (got[b, rows, sl].float().cpu() - want[0, rows]).abs().max().item() <= tol, (b, h)
        want = attention_lse(q[b:b + 1, :, sl], k[b:b + 1, :, sl], H, mask=mask)[0, 0]
        assert ((lse[b, h].cpu() - want).abs() / (1 + want.abs()))[rows].max().item() <= 1e-3, (b, h)
    heads = lambda t: t.view(B, L, R, H).permute(0, 2, 1, 3).contiguous().to(gpu)
    same = capi.forward(heads(q), heads(k), heads(v), H, layout="bhld", causal=causal)
    assert torch.equal(same.permute(0, 2, 1, 3).reshape(B, L, R * H), got)


@pytest.mark.parametrize("B,R,L", [
    (4, 16, 4096),      # 256 pairs of 512-query tiles
    (16, 16, 1024),     # one pair per head: both tiles are diagonal tiles
    (16, 16, 1000),     # ... with a ragged second tile
    (2, 85, 2500),      # five tiles per head: two pairs and the middle tile alone, ragged end
    (1, 16, 16384),     # 16 pairs per head, up to 32 key tiles below the diagonal
    (2, 40, 4096),      # 320 pairs would be 1.25 rounds: tiles dealt out to a resident grid
    (2, 64, 1300),      # ... three tiles per head, ragged end
    (3, 20, 4096),      # 240 pairs: a single round, not quite full
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_causal_kernel_with_16_row_matrix_tiles(gpu, B, R, L, dtype):
    # Causal launches at head_dim 64 from seven eighths of a round of 512-query workgroups on (pairs of
    # query tiles, or tiles dealt out to a resident grid): the 16 x 16 kernel, whose waves own blocks of
    # 16 queries dealt out so that all eight reach their diagonals together.
    H = 64
    assert capi.launch_plan(B, R, L, H, causal=True)["matrix_tile"] == 16
    q, k, v = (_rand((B, L, R * H), 4050 + L + i).to(dtype) for i in range(3))
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=True, return_lse=True)
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got[:, 0].cpu(), v[:, 0])           # the first query sees the first key only
    tol = TOL if dtype == torch.float16 else BF16_TOL
    mask = causal_mask(1, L)
    for b, h in [(0, 0), (B // 2, R // 3), (B - 1, R - 1)]:
        sl = slice(h * H, (h + 1) * H)
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H, mask=mask)
        assert _max_err(got[b:b + 1, :, sl], want) <= tol, (b, h)
        want = attention_lse(q[b:b + 1, :, sl], k[b:b + 1, :, sl], H, mask=mask)[0, 0]
        assert ((lse[b, h].cpu() - want).abs() / (1 + want.abs())).max().item() <= 1e-3, (b, h)
    # the same rows through the additive-mask path (the 32 x 32 kernel): two kernels, one result
    if L <= 4096:
        other = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=causal_mask(B, L).to(dtype).to(gpu))
        assert (other.float() - got.float()).abs().max().item() <= (2e-3 if dtype == torch.float16 else BF16_TOL)


@pytest.mark.parametrize("B,R,L,H", [(4, 16, 2048, 64), (2, 64, 1024, 128)])
@pytest.mark.parametrize("kind", ["std3", "rising", "falling"])
def test_eight_wave_kernel_on_adversarial_scores(gpu, B, R, L, H, kind):
    # Grids large enough for the eight-wave kernel, with scores that stress its running reference
    # maximum: |score| > 20 all over (std3), or a score that climbs (falls) by about 100 along the
    # key axis, so that the reference is overtaken again and again (never after the first key).
    q, k, v = (_rand((B, L, R * H), 4100 + L + i) for i in range(3))
    if kind == "std3":
        q, k = (q.float() * 3).half(), (k.float() * 3).half()
    else:
        g = torch.Generator().manual_seed(4107)
        u = torch.randn(R * H, generator=g)
        u = u / u.view(R, H).norm(dim=1).repeat_interleave(H)           # unit vector per head
        ramp = torch.linspace(0, 1, L) if kind == "rising" else torch.linspace(1, 0, L)
        q = (q.float() * 0.3 + 10.0 * u).half()
        k = (k.float() * 0.3 + (10.0 * math.sqrt(H)) * ramp.view(1, L, 1) * u).half()
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H)
    assert torch.isfinite(got.float()).all()
    _check_pairs(got, q, k, v, H, [(0, 0), (B - 1, R // 2), (B - 1, R - 1)])
    sl = slice(0, H)
    scores = (q[0, :, sl].float() @ k[0, :, sl].float().T) / math.sqrt(H)
    assert scores.abs().max() > 20


@pytest.mark.parametrize("B,R,L", [(4, 16, 4096), (16, 16, 1024), (2, 40, 4096)])
@pytest.mark.parametrize("kind", ["std3", "rising", "falling"])
def test_causal_16_row_kernel_on_adversarial_scores(gpu, B, R, L, kind):
    # The same stress as above under the causal flag, where the 16 x 16 kernel leaves the blocks of a
    # wave one after the other: the reference is overtaken inside the sub-tiles in which only some
    # of a wave's blocks still take part (pairs of tiles, one pair per head, tiles dealt out).
    H = 64
    assert capi.launch_plan(B, R, L, H, causal=True)["matrix_tile"] == 16
    q, k, v = (_rand((B, L, R * H), 4200 + L + i) for i in range(3))
    if kind == "std3":
        q, k = (q.float() * 3).half(), (k.float() * 3).half()
    else:
        g = torch.Generator().manual_seed(4207)
        u = torch.randn(R * H, generator=g)
        u = u / u.view(R, H).norm(dim=1).repeat_interleave(H)
        ramp = torch.linspace(0, 1, L) if kind == "rising" else torch.linspace(1, 0, L)
        q = (q.float() * 0.3 + 10.0 * u).half()
        k = (k.float() * 0.3 + (10.0 * math.sqrt(H)) * ramp.view(1, L, 1) * u).half()
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=True)
    assert torch.isfinite(got.float()).all()
    _check_pairs(got, q, k, v, H, [(0, 0), (B - 1, R // 2), (B - 1, R - 1)], mask=causal_mask(B, L))


@pytest.mark.parametrize("B,R,L,H", [(2, 16, 4096, 64), (2, 64, 1024, 128)])
@pytest.mark.parametrize("step_log2", [6.5, 14.0, 15.5, 16.5, 18.0, 21.0, 22.5, 26.0])
def test_eight_wave_kernel_reference_lag(gpu, B, R, L, H, step_log2):
    # All scores are 0 up to key 96 and jump by step_log2 (in units of log2) from there on, so the
    # reference the kernel took from the first keys lags by exactly that much: probabilities taken
    # against it land below, inside and beyond the window in which the fp16 pack saturates at 65504
    # instead of overflowing to inf (the check must catch those too).  With the jump the first 96
    # keys carry a weight of 2^-step each, so the output is the mean of V over keys 96.. to within
    # that weight.
    q = torch.zeros(B, L, R * H)
    k = torch.zeros(B, L, R * H)
    q[:, :, ::H] = math.sqrt(H)                       # component 0 of every head: raw score = sqrt(H) * k0
    k[:, 96:, ::H] = step_log2 / math.log2(math.e)    # scaled score in natural-log units
    q, k = q.half(), k.half()
    v = _rand((B, L, R * H), 4300 + L)
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H)
    assert torch.isfinite(got.float()).all()
    _check_pairs(got, q, k, v, H, [(0, 0), (B - 1, R - 1)])
    if step_log2 >= 14:
        want = v[:, 96:].float().mean(dim=1, keepdim=True)
        assert (got.float().cpu() - want).abs().max().item() <= 5e-3


@pytest.mark.parametrize("B,R,L,H", [(2, 16, 4096, 64), (1, 8, 16384, 128), (1, 2, 1024, 64)])
@pytest.mark.parametrize("gap_log2", [10.5, 14.5, 16.5, 17.5, 18.5, 19.0, 22.0])
def test_heavy_tail_of_small_weights(gpu, B, R, L, H, gap_log2):
    # One dominant key, then L - 1 equal keys gap_log2 (log2 units) below it.  Each of them weighs
    # 2^-gap, together (L - 1) 2^-gap: 6 % of the row at gap 18 and L = 16384.  The probabilities
    # are rounded to fp16 before the second product, so a kernel whose reference pushes such
    # weights into the fp16 subnormals (or below 2^-24, to zero) loses that share of the row; the
    # float32 oracle keeps it.  Both kernel families, through eight-wave and four-wave grids.
    t = gap_log2 / math.log2(math.e) / math.sqrt(H)      # key 0 = t * ones: scaled score H t / sqrt(H)
    q = torch.ones(B, L, R * H).half()
    k = torch.zeros(B, L, R * H)
    k[:, 0] = t
    k = k.half()
    gap = k[0, 0, 0].float().item() * math.sqrt(H) * math.log2(math.e)      # what fp16 made of it
    v = _rand((B, L, R * H), 4400 + L)
    v[:, 0] = 4.0                                      # the dominant key's value stands out
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H)
    assert torch.isfinite(got.float()).all()
    tail = (L - 1) * 2.0 ** -gap
    want = (4.0 + tail * v[:, 1:].float().mean(dim=1)) / (1.0 + tail)       # closed form, every row the same
    assert (got.float().cpu() - want.view(B, 1, R * H)).abs().max().item() <= TOL
    _check_pairs(got, q, k, v, H, [(0, 0), (B - 1, R - 1)])


@pytest.mark.parametrize("R,L,H", [(8, 65536, 64), (4, 131072, 128)])
def test_long_sequences_where_the_reference_bias_is_most_negative(gpu, R, L, H):
    """L = 65536 and 131072: the launcher's bias is -5 and -6 (a key at the reference gets the weight
    32 or 64), the leash of the speculative reference 10 and 9 log2 units.  Even heads: one dominant
    key and a heavy tail 17.5 units below it (closed form).  Odd heads: scores that climb by 60
    log2 units along the key axis, so the reference is rebased again and again (the row then
    concentrates on the last keys).  Output and log-sum-exp against float32 evaluations of the
    sampled rows."""
    B = 1
    assert capi.load_library().fa_fwd_reference_bias(L) <= -5
    t = 17.5 / math.log2(math.e) / math.sqrt(H)
    q = torch.ones(B, L, R * H)
    k = torch.zeros(B, L, R * H)
    climb = torch.linspace(0.0, 60.0 / math.log2(math.e) / math.sqrt(H), L)
    for h in range(R):
        if h % 2 == 0:
            k[:, 0, h * H:(h + 1) * H] = t
        else:
            k[:, :, h * H:(h + 1) * H] = climb[None, :, None]
    q, k = q.half(), k.half()
    v = _rand((B, L, R * H), 6600 + H)
    v[:, 0] = 4.0
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, return_lse=True)
    got, lse = got.float().cpu(), lse.cpu()
    assert torch.isfinite(got).all() and torch.isfinite(lse).all()
    rows = torch.tensor([0, 1, 63, 64, 511, 512, L // 2, L - 513, L - 2, L - 1])
    for h in range(R):
        sl = slice(h * H, (h + 1) * H)
        scores = (q[0, rows, sl].float() @ k[0, :, sl].float().T) / math.sqrt(H)
        want = torch.softmax(scores, dim=-1) @ v[0, :, sl].float()
        assert (got[0, rows, sl] - want).abs().max().item() <= TOL, h
        assert (lse[0, h, rows] - torch.logsumexp(scores, dim=-1)).abs().max().item() <= 1e-3 * math.log(L), h
    # even heads, every row: the closed form
    gap = k[0, 0, 0].float().item() * math.sqrt(H) * math.log2(math.e)
    tail = (L - 1) * 2.0 ** -gap
    for h in range(0, R, 2):
        sl = slice(h * H, (h + 1) * H)
        want = (4.0 + tail * v[0, 1:, sl].float().mean(dim=0)) / (1.0 + tail)
        assert (got[0, :, sl] - want).abs().max().item() <= TOL, h


@pytest.mark.parametrize("B,R,L,H", [
    (4, 16, 4096, 64),      # eight-wave workgroups, each taking a pair of query tiles (8 tiles per head)
    (2, 64, 1300, 64),      # ... with an odd number of tiles (the middle one runs alone) and a ragged end
    (2, 64, 1024, 128),     # head_dim 128, four tiles of 256 queries
    (4, 64, 1250, 128),     # head_dim 128, five tiles, ragged end
    (8, 64, 512, 64), (3, 100, 300, 32),     # four-wave workgroups
    (8, 12, 1024, 64), (1, 20, 4096, 64),    # eight 32-row waves: pairs of 256-query tiles filling most of one round
    (3, 16, 2000, 32), (16, 16, 500, 16),    # ... at the smaller head dims, with ragged ends
    (2, 40, 2048, 128), (2, 40, 4096, 64),   # 320 pairs would leave a second round three quarters empty: tiles dealt out to a resident grid
    (2, 40, 2300, 128), (2, 48, 5000, 32),   # ... with an odd number of tiles and ragged ends
    (1, 40, 2048, 128), (1, 40, 4000, 64),   # ... fewer pairs than compute units: single tiles spread over all of them
])
def test_causal_on_large_grids(gpu, B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 3950 + L + i) for i in range(3))
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=True, return_lse=True)
    assert torch.isfinite(got.float()).all()
    mask = causal_mask(B, L)
    pairs = [(0, 0), (B - 1, R // 2), (B - 1, R - 1)]
    _check_pairs(got, q, k, v, H, pairs, mask=mask)
    assert torch.equal(got[:, 0].cpu(), v[:, 0])
    for b, h in pairs:
        sl = slice(h * H, (h + 1) * H)
        want = attention_lse(q[b:b + 1, :, sl], k[b:b + 1, :, sl], H, mask=mask[b:b + 1])[0, 0]
        assert ((lse[b, h].cpu() - want).abs() / (1 + want.abs())).max().item() <= 1e-3


@pytest.mark.parametrize("B,R,L,H", [
    (8, 64, 512, 64), (16, 40, 384, 16), (2, 64, 1024, 32),     # eight-wave kernel, mask staged through LDS
    (4, 40, 704, 128),                                           # ... head_dim 128, ragged end
    (2, 64, 1023, 64),                                           # element-wise mask loads (L % 4 != 0)
    (4, 40, 700, 128),                                           # 8-byte mask loads (L % 8 != 0)
    (2, 12, 2048, 64), (1, 500, 256, 64), (2, 12, 2040, 16), (1, 40, 2104, 32),   # eight 32-row waves, 256-query workgroups
    (1, 40, 2048, 128), (4, 40, 512, 128),   # head_dim 128: 256-query workgroups on a part-filled second round
    (4, 12, 1536, 64),                       # 64-row waves on a lone round filled to 56 %
])
def test_additive_mask_on_large_grids(gpu, B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 3970 + L + i) for i in range(3))
    g = torch.Generator().manual_seed(3975)
    mask = torch.where(torch.rand(B, L, L, generator=g) < 0.3, float("-inf"), 0.0)
    mask = (mask + torch.randn(B, L, L, generator=g) * 0.5).to(torch.float16)
    mask[:, :, 0] = 0
    mask[0, 5] = float("-inf")                  # two fully masked rows: zeros, not NaN
    mask[B - 1, L - 1] = float("-inf")
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=mask.to(gpu))
    assert torch.isfinite(got.float()).all()
    assert (got[0, 5] == 0).all() and (got[B - 1, L - 1] == 0).all()
    mask[0, 5] = 0                              # the oracle would give NaN there; compare the other rows
    mask[B - 1, L - 1] = 0
    keep = torch.ones(B, L, dtype=torch.bool)
    keep[0, 5] = keep[B - 1, L - 1] = False
    for b, h in [(0, 0), (B // 2, R // 2), (B - 1, R - 1)]:
        sl = slice(h * H, (h + 1) * H)
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H, mask=mask[b:b + 1].float())
        err = (got[b, :, sl].float().cpu() - want[0]).abs()
        assert err[keep[b]].max().item() <= TOL, (b, h)


def _block_mask(kind, B, L, seed):
    """Masks under the reference's contract (zero where a pair takes part, -inf where it is muted,
    reference README.md:88-89), made of large all-zero and all-muted blocks: what the kernels'
    classification of mask blocks (zero / muted / mixed) is written for."""
    g = torch.Generator().manual_seed(seed)
    neg = float("-inf")
    m = torch.zeros(B, L, L)
    if kind == "causal":
        m = torch.full((L, L), neg).triu(1).expand(B, L, L).clone()
    elif kind == "padding":                     # batch b keeps its first n_b keys
        for b in range(B):
            m[b, :, L - 1 - (b * 37 + L // 3) % (L - 1):] = neg
    elif kind == "documents":                   # block diagonal: three to five documents per batch
        for b in range(B):
            cuts = sorted(set(torch.randint(1, L, (4,), generator=g).tolist()) | {0, L})
            m[b] = neg
            for lo, hi in zip(cuts[:-1], cuts[1:]):
                m[b, lo:hi, lo:hi] = 0
    elif kind in ("blocks", "finite_min"):      # 32 x 32 blocks: 40 % zero, 35 % muted, 25 % element-wise
        nb = (L + 31) // 32
        cls = torch.rand(B, nb, nb, generator=g)
        up = lambda t: t.repeat_interleave(32, 1).repeat_interleave(32, 2)[:, :L, :L]
        low = -65504.0 if kind == "finite_min" else neg
        m = torch.where(up(cls) < 0.35, low, 0.0)
        noisy = torch.where(torch.rand(B, L, L, generator=g) < 0.5, low, 0.0) + torch.randn(B, L, L, generator=g) * 0.25
        m = torch.where(up(cls) > 0.75, noisy, m)
        m[:, :, 0] = 0                          # every row keeps a key
    else:
        raise ValueError(kind)
    return m.to(torch.float16)


@pytest.mark.parametrize("B,R,L,H", [
    (4, 16, 2048, 64),       # eight 64-row waves
    (2, 40, 1024, 128),      # eight 32-row waves, head_dim 128
    (2, 12, 2048, 64),       # eight 32-row waves, 256-query workgroups
    (2, 64, 1000, 32),       # ... ragged end
    (2, 2, 200, 64),         # four waves
    (1, 4, 1023, 64),        # four waves, element-wise mask loads
])
@pytest.mark.parametrize("kind", ["causal", "padding", "documents", "blocks", "finite_min"])
def test_block_structured_masks(gpu, B, R, L, H, kind):
    q, k, v = (_rand((B, L, R * H), 5100 + L + i) for i in range(3))
    mask = _block_mask(kind, B, L, 5110 + L)
    dead = [(0, min(L - 1, 40)), (B - 1, L - 1)]      # two fully muted rows: zeros, not NaN
    for b, r in dead:
        mask[b, r] = float("-inf")
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=mask.to(gpu))
    assert torch.isfinite(got.float()).all()
    keep = torch.ones(B, L, dtype=torch.bool)
    for b, r in dead:
        assert (got[b, r] == 0).all()
        mask[b, r] = 0                                # the oracle would give NaN there
        keep[b, r] = False
    for b, h in sorted({(0, 0), (B // 2, R // 2), (B - 1, R - 1)}):
        sl = slice(h * H, (h + 1) * H)
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H, mask=mask[b:b + 1].float())
        err = (got[b, :, sl].float().cpu() - want[0]).abs()
        assert err[keep[b]].max().item() <= TOL, (b, h)
    if kind == "causal":      # the same result as the causal flag, row for row
        flag = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=True)
        diff = (flag.float() - got.float()).abs().cpu()
        assert diff[keep].max().item() <= 2e-3


@pytest.mark.parametrize("B,R,L,H", [(4, 16, 2048, 64), (2, 40, 1024, 128), (2, 2, 200, 64)])
def test_block_structured_masks_bf16(gpu, B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 5200 + L + i).to(torch.bfloat16) for i in range(3))
    mask = _block_mask("blocks", B, L, 5210 + L).to(torch.bfloat16)
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=mask.to(gpu))
    _check_pairs_tol(got, q, k, v, H, [(0, 0), (B - 1, R - 1)], mask.float(), BF16_TOL)


# ---- bfloat16 inputs (FA_FLAG_BF16) ------------------------------------------------------------------

BF16_TOL = 2e-2   # bf16 keeps 8 significant bits: the output rounding alone is 2^-9 * |o|


@pytest.mark.parametrize("B,R,L,H,causal", [
    (1, 2, 64, 64, False), (2, 3, 200, 32, False), (1, 2, 333, 16, True), (2, 2, 300, 128, False),
    (4, 16, 2048, 64, False), (4, 16, 2048, 64, True),       # eight-wave kernel
    (2, 64, 1024, 128, False), (2, 64, 1024, 128, True),
    (2, 8, 1000, 64, False),
    (2, 8, 3073, 64, False),                                  # eight 32-row waves, two workgroups per CU
    (8, 12, 1024, 64, True), (3, 16, 2000, 32, True),         # ... causal, one workgroup per CU
    (2, 40, 2048, 128, True), (1, 40, 4000, 64, True),        # causal, query tiles dealt out to a resident grid
])
def test_bf16_inputs(gpu, B, R, L, H, causal):
    q, k, v = (_rand((B, L, R * H), 4200 + L + i).to(torch.bfloat16) for i in range(3))
    got, lse = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, causal=causal, return_lse=True)
    assert got.dtype == torch.bfloat16 and torch.isfinite(got.float()).all()
    mask = causal_mask(B, L) if causal else None
    pairs = sorted({(0, 0), (B - 1, R // 2), (B - 1, R - 1)})
    for b, h in pairs:
        sl = slice(h * H, (h + 1) * H)
        m = None if mask is None else mask[b:b + 1]
        want = attention(q[b:b + 1, :, sl], k[b:b + 1, :, sl], v[b:b + 1, :, sl], H, mask=m)
        assert _max_err(got[b:b + 1, :, sl], want) <= BF16_TOL, (b, h)
        want_lse = attention_lse(q[b:b + 1, :, sl], k[b:b + 1, :, sl], H, mask=m)[0, 0]
        assert ((lse[b, h].cpu() - want_lse).abs() / (1 + want_lse.abs())).max().item() <= 2e-3


@pytest.mark.parametrize("B,R,L,H", [(2, 2, 200, 64), (8, 64, 512, 64), (2, 12, 2048, 64), (2, 12, 2040, 16)])
def test_bf16_additive_mask_and_closed_forms(gpu, B, R, L, H):
    q, k, v = (_rand((B, L, R * H), 4300 + i).to(torch.bfloat16) for i in range(3))
    g = torch.Generator().manual_seed(4310)
    mask = torch.where(torch.rand(B, L, L, generator=g) < 0.3, float("-inf"), 0.0)
    mask = (mask + torch.randn(B, L, L, generator=g) * 0.5).to(torch.bfloat16)
    mask[:, :, 0] = 0
    got = capi.forward(q.to(gpu), k.to(gpu), v.to(gpu), H, mask=mask.to(gpu))
    _check_pairs_tol(got, q, k, v, H, [(0, 0), (B - 1, R - 1)], mask.float(), BF16_TOL)
    # constant V comes back exactly (1.5 is a bf16 number), zero queries give the column mean
    vc = torch.full_like(v, 1.5)
    assert (capi.forward(q.to(gpu), k.to(gpu), vc.to(gpu), H).float() == 1.5).all()
    zq = capi.forward(torch.zeros_like(q).to(gpu), k.to(gpu), v.to(gpu), H)
    want = v.double().mean(dim=1, keepdim=True).float().expand(B, L, R * H)
    assert _max_err(zq, want) <= 2e-3
    with pytest.raises(TypeError):
        capi.forward(q.to(gpu), k.half().to(gpu), v.to(gpu), H)


@pytest.mark.parametrize("B,R,L,H", [(2, 3, 200, 64), (4, 16, 2048, 64), (2, 40, 1024, 128)])
def test_extensions_through_the_compiled_module(gpu, B, R, L, H):
    """fused_attn.attention_forward_ex: causal, mask, log-sum-exp, bf16, the [B, R, L, H] layout and
    strided views give what capi.forward gives (bit for bit: the same library call) and what the
    oracle says."""
    import fused_attn

    q, k, v = (_rand((B, L, R * H), 5300 + L + i) for i in range(3))
    dq, dk, dv = q.to(gpu), k.to(gpu), v.to(gpu)
    plain = fused_attn.attention_forward_ex(dq, dk, dv, H)
    assert isinstance(plain, torch.Tensor) and plain.shape == dq.shape and plain.is_contiguous()
    assert torch.equal(plain, fused_attn.attention_forward(H, min(128, 2 * H), dq, dk, dv))
    out, lse = fused_attn.attention_forward_ex(dq, dk, dv, H, causal=True, return_lse=True)
    want_out, want_lse = capi.forward(dq, dk, dv, H, causal=True, return_lse=True)
    assert torch.equal(out, want_out) and torch.equal(lse, want_lse) and lse.shape == (B, R, L)
    _check_pairs(out, q, k, v, H, [(0, 0), (B - 1, R - 1)], mask=causal_mask(B, L))
    mask = _block_mask("blocks", B, L, 5310 + L)
    masked = fused_attn.attention_forward_ex(dq, dk, dv, H, mask=mask.to(gpu))
    assert torch.equal(masked, capi.forward(dq, dk, dv, H, mask=mask.to(gpu)))
    _check_pairs(masked, q, k, v, H, [(B - 1, R - 1)], mask=mask.float())
    # [B, R, L, H] views of the same data (no copy), output dense in that layout
    q4, k4, v4 = (t.view(B, L, R, H).transpose(1, 2) for t in (dq, dk, dv))
    bhld = fused_attn.attention_forward_ex(q4, k4, v4, H, layout="bhld")
    assert bhld.shape == (B, R, L, H) and bhld.is_contiguous()
    assert torch.equal(bhld.transpose(1, 2).reshape(B, L, R * H), plain)
    # bf16, scale
    qb, kb, vb = (t.to(torch.bfloat16) for t in (dq, dk, dv))
    assert torch.equal(fused_attn.attention_forward_ex(qb, kb, vb, H), capi.forward(qb, kb, vb, H))
    assert torch.equal(fused_attn.attention_forward_ex(dq, dk, dv, H, scale=0.3), capi.forward(dq, dk, dv, H, scale=0.3))
    # rejections that need device tensors
    with pytest.raises(RuntimeError, match="cannot be combined"):
        fused_attn.attention_forward_ex(dq, dk, dv, H, mask=mask.to(gpu), causal=True)
    with pytest.raises(RuntimeError, match="strides of queries"):
        fused_attn.attention_forward_ex(dq, torch.zeros(B, L, 2 * R * H, dtype=torch.float16, device=gpu)[:, :, :R * H], dv, H)
    with pytest.raises(RuntimeError, match="dtype of queries"):
        fused_attn.attention_forward_ex(dq, kb, dv, H)
    with pytest.raises(RuntimeError, match="mask must have shape"):
        fused_attn.attention_forward_ex(dq, dk, dv, H, mask=mask.to(gpu)[:, :, :L - 8].contiguous())
    with pytest.raises(RuntimeError, match="last dimension"):
        fused_attn.attention_forward_ex(dq.transpose(1, 2), dk.transpose(1, 2), dv.transpose(1, 2), H)
    with pytest.raises(RuntimeError, match="scale must be"):
        fused_attn.attention_forward_ex(dq, dk, dv, H, scale=-1.0)


def test_causal_with_mask_is_rejected(gpu):
    x = torch.zeros(1, 64, 64, dtype=torch.float16, device=gpu)
    m = torch.zeros(1, 64, 64, dtype=torch.float16, device=gpu)
    with pytest.raises(capi.FusedAttnError):
        capi.forward(x, x, x, 64, mask=m, causal=True)


# ---- argument rejection that needs device tensors ---------------------------------------------------

def test_binding_rejections_on_device_tensors(gpu):
    import fused_attn

    x = torch.zeros(2, 64, 128, dtype=torch.float16, device=gpu)
    with pytest.raises(RuntimeError, match="contiguous"):
        fused_attn.attention_forward(64, 64, x.transpose(0, 1), x, x)
    with pytest.raises(RuntimeError, match="3-D"):
        fused_attn.attention_forward(64, 64, x[0], x, x)
    with pytest.raises(RuntimeError, match="shape of queries"):
        fused_attn.attention_forward(64, 64, x, x[:, :32].contiguous(), x)
    with pytest.raises(RuntimeError, match="multiple of head_dim"):
        fused_attn.attention_forward(128, 64, x[:, :, :64].contiguous(), x[:, :, :64].contiguous(),
                                     x[:, :, :64].contiguous())
    with pytest.raises(RuntimeError, match="mask must have shape"):
        fused_attn.attention_forward(64, 64, x, x, x, torch.zeros(2, 64, 32, dtype=torch.float16, device=gpu))
    # a sequence length that is not a multiple of chunk_size is accepted (the reference rejects it)
    y = torch.zeros(1, 50, 64, dtype=torch.float16, device=gpu)
    assert fused_attn.attention_forward(64, 64, y, y, y).shape == y.shape
