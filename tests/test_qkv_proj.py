"""GPU parity of the fused QKV projection front end (fa_qkv_proj) against the CPU oracle, and the
projection feeding the attention kernel through views of its packed output.

Tolerance: the projection accumulates in float32 and rounds once to fp16, so against the float32
oracle the error is the fp16 rounding of the result: |got - want| <= 2e-3 + 1e-3 |want| (bf16:
8 significant bits, 2e-2 + 1e-2 |want|).
"""
import math

import pytest
import torch

from fused_attention_amd import capi
from oracle import attention, qkv_projection, rope_tables

pytestmark = pytest.mark.gpu


def _rand(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(torch.float16)


def _close(got, want, atol=2e-3, rtol=1e-3):
    got = got.float().cpu()
    assert torch.isfinite(got).all()
    excess = (got - want).abs() - (atol + rtol * want.abs())
    assert excess.max().item() <= 0, "max excess %.3e" % excess.max().item()


@pytest.mark.parametrize("B,L,Fin,R,H", [
    (1, 64, 64, 1, 64),          # one tile, mostly empty
    (2, 300, 128, 2, 64),        # ragged rows, one feature tile partly filled
    (1, 257, 192, 3, 64),        # one row into the second row tile; 576 features = 2.25 tiles
    (3, 100, 64, 4, 16),         # head_dim 16
    (2, 129, 256, 6, 32),        # head_dim 32
    (1, 1000, 512, 4, 128),      # head_dim 128
    (4, 512, 1024, 16, 64),      # eight row tiles x twelve feature tiles
    (1, 8000, 192, 16, 64),      # 384 tiles on 256 workgroups: a second tile behind the first, three slices per tile
    (2, 5000, 64, 8, 128),       # 480 tiles of one slice each: every step ends a tile
    (1, 5476, 128, 16, 64),      # 264 tiles: eight workgroups take a second one; the last row tile holds 100 rows
])
@pytest.mark.parametrize("mode", ["plain", "bias", "rope", "bias+rope"])
def test_projection_matches_the_oracle(gpu, B, L, Fin, R, H, mode):
    F = R * H
    x = _rand((B, L, Fin), 7000 + L)
    w = _rand((Fin, 3 * F), 7001 + L, 1.0 / math.sqrt(Fin))
    bias = _rand((3 * F,), 7002 + L) if "bias" in mode else None
    rope = rope_tables(L, H) if "rope" in mode else None
    want = qkv_projection(x, w, bias, R, H, *(rope or (None, None)))
    got = capi.qkv_project(x.to(gpu), w.to(gpu), R, H, bias=bias.to(gpu) if bias is not None else None,
                           rope=tuple(t.to(gpu) for t in rope) if rope else None)
    assert got.shape == (B, L, 3, F) and got.dtype == torch.float16
    _close(got, want)


def test_projection_closed_forms_on_the_gpu(gpu):
    # identity weights return the input three times, bit for bit; one-hot columns pick input features
    B, L, R, H = 2, 333, 4, 64
    F = R * H
    x = _rand((B, L, F), 7100)
    eye3 = torch.eye(F).repeat(1, 3).half()
    got = capi.qkv_project(x.to(gpu), eye3.to(gpu), R, H).cpu()
    for s in range(3):
        assert torch.equal(got[:, :, s], x)
    w = torch.zeros(F, 3 * F)
    w[5, 0], w[7, F + 1], w[F - 1, 3 * F - 1] = 1.0, 2.0, -1.0
    got = capi.qkv_project(x.to(gpu), w.half().to(gpu), R, H).cpu()
    assert torch.equal(got[:, :, 0, 0], x[:, :, 5]) and torch.equal(got[:, :, 1, 1], (2.0 * x[:, :, 7].float()).half())
    assert torch.equal(got[:, :, 2, F - 1], -x[:, :, F - 1])
    got[:, :, 0, 0], got[:, :, 1, 1], got[:, :, 2, F - 1] = 0, 0, 0
    assert got.abs().sum().item() == 0
    # the rotation at position 0 is the identity, and rotations keep the norm of every head
    cos, sin = rope_tables(L, H)
    rot = capi.qkv_project(x.to(gpu), eye3.to(gpu), R, H, rope=(cos.to(gpu), sin.to(gpu))).float().cpu()
    assert torch.equal(rot[:, 0], x[:, 0].float().unsqueeze(1).expand(B, 3, F))
    assert torch.equal(rot[:, :, 2], x.float())
    n_in = x.float().view(B, L, R, H).norm(dim=-1)
    n_out = rot[:, :, 0].view(B, L, R, H).norm(dim=-1)
    assert (n_in - n_out).abs().max().item() <= 2e-2


def test_bf16_projection(gpu):
    B, L, Fin, R, H = 2, 300, 256, 4, 64
    x = _rand((B, L, Fin), 7200).to(torch.bfloat16)
    w = _rand((Fin, 3 * R * H), 7201, 1.0 / 16).to(torch.bfloat16)
    bias = _rand((3 * R * H,), 7202).to(torch.bfloat16)
    rope = rope_tables(L, H)
    want = qkv_projection(x, w, bias, R, H, *rope)
    got = capi.qkv_project(x.to(gpu), w.to(gpu), R, H, bias=bias.to(gpu), rope=tuple(t.to(gpu) for t in rope))
    assert got.dtype == torch.bfloat16
    _close(got, want, atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize("B,L,R,H,causal", [(2, 500, 4, 64, False), (1, 2048, 8, 128, True), (4, 1024, 12, 64, False)])
def test_projection_feeds_the_attention_kernel_without_a_copy(gpu, B, L, R, H, causal):
    # hidden state -> packed qkv (with rotary encoding) -> attention over the three views: against
    # the oracle's projection followed by the oracle's attention on the fp16-rounded q, k, v
    F = R * H
    x = _rand((B, L, F), 7300 + L)
    w = _rand((F, 3 * F), 7301 + L, 1.0 / math.sqrt(F))
    rope = rope_tables(L, H)
    qkv = capi.qkv_project(x.to(gpu), w.to(gpu), R, H, rope=tuple(t.to(gpu) for t in rope))
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    assert not q.is_contiguous() and q.data_ptr() == qkv.data_ptr()
    got = capi.forward(q, k, v, H, causal=causal)
    _close(qkv, qkv_projection(x, w, None, R, H, *rope))
    qc, kc, vc = (t.cpu().contiguous() for t in (q, k, v))
    mask = None
    if causal:
        from oracle import causal_mask

        mask = causal_mask(B, L)
    want = attention(qc, kc, vc, H, mask=mask)
    assert (got.float().cpu() - want).abs().max().item() <= 5e-3


def test_projection_rejections(gpu):
    x = _rand((1, 64, 64), 7400).to(gpu)
    w = _rand((64, 192), 7401).to(gpu)
    lib = capi.load_library()
    ok = (x.data_ptr(), w.data_ptr(), None, torch.empty(1, 64, 3, 64, dtype=torch.float16, device=gpu).data_ptr())

    def status(B=1, L=64, Fin=64, R=1, H=64, cos=None, sin=None, flags=0, ptrs=ok):
        return lib.fa_qkv_proj(*ptrs, B, L, Fin, R, H, cos, sin, flags, None)

    assert status() == 0
    assert status(Fin=96) == -3 and status(R=1, H=32) == -3          # contraction and slice width: multiples of 64
    assert status(H=48) == -2 and status(L=0) == -3 and status(flags=1) == -7
    assert status(cos=x.data_ptr()) == -1                             # one table without the other
    assert status(ptrs=(None,) + ok[1:]) == -1 and status(ptrs=(ok[0] + 2,) + ok[1:]) == -5
    torch.cuda.synchronize()
    with pytest.raises(ValueError, match="w must have shape"):
        capi.qkv_project(x, w[:, :128], 1, 64)
    with pytest.raises(ValueError, match="rope cos"):
        capi.qkv_project(x, w, 1, 64, rope=(torch.zeros(64, 16, device=gpu), torch.zeros(64, 32, device=gpu)))
    with pytest.raises(ValueError, match="GPU of x"):
        capi.qkv_project(x, w.cpu(), 1, 64)


def test_projection_through_the_torch_binding(gpu):
    import fused_attn

    B, L, Fin, R, H = 2, 200, 128, 2, 64
    x, w, b = _rand((B, L, Fin), 7500), _rand((Fin, 3 * R * H), 7501, 0.1), _rand((3 * R * H,), 7502)
    cos, sin = rope_tables(L, H)
    got = fused_attn.qkv_projection(x.to(gpu), w.to(gpu), b.to(gpu), R, H, cos.to(gpu), sin.to(gpu))
    assert got.shape == (B, L, 3, R * H) and got.dtype == torch.float16 and got.device.type == "cuda"
    _close(got, qkv_projection(x, w, b, R, H, cos, sin))
    same = capi.qkv_project(x.to(gpu), w.to(gpu), R, H, bias=b.to(gpu), rope=(cos.to(gpu), sin.to(gpu)))
    assert torch.equal(got, same)
    with pytest.raises(RuntimeError, match="weight must have shape"):
        fused_attn.qkv_projection(x.to(gpu), w[:, :64].contiguous().to(gpu), None, R, H)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        fused_attn.qkv_projection(x, w, None, R, H)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        fused_attn.qkv_projection(x.to(gpu), w[:, :96].contiguous().to(gpu), None, 1, 32)


@pytest.mark.parametrize("B,L,Fin,R,H,causal", [(2, 200, 128, 2, 64, False), (2, 1024, 512, 8, 64, True),
                                                 (1, 2048, 256, 16, 128, False)])
def test_projection_into_attention_through_the_compiled_module(gpu, B, L, Fin, R, H, causal):
    """fused_attn.qkv_projection -> fused_attn.attention_forward_ex on the three slices of the packed
    tensor, no copy in between, against oracle projection + oracle attention."""
    import fused_attn
    from oracle import attention, causal_mask

    x, w, b = _rand((B, L, Fin), 7600), _rand((Fin, 3 * R * H), 7601, 1.0 / math.sqrt(Fin)), _rand((3 * R * H,), 7602, 0.1)
    cos, sin = rope_tables(L, H)
    qkv = fused_attn.qkv_projection(x.to(gpu), w.to(gpu), b.to(gpu), R, H, cos.to(gpu), sin.to(gpu))
    views = [qkv[:, :, s] for s in range(3)]
    assert all(not t.is_contiguous() and t.data_ptr() == qkv.data_ptr() + s * R * H * 2 for s, t in enumerate(views))
    out = fused_attn.attention_forward_ex(*views, H, causal=causal)
    assert out.shape == (B, L, R * H) and out.is_contiguous()
    ref = qkv_projection(x, w, b, R, H, cos, sin)                 # float32 [B, L, 3, R H]
    ref = ref.to(torch.float16).float()                           # the kernel's q, k, v are rounded to fp16
    want = attention(ref[:, :, 0].contiguous(), ref[:, :, 1].contiguous(), ref[:, :, 2].contiguous(), H,
                     mask=causal_mask(B, L) if causal else None)
    assert torch.isfinite(out.float()).all()
    assert (out.float().cpu() - want).abs().max().item() <= 5e-3


def test_projection_and_attention_captured_in_one_graph(gpu):
    # Neither launch allocates or clears anything, so hidden state -> qkv -> attention is recorded as
    # two kernel nodes; replays follow the contents of the captured input buffer and agree bitwise
    # with eager launches, with eager work between the replays.
    B, L, R, H = 2, 512, 8, 64
    F = R * H
    x = _rand((B, L, F), 7600).to(gpu)
    w = _rand((F, 3 * F), 7601, 1.0 / math.sqrt(F)).to(gpu)
    rope = tuple(t.to(gpu) for t in rope_tables(L, H))
    qkv = torch.empty(B, L, 3, F, dtype=torch.float16, device=gpu)
    out = torch.empty(B, L, F, dtype=torch.float16, device=gpu)

    def run(qkv_buf, out_buf):
        capi.qkv_project(x, w, R, H, rope=rope, out=qkv_buf)
        capi.forward(qkv_buf[:, :, 0], qkv_buf[:, :, 1], qkv_buf[:, :, 2], H, out=out_buf, causal=True)

    run(qkv, out)                                    # warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(qkv, out)
    for rep in range(3):
        if rep:
            x.copy_(_rand((B, L, F), 7610 + rep))
        qkv_e, out_e = torch.empty_like(qkv), torch.empty_like(out)
        run(qkv_e, out_e)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(qkv, qkv_e) and torch.equal(out, out_e)
    _close(qkv, qkv_projection(x.cpu(), w.cpu(), None, R, H, *(t.cpu() for t in rope)))
