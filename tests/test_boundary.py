"""The drop-in boundary without a GPU: the C-ABI library loads and exports what the header
declares, rejects bad arguments with status codes before any launch, and the torch binding keeps
the reference's entry point (reference src/fused_attn_extention.cu:15-22,119-129) and raises on
arguments the reference rejects (:24-47)."""
import ctypes
import inspect
import os
import re

import pytest
import torch

from fused_attention_amd import capi

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(REPO, "include", "fused_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(fa_[a-z_]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    lib = capi.load_library()
    declared = _declared_functions()
    assert declared == set(capi.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name


def test_query_matches_the_supported_head_dims():
    lib = capi.load_library()
    assert [h for h in range(0, 300) if lib.fa_fwd_query(h)] == [16, 32, 64, 128]


def test_status_codes_for_rejected_arguments():
    ok_ptr = 0x1000  # never dereferenced: every case below is rejected during validation
    B, R, L, H = 1, 2, 64, 64
    good = dict(q_ptr=ok_ptr, k_ptr=ok_ptr, v_ptr=ok_ptr, mask_ptr=0, out_ptr=ok_ptr, B=B, R=R, L=L, H=H,
                stride_b=L * R * H, stride_h=H, stride_l=R * H, scale=0.125)

    def status(**kw):
        return capi.fwd_raw(**{**good, **kw})

    assert status(q_ptr=0) == -1 and status(out_ptr=0) == -1
    assert status(H=48) == -2 and status(H=256) == -2 and status(H=0) == -2
    assert status(L=0) == -3 and status(B=0) == -3 and status(R=-1) == -3
    assert status(stride_l=H - 8) == -4          # rows would overlap
    assert status(stride_l=R * H + 4) == -4      # rows not 16-byte aligned
    assert status(stride_h=-H) == -4
    assert status(k_ptr=ok_ptr + 2) == -5
    assert status(L=2 ** 31) == -6
    assert status(B=2 ** 20, R=2 ** 20) == -6
    assert status(stride_l=2 ** 24 + 8, stride_b=2 ** 40) == -6   # row pitch beyond the loaders' 32-bit tile offsets
    lib = capi.load_library()
    assert lib.fa_fwd_ex(ok_ptr, ok_ptr, ok_ptr, None, ok_ptr, None, B, R, L, H, L * R * H, H, R * H, 0.125, 4, None) == -7
    assert lib.fa_fwd_ex(ok_ptr, ok_ptr, ok_ptr, ok_ptr, ok_ptr, None, B, R, L, H, L * R * H, H, R * H, 0.125, 1, None) == -7
    def strided(in_strides, out_strides, flags=0):
        return lib.fa_fwd_strided(ok_ptr, ok_ptr, ok_ptr, None, ok_ptr, None, B, R, L, H, *in_strides, *out_strides,
                                  0.125, flags, None)

    packed = (L * 3 * R * H, H, 3 * R * H)       # q, k, v as slices of [B, L, 3, R, H]
    dense = (L * R * H, H, R * H)
    assert strided(packed, (L * R * H, H, H - 8)) == -4       # output rows would overlap
    assert strided(packed, (L * R * H, H + 4, R * H)) == -4   # output heads not 16-byte aligned
    assert strided((L * R * H, H, R * H + 2), dense) == -4
    assert strided(packed, (2 ** 62 + 8, H, R * H)) == -6         # output extent beyond the index range
    assert strided(packed, dense, flags=8) == -7
    assert status(scale=0.0) == -8 and status(scale=-0.125) == -8 and status(scale=float("nan")) == -8 and status(scale=float("inf")) == -8
    for code in (-1, -2, -3, -4, -5, -6, -7, -8):
        assert "fa_fwd" in capi.strerror(code)
    assert capi.strerror(0) == "success"


def _items_of_plan(plan, heads, L, causal):
    """Replays how the kernels turn a workgroup index into (head, query tile) items
    (fwd_kernel and fwd_kernel_pingpong in fused_attn_kernel_impl.inc) for a launch plan."""
    rows = plan["waves"] * plan["rows_per_wave"]
    tiles = -(-L // rows)
    per_xcd = plan["workgroups"] // 8
    items = []
    for wg in range(plan["workgroups"]):
        logical = (wg % 8) * per_xcd + wg // 8
        if logical >= plan["working"]:
            continue
        if plan["heads_per_xcd"] > 0:                      # causal, tiles dealt out to a resident grid
            w, rnd = wg // 8, 0
            while True:
                j = rnd * per_xcd + (per_xcd - 1 - w if rnd & 1 else w)
                if j >= plan["heads_per_xcd"] * tiles:
                    break
                items.append((wg % 8 + 8 * (j % plan["heads_per_xcd"]), tiles - 1 - j // plan["heads_per_xcd"]))
                rnd += 1
        elif plan["waves"] == 8 and (causal or plan["per_head"] < tiles):   # a pair of tiles per workgroup (causal; some masked launches)
            head, slot = divmod(logical, plan["per_head"])
            items.append((head, tiles - 1 - slot))
            if 2 * slot != tiles - 1:
                items.append((head, slot))
        else:
            head, slot = divmod(logical, plan["per_head"])
            items.append((head, tiles - 1 - slot if causal else slot))
    return items, tiles


def test_every_launch_plan_covers_every_query_tile_once():
    """The launcher's grid and schedule parameters against the kernels' decoding of them, on the
    CPU: every (head, query tile) exactly once, no index out of range, for plain, masked and
    causal launches over shapes that reach every branch of the shape and schedule choice."""
    import random

    rng = random.Random(20261127)
    shapes = [(4, 16, 4096, 64), (1, 32, 16384, 128), (4, 40, 2048, 128), (8, 12, 1024, 64), (2, 8, 3073, 64),
              (2, 40, 2048, 128), (2, 40, 4096, 64), (2, 40, 2300, 128), (1, 40, 2048, 128), (1, 40, 4000, 64),
              (2, 48, 5000, 32), (1, 20, 4096, 64), (16, 16, 500, 16), (1, 1, 1, 16), (3, 5, 7, 32), (1, 500, 256, 64),
              (1, 8, 65537, 64), (64, 12, 128, 64), (1, 96, 100000, 128)]
    for _ in range(400):
        H = rng.choice([16, 32, 64, 128])
        L = rng.choice([rng.randint(1, 300), rng.randint(301, 3000), rng.randint(3001, 20000)])
        heads = rng.choice([1, 3, 8, 12, 16, 20, 24, 40, 48, 64, 80, 96, 120, 160, 256, 320, 640])
        B = rng.choice([b for b in (1, 2, 4, 8) if heads % b == 0])
        shapes.append((B, heads // B, L, H))
    dealt = paired_masks = 0
    for B, R, L, H in shapes:
        for causal, has_mask in ((False, False), (True, False), (False, True)):
            if has_mask and L % 8:
                continue
            plan = capi.launch_plan(B, R, L, H, causal=causal, has_mask=has_mask)
            assert plan["waves"] in (4, 8) and plan["rows_per_wave"] in (32, 64) and plan["workgroups"] % 8 == 0
            assert plan["heads_per_xcd"] == 0 or (causal and plan["waves"] == 8 and H >= 64 and (B * R) % 8 == 0)
            items, tiles = _items_of_plan(plan, B * R, L, causal)
            assert len(items) == B * R * tiles, (B, R, L, H, causal, has_mask, plan)
            assert set(items) == {(h, t) for h in range(B * R) for t in range(tiles)}, (B, R, L, H, causal, has_mask, plan)
            dealt += plan["heads_per_xcd"] > 0
            paired_masks += has_mask and plan["waves"] == 8 and plan["per_head"] < tiles
            if not causal and not has_mask:
                assert plan["per_head"] == tiles
    assert dealt > 10          # the dealt schedule was among the plans
    assert paired_masks > 10   # ... and masked launches in pairs of tiles


def _tiles_of_projection_plan(plan):
    """Replays how qkv_proj_kernel (qkv_proj_kernel.hpp) turns a workgroup index into output tiles
    (row tile, feature tile)."""
    per_xcd = plan["workgroups"] // 8
    tiles_m = plan["tiles"] // plan["tiles_n"]
    band_of = 4
    tiles = []
    for wg in range(plan["workgroups"]):
        logical = (wg % 8) * per_xcd + wg // 8
        if logical >= plan["working"]:
            continue
        for tile in range(logical, plan["tiles"], plan["working"]):
            band, in_band = divmod(tile, band_of * plan["tiles_n"])
            band_rows = min(band_of, tiles_m - band * band_of)
            row_tile = band * band_of + in_band % band_rows
            col_tile = in_band // band_rows
            assert row_tile < tiles_m and col_tile < plan["tiles_n"]
            tiles.append((row_tile, col_tile))
    return tiles, tiles_m


def test_every_projection_plan_covers_every_output_tile_once():
    """fa_qkv_proj's grid parameters against the kernel's decoding of them, on the CPU: every
    256 x 256 output tile exactly once, over shapes with 1 ... 1920 tiles."""
    shapes = [(4, 2048, 5120, 40, 128), (4, 4096, 1024, 16, 64), (1, 8000, 192, 16, 64), (2, 5000, 64, 8, 128),
              (1, 64, 64, 1, 64), (1, 257, 192, 3, 64), (1, 16384, 4096, 32, 128), (1, 5400, 64, 16, 64),
              (3, 2222, 128, 12, 64), (1, 66000, 64, 1, 64), (2, 4096, 64, 11, 64)]
    for B, L, F_in, R, H in shapes:
        plan = capi.projection_plan(B, L, F_in, R, H)
        tiles, tiles_m = _tiles_of_projection_plan(plan)
        assert plan["tiles"] == -(-B * L // 256) * -(-3 * R * H // 256)
        assert plan["working"] == min(plan["tiles"], 256) and plan["workgroups"] >= plan["working"]
        assert len(tiles) == plan["tiles"], (B, L, F_in, R, H, plan)
        assert set(tiles) == {(r, c) for r in range(tiles_m) for c in range(plan["tiles_n"])}, (B, L, R, H, plan)
    with pytest.raises(capi.FusedAttnError):
        capi.projection_plan(1, 64, 100, 1, 64)          # contraction length not a multiple of 64


def test_benchmark_workloads_take_the_kernels_the_documentation_names():
    def plan(B, R, L, H, **kw):
        p = capi.launch_plan(B, R, L, H, **kw)
        return p["waves"], p["rows_per_wave"], p["heads_per_xcd"] > 0

    assert plan(4, 16, 4096, 64) == (8, 64, False)                       # c3: 512 workgroups of 512 queries
    assert plan(1, 32, 16384, 128) == (8, 32, False)                     # c4
    assert plan(4, 40, 2048, 128) == (8, 32, False)                      # README shape
    assert plan(8, 12, 1024, 64) == (8, 64, False)                       # c2
    assert plan(2, 8, 3073, 64) == (8, 32, False)                        # c5b: 256-query workgroups
    assert plan(1, 4, 256, 64) == (4, 32, False)                         # c1
    assert plan(2, 8, 1000, 64) == (4, 32, False)                        # c5a
    assert plan(4, 16, 4096, 64, causal=True) == (8, 64, False)          # one whole round of pairs
    assert plan(1, 32, 16384, 128, causal=True) == (8, 32, False)        # four whole rounds of pairs
    assert plan(4, 40, 2048, 128, causal=True) == (8, 32, True)          # 2.5 rounds of pairs: dealt
    assert plan(2, 40, 4096, 64, causal=True) == (8, 64, True)
    assert plan(2, 48, 5000, 32, causal=True) == (8, 64, False)          # never dealt below head_dim 64
    assert plan(8, 12, 1024, 64, causal=True)[:2] == (8, 32)             # pairs of 256-query tiles
    assert plan(2, 12, 2048, 64, causal=True) == (4, 32, False)
    assert plan(4, 16, 4096, 64, has_mask=True) == (8, 64, False)
    assert plan(1, 40, 2048, 128, has_mask=True) == (8, 32, False)
    assert plan(2, 12, 2048, 64, has_mask=True) == (8, 32, False)
    assert plan(64, 12, 128, 64, has_mask=True) == (4, 32, False)


def test_the_16_row_matrix_tile_is_taken_on_whole_rounds_only():
    tile = lambda B, R, L, H, **kw: capi.launch_plan(B, R, L, H, **kw)["matrix_tile"]
    wgs = lambda B, R, L, H: capi.launch_plan(B, R, L, H)["working"]
    assert (wgs(4, 16, 4096, 64), tile(4, 16, 4096, 64)) == (512, 16)     # c3: two whole rounds
    assert (wgs(4, 16, 2048, 64), tile(4, 16, 2048, 64)) == (256, 16)     # one whole round
    assert (wgs(8, 32, 1000, 64), tile(8, 32, 1000, 64)) == (512, 16)     # ragged tiles make no difference
    assert (wgs(2, 60, 2048, 64), tile(2, 60, 2048, 64)) == (480, 16)     # last round seven eighths full
    assert (wgs(2, 56, 2048, 64), tile(2, 56, 2048, 64)) == (448, 32)     # ... three quarters full
    assert (wgs(6, 16, 2048, 64), tile(6, 16, 2048, 64)) == (384, 32)     # one and a half rounds
    assert (wgs(9, 16, 4096, 64), tile(9, 16, 4096, 64)) == (1152, 32)    # four and a half
    assert (wgs(8, 12, 1024, 64), tile(8, 12, 1024, 64)) == (192, 32)     # c2: less than one round
    assert tile(4, 16, 4096, 64, causal=True) == 16                       # causal: whole rounds of pairs of tiles
    assert tile(2, 85, 2500, 64, causal=True) == 16                       # ... 510 pairs and lone middle tiles
    assert tile(2, 64, 1300, 64, causal=True) == 16                       # ... and where the tiles are dealt out to a resident grid
    assert tile(3, 12, 4096, 64, causal=True) == 32                       # 144 pairs: little more than half a round
    assert tile(3, 20, 4096, 64, causal=True) == 16                       # 240 pairs: causal launches from 7/8 of a round on,
    assert tile(5, 20, 4096, 64, causal=True) == 16                       # ... whatever the last round holds (400 pairs)
    assert tile(5, 20, 2048, 64, causal=True) == 32                       # 200 pairs
    assert tile(4, 16, 4096, 64, has_mask=True) == 32                     # never with a mask
    assert tile(4, 32, 4096, 32) == 32 and tile(16, 16, 4096, 16) == 32   # head_dim 64 and 128 only
    assert (wgs(1, 32, 16384, 128), tile(1, 32, 16384, 128)) == (2048, 16)    # c4: eight rounds of 256-query workgroups
    assert (wgs(4, 40, 2048, 128), tile(4, 40, 2048, 128)) == (1280, 16)      # the reference's benchmark shape: five rounds
    assert (wgs(1, 28, 2048, 128), tile(1, 28, 2048, 128)) == (224, 16)       # seven eighths of a round
    assert (wgs(1, 48, 2048, 128), tile(1, 48, 2048, 128)) == (384, 32)       # one and a half rounds
    assert (wgs(1, 24, 2048, 128), tile(1, 24, 2048, 128)) == (192, 32)
    assert tile(1, 32, 16384, 128, causal=True) == 16 and tile(4, 40, 2048, 128, causal=True) == 16   # pairs; dealt
    assert tile(4, 40, 2048, 128, has_mask=True) == 32


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", os.path.join(REPO, "does_not_exist.so"))
    with pytest.raises(OSError, match="no fallback"):
        capi.load_library()


def test_binding_signature_matches_the_reference():
    import fused_attn

    doc = fused_attn.attention_forward.__doc__
    names = re.findall(r"(\w+): ", doc.split("->")[0])
    assert names == ["head_dim", "chunk_size", "queries", "keys", "values", "mask"]
    assert "mask: torch.Tensor | None = None" in doc or "mask: Optional[torch.Tensor] = None" in doc
    assert "Fused multihead attention" in doc


def test_binding_exposes_the_projection_front_end():
    import fused_attn

    doc = fused_attn.qkv_projection.__doc__
    names = re.findall(r"(\w+): ", doc.split("->")[0])
    assert names == ["hidden", "weight", "bias", "num_heads", "head_dim", "rope_cos", "rope_sin"]
    x = torch.zeros(1, 64, 64, dtype=torch.float16)
    w = torch.zeros(64, 192, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU tensor"):          # host tensors never reach the library
        fused_attn.qkv_projection(x, w, None, 1, 64)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        fused_attn.qkv_projection(x.float(), w.float(), None, 1, 64)
    with pytest.raises(ValueError, match="GPU of x"):
        capi.qkv_project(x, w, 1, 64)
    with pytest.raises(ValueError, match="w must have shape"):
        capi.qkv_project(x, w[:, :128], 1, 64)
    with pytest.raises(ValueError, match="multiple of 64"):
        capi.qkv_project(x, torch.zeros(64, 96, dtype=torch.float16), 1, 32)      # slices of 32 features
    with pytest.raises(ValueError, match="F_in"):
        capi.qkv_project(torch.zeros(1, 64, 96, dtype=torch.float16), torch.zeros(96, 192, dtype=torch.float16), 1, 64)
    with pytest.raises(ValueError, match="head_dim must be"):
        capi.qkv_project(x, w, 1, 48)
    with pytest.raises(ValueError, match="pair"):
        capi.qkv_project(x, w, 1, 64, rope=torch.zeros(64, 32))                    # one tensor is not a pair of tables
    # the library's own shape and size codes, through the entry that never launches (pointer and
    # alignment codes need real allocations: tests/test_qkv_proj.py)
    lib = capi.load_library()
    out = (ctypes.c_int * 4)()
    assert lib.fa_qkv_proj_plan(1, 64, 96, 1, 64, out) == -3     # F_in not a multiple of 64
    assert lib.fa_qkv_proj_plan(1, 64, 64, 3, 16, out) == -3     # R * H not a multiple of 64
    assert lib.fa_qkv_proj_plan(1, 64, 64, 1, 48, out) == -2
    assert lib.fa_qkv_proj_plan(1, 0, 64, 1, 64, out) == -3
    assert lib.fa_qkv_proj_plan(2 ** 20, 2 ** 12, 64, 1, 64, out) == -6
    assert lib.fa_qkv_proj_plan(1, 64, 64, 1, 64, None) == -1
    assert lib.fa_qkv_proj_plan(1, 64, 64, 1, 64, out) == 0


def test_binding_exposes_the_extensions_of_the_c_abi():
    """attention_forward_ex: names, defaults, and every rejection that needs no GPU."""
    import fused_attn

    doc = fused_attn.attention_forward_ex.__doc__
    names = re.findall(r"(\w+): ", doc.split("->")[0])
    assert names == ["queries", "keys", "values", "head_dim", "mask", "causal", "return_lse", "layout", "scale"]
    assert "causal: bool = False" in doc and "return_lse: bool = False" in doc and "layout: str = 'blf'" in doc
    x = torch.zeros(2, 64, 128, dtype=torch.float16)

    def rejected(match, *args, **kw):
        with pytest.raises(RuntimeError, match=match):
            fused_attn.attention_forward_ex(*args, **kw)

    rejected("GPU tensor", x, x, x, 64)
    rejected("head_dim must be", x, x, x, 48)
    rejected("float16 or bfloat16", x.float(), x.float(), x.float(), 64)
    rejected("layout must be", x, x, x, 64, layout="bshd")
    rejected("takes 4-D", x, x, x, 64, layout="bhld")
    rejected("takes 3-D", x.view(2, 64, 2, 64), x.view(2, 64, 2, 64), x.view(2, 64, 2, 64), 64)
    with pytest.raises(TypeError):
        fused_attn.attention_forward_ex(x, x, 64)


def test_reference_bias_follows_the_sequence_length():
    """11 - ceil(log2 L) inside [-8, 6], as the launcher computes it (exported for this purpose)."""
    lib = capi.load_library()
    want = {1: 6, 2: 6, 32: 6, 33: 5, 64: 5, 1000: 1, 1024: 1, 1025: 0, 3073: -1, 4096: -1, 4097: -2, 16384: -3,
            65536: -5, 65537: -6, 2 ** 19: -8, 2 ** 19 + 1: -8, 2 ** 22: -8, 2 ** 31 - 4097: -8}
    for L, b in want.items():
        assert lib.fa_fwd_reference_bias(L) == float(b), L
    lo = [lib.fa_fwd_reference_bias(L) for L in range(1, 5000)]
    assert all(a >= b for a, b in zip(lo, lo[1:]))               # never grows with the length
    # the share of a row that L weights at the bottom of the fp16 range can take: L 2^-(24 - bias)
    for L in (64, 1000, 4096, 65536, 2 ** 19):
        assert L * 2.0 ** -(24 - lib.fa_fwd_reference_bias(L)) <= 2.0 ** -13 + 1e-12
    assert 2 ** 22 * 2.0 ** -(24 + 8) == 2.0 ** -10              # past the clamp the bound loosens: documented


def test_binding_rejects_what_the_reference_rejects():
    import fused_attn

    x = torch.zeros(1, 64, 128, dtype=torch.float16)
    bad_ints = [(8, 16), (256, 64), (48, 32), (64, 8), (64, 256), (64, 48), (16, 64), (128, 16)]
    for head_dim, chunk in bad_ints:
        with pytest.raises(RuntimeError):
            fused_attn.attention_forward(head_dim, chunk, x, x, x)
    with pytest.raises(RuntimeError, match="float16"):
        fused_attn.attention_forward(64, 64, x.float(), x, x)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        fused_attn.attention_forward(64, 64, x, x, x)  # host tensors, as the reference demands a device tensor
    with pytest.raises(TypeError):
        fused_attn.attention_forward(64, 64, x, x)      # values is required


def test_python_wrapper_forwards_to_the_binding():
    import fused_attention_amd

    sig = inspect.signature(fused_attention_amd.attention_forward)
    assert list(sig.parameters) == ["head_dim", "chunk_size", "queries", "keys", "values", "mask"]


def test_ctypes_wrapper_checks_tensors_before_any_address_reaches_the_library(monkeypatch):
    # The library sees raw addresses only: a host tensor, a mask of the wrong extent or a feature
    # count that head_dim does not divide must raise here, not fault on the GPU (the same checks
    # as the binding's, reference src/fused_attn_extention.cu:24-64).
    def no_library():
        raise AssertionError("the library was reached")

    monkeypatch.setattr(capi, "load_library", no_library)
    B, L, R, H = 2, 64, 2, 64
    q = torch.zeros(B, L, R * H, dtype=torch.float16)
    out = torch.zeros_like(q)

    def both(match, exc=ValueError, **kw):
        args = dict(q=q, k=q, v=q, head_dim=H, out=out)
        args.update(kw)
        with pytest.raises(exc, match=match):
            capi.forward(**args)
        with pytest.raises(exc, match=match):
            capi.forward_timed(iters=1, **args)

    both("GPU tensor")                                              # host tensors, everything else in order
    for bad_mask in (torch.zeros(1, L, L), torch.zeros(L, L), torch.zeros(B, 1, L, L), torch.zeros(B, L, L - 8),
                     torch.zeros(B, L + 8, L + 8)):
        both("mask must have shape", mask=bad_mask.half())
    both("mask must be contiguous", mask=torch.zeros(B, L, 2 * L, dtype=torch.float16)[:, :, ::2])
    both("dtype of q", exc=TypeError, mask=torch.zeros(B, L, L))
    both("multiple of head_dim", head_dim=128, q=q[:, :, :H + 32], k=q[:, :, :H + 32], v=q[:, :, :H + 32],
         out=out[:, :, :H + 32])
    both("head_dim must be", head_dim=48)
    both("one shape", k=q[:, :32])
    both("same strides", k=torch.zeros(B, L, 2 * R * H, dtype=torch.float16)[:, :, :R * H])
    both("3-D", q=q[0], k=q[0], v=q[0], out=out[0])
    both("4-D", layout="bhld")
    both("last dimension", layout="bhld", q=q.view(B, L, R, H), k=q.view(B, L, R, H), v=q.view(B, L, R, H),
         out=out.view(B, L, R, H), head_dim=32)
    both("float16 or bfloat16", exc=TypeError, q=q.float(), k=q.float(), v=q.float(), out=out.float())
    both("torch.Tensor", exc=TypeError, k=[1, 2, 3])
    with pytest.raises(ValueError, match="shape of q"):
        capi.forward(q, q, q, H, out=out[:, :32])


def test_bench_refuses_more_than_one_gpu_and_a_machine_without_one():
    """bench.py measures one GPU; with --gpus 2 it says so and exits, and on a machine without a
    GPU it fails instead of timing anything else."""
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stdout + r.stderr)
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--steps", "1", "--warmup", "0"],
                           capture_output=True, text=True)
        assert r.returncode != 0 and "needs a GPU" in (r.stdout + r.stderr)
        assert '"metric"' not in r.stdout
