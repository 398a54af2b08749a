"""The drop-in boundary without a GPU: the C-ABI library loads and exports what the header
declares, rejects bad arguments with status codes before any launch, and the torch binding keeps
the reference's entry point (reference src/fused_attn_extention.cu:15-22,119-129) and raises on
arguments the reference rejects (:24-47)."""
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
