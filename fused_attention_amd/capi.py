"""ctypes view of libfused_attn_gfx950.so (the C ABI declared in include/fused_attn.h).

`forward` and `forward_timed` check what the library cannot see from raw addresses (tensor
devices, shapes, the mask's extent) and raise before any address reaches it; value ranges,
alignment and strides are checked by the library and reported through its status codes.
"""
import ctypes
import math
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libfused_attn_gfx950.so")

# every symbol include/fused_attn.h declares
EXPORTS = ("fa_fwd", "fa_fwd_ex", "fa_fwd_strided", "fa_fwd_plan", "fa_fwd_query", "fa_fwd_reference_bias", "fa_strerror",
           "fa_fwd_timed", "fa_fwd_timed_ex", "fa_qkv_proj", "fa_qkv_proj_plan")
FLAG_CAUSAL = 1
FLAG_BF16 = 2

_lib = None


class FusedAttnError(RuntimeError):
    """A non-zero status from the kernel library."""

    def __init__(self, status, text):
        super().__init__("%s (status %d)" % (text, status))
        self.status = status


def load_library():
    """Loads the kernel library once.  Raises OSError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise OSError(
            "%s is missing: build it with `python -m fused_attention_amd.build` "
            "(there is no fallback implementation)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    i64, vp, f32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float
    fwd_args = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, f32, vp]
    lib.fa_fwd.argtypes = fwd_args
    lib.fa_fwd.restype = ctypes.c_int
    lib.fa_fwd_ex.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, f32,
                              ctypes.c_int, vp]
    lib.fa_fwd_ex.restype = ctypes.c_int
    lib.fa_fwd_strided.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64,
                                   f32, ctypes.c_int, vp]
    lib.fa_fwd_strided.restype = ctypes.c_int
    lib.fa_fwd_timed.argtypes = fwd_args + [ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
    lib.fa_fwd_timed.restype = ctypes.c_int
    lib.fa_fwd_timed_ex.argtypes = lib.fa_fwd_strided.argtypes + [ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
    lib.fa_fwd_timed_ex.restype = ctypes.c_int
    lib.fa_qkv_proj.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, vp, ctypes.c_int, vp]
    lib.fa_qkv_proj.restype = ctypes.c_int
    lib.fa_qkv_proj_plan.argtypes = [i64, i64, i64, i64, i64, ctypes.POINTER(ctypes.c_int)]
    lib.fa_qkv_proj_plan.restype = ctypes.c_int
    lib.fa_fwd_plan.argtypes = [i64, i64, i64, i64, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int)]
    lib.fa_fwd_plan.restype = ctypes.c_int
    lib.fa_fwd_query.argtypes = [i64]
    lib.fa_fwd_query.restype = ctypes.c_int
    lib.fa_fwd_reference_bias.argtypes = [i64]
    lib.fa_fwd_reference_bias.restype = f32
    lib.fa_strerror.argtypes = [ctypes.c_int]
    lib.fa_strerror.restype = ctypes.c_char_p
    _lib = lib
    return lib


def strerror(status):
    return load_library().fa_strerror(int(status)).decode()


def _check(status):
    if status != 0:
        raise FusedAttnError(status, strerror(status))


def launch_plan(B, R, L, H, causal=False, has_mask=False):
    """What fa_fwd_plan reports for a problem, as a dict.  Needs no GPU."""
    out = (ctypes.c_int * 7)()
    _check(load_library().fa_fwd_plan(B, R, L, H, FLAG_CAUSAL if causal else 0, 1 if has_mask else 0, out))
    keys = ("waves", "rows_per_wave", "workgroups", "working", "per_head", "heads_per_xcd", "matrix_tile")
    return dict(zip(keys, out))


def projection_plan(B, L, F_in, R, H):
    """What fa_qkv_proj_plan reports for a problem, as a dict.  Needs no GPU."""
    out = (ctypes.c_int * 4)()
    _check(load_library().fa_qkv_proj_plan(B, L, F_in, R, H, out))
    keys = ("workgroups", "working", "tiles", "tiles_n")
    return dict(zip(keys, out))


def fwd_raw(q_ptr, k_ptr, v_ptr, mask_ptr, out_ptr, B, R, L, H, stride_b, stride_h, stride_l,
            scale, stream=0):
    """fa_fwd on raw device addresses (ints).  Returns the status code without raising."""
    return load_library().fa_fwd(q_ptr, k_ptr, v_ptr, mask_ptr or None, out_ptr, B, R, L, H,
                                 stride_b, stride_h, stride_l, scale, stream or None)


def _layout(q, head_dim, layout):
    if layout == "blf":      # [B, L, R*H]: the reference layout
        B, L, F = q.shape
        R = F // head_dim
        return B, R, L, L * F, head_dim, F
    if layout == "bhld":     # [B, R, L, H]
        B, R, L, H = q.shape
        return B, R, L, R * L * H, L * H, H
    raise ValueError("layout must be 'blf' or 'bhld'")


def _strides(t, head_dim, layout, name):
    """(stride_b, stride_h, stride_l) in elements of a tensor or view whose last dimension is dense."""
    if t.stride(-1) != 1:
        raise ValueError("%s: the last dimension must be contiguous" % name)
    if layout == "blf":
        return t.stride(0), head_dim, t.stride(1)
    return t.stride(0), t.stride(1), t.stride(2)


def _current_stream(q):
    import torch

    return torch.cuda.current_stream(q.device).cuda_stream


def _checked_problem(q, k, v, head_dim, out, mask, layout):
    """Everything the library cannot see from raw addresses, checked before any address reaches it
    (the same checks as the torch binding, reference src/fused_attn_extention.cu:24-64): dtypes,
    GPU residency on one device, dimensionality, equal shapes and strides, num_features a
    multiple of head_dim, a contiguous [B, L, L] mask.  Returns (B, R, L, q/k/v strides).
    Raises TypeError / ValueError; needs neither the library nor a GPU to do so."""
    import torch

    named = (("q", q), ("k", k), ("v", v), ("out", out), ("mask", mask))
    for name, t in named:
        if t is not None and not isinstance(t, torch.Tensor):
            raise TypeError("%s must be a torch.Tensor, got %s" % (name, type(t).__name__))
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("q, k, v must be float16 or bfloat16, got %s" % q.dtype)
    for name, t in named[1:]:
        if t is not None and t.dtype != q.dtype:
            raise TypeError("%s must have the dtype of q (%s), got %s" % (name, q.dtype, t.dtype))
    if int(head_dim) != head_dim or head_dim not in (16, 32, 64, 128):
        raise ValueError("head_dim must be 16, 32, 64 or 128, got %r" % (head_dim,))
    if layout not in ("blf", "bhld"):
        raise ValueError("layout must be 'blf' or 'bhld'")
    want_dim = 3 if layout == "blf" else 4
    if q.dim() != want_dim:
        raise ValueError("layout %r takes %d-D tensors, q has %d dimensions" % (layout, want_dim, q.dim()))
    if layout == "blf":
        if q.shape[2] % head_dim != 0:
            raise ValueError("num_features (%d) must be a multiple of head_dim (%d)" % (q.shape[2], head_dim))
    elif q.shape[3] != head_dim:
        raise ValueError("the last dimension (%d) must equal head_dim (%d)" % (q.shape[3], head_dim))
    if min(q.shape) < 1:
        raise ValueError("q must not have an empty dimension, got %s" % (tuple(q.shape),))
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k, v must have one shape")
    if out is not None and out.shape != q.shape:
        raise ValueError("out must have the shape of q")
    B, R, L = _layout(q, head_dim, layout)[:3]
    strides = _strides(q, head_dim, layout, "q")
    if _strides(k, head_dim, layout, "k") != strides or _strides(v, head_dim, layout, "v") != strides:
        raise ValueError("q, k, v must have the same strides")
    if mask is not None:
        if tuple(mask.shape) != (B, L, L):
            raise ValueError("mask must have shape [batch, seq_len, seq_len] = [%d, %d, %d], got %s"
                             % (B, L, L, tuple(mask.shape)))
        if not mask.is_contiguous():
            raise ValueError("mask must be contiguous")
    # last, so that the checks above can be exercised on host tensors
    for name, t in named:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("%s must be a GPU tensor, got device %s" % (name, t.device))
        if t.device != q.device:
            raise ValueError("%s is on %s but q is on %s" % (name, t.device, q.device))
    return B, R, L, strides


def forward(q, k, v, head_dim, out=None, mask=None, layout="blf", scale=None, causal=False,
            return_lse=False):
    """Runs fa_fwd_strided on torch GPU tensors (fp16 or bf16) on torch's current stream.

    layout 'blf' takes [B, L, R*head_dim] tensors, 'bhld' takes [B, R, L, head_dim] tensors.
    q, k and v may be views (slices of one packed projection output, say) as long as their last
    dimension is dense and the three have the same strides; `out` may be a view of its own.  The
    mask is contiguous [B, L, L].  causal=True restricts query i to keys j <= i.  q, k, v (and out,
    mask when given) must share one dtype and one GPU; bfloat16 tensors set FA_FLAG_BF16.  Returns
    `out` (allocated like q when not given), or (out, lse) with lse a float32 [B, R, L] tensor
    when return_lse is set.
    """
    import torch

    B, R, L, (sb, sh, sl) = _checked_problem(q, k, v, head_dim, out, mask, layout)
    flags = (FLAG_CAUSAL if causal else 0) | (FLAG_BF16 if q.dtype == torch.bfloat16 else 0)
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    ob, oh, ol = _strides(out, head_dim, layout, "out")
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    lse = torch.empty((B, R, L), dtype=torch.float32, device=q.device) if return_lse else None
    with torch.cuda.device(q.device):
        status = load_library().fa_fwd_strided(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr() if mask is not None else None,
            out.data_ptr(), lse.data_ptr() if lse is not None else None, B, R, L, head_dim, sb, sh, sl,
            ob, oh, ol, scale, flags, _current_stream(q) or None)
    _check(status)
    return (out, lse) if return_lse else out


def forward_timed(q, k, v, head_dim, out, iters, mask=None, layout="blf", scale=None, causal=False):
    """Average milliseconds per launch over `iters` back-to-back launches of the launch `forward`
    would make (HIP events on the launch stream, measured inside the library by fa_fwd_timed_ex).
    Same tensors as `forward` (fp16 or bf16, views allowed); `out` is required."""
    import torch

    B, R, L, (sb, sh, sl) = _checked_problem(q, k, v, head_dim, out, mask, layout)
    if out is None:
        raise ValueError("forward_timed needs an `out` tensor")
    flags = (FLAG_CAUSAL if causal else 0) | (FLAG_BF16 if q.dtype == torch.bfloat16 else 0)
    ob, oh, ol = _strides(out, head_dim, layout, "out")
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(q.device):
        status = load_library().fa_fwd_timed_ex(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr() if mask is not None else None,
            out.data_ptr(), None, B, R, L, head_dim, sb, sh, sl, ob, oh, ol, scale, flags,
            _current_stream(q) or None, int(iters), ctypes.byref(ms))
    _check(status)
    return float(ms.value)


def qkv_project(x, w, num_heads, head_dim, bias=None, rope=None, out=None):
    """fa_qkv_proj on torch GPU tensors, on torch's current stream: x [B, L, F_in] times w
    [F_in, 3 * num_heads * head_dim] (+ bias) -> packed [B, L, 3, num_heads * head_dim] (fp16 or
    bf16, like x).  rope = (cos, sin), float32 [L, head_dim / 2] tables of a rotate-half rotary
    encoding applied to the q and k slices.  The three slices out[:, :, s] are views that
    `forward` takes as q, k and v without a copy."""
    import torch

    for name, t in (("x", x), ("w", w), ("bias", bias), ("out", out)):
        if t is not None and not isinstance(t, torch.Tensor):
            raise TypeError("%s must be a torch.Tensor, got %s" % (name, type(t).__name__))
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("x must be float16 or bfloat16, got %s" % x.dtype)
    if x.dim() != 3 or w.dim() != 2:
        raise ValueError("x must be [B, L, F_in] and w [F_in, 3 F]")
    if int(head_dim) != head_dim or head_dim not in (16, 32, 64, 128):
        raise ValueError("head_dim must be 16, 32, 64 or 128, got %r" % (head_dim,))
    if int(num_heads) != num_heads or num_heads < 1:
        raise ValueError("num_heads must be a positive integer, got %r" % (num_heads,))
    B, L, f_in = x.shape
    F = num_heads * head_dim
    if F % 64 != 0:
        raise ValueError("num_heads * head_dim (%d) must be a multiple of 64: the three slices of the packed "
                         "output start on 64-feature boundaries" % F)
    if f_in % 64 != 0:
        raise ValueError("F_in (%d) must be a multiple of 64: the contraction is walked in steps of 64" % f_in)
    if tuple(w.shape) != (f_in, 3 * F):
        raise ValueError("w must have shape [F_in, 3 * num_heads * head_dim] = [%d, %d], got %s"
                         % (f_in, 3 * F, tuple(w.shape)))
    if bias is not None and tuple(bias.shape) != (3 * F,):
        raise ValueError("bias must have shape [%d], got %s" % (3 * F, tuple(bias.shape)))
    if out is None:
        out = torch.empty((B, L, 3, F), dtype=x.dtype, device=x.device)
    elif tuple(out.shape) != (B, L, 3, F):
        raise ValueError("out must have shape [%d, %d, 3, %d], got %s" % (B, L, F, tuple(out.shape)))
    tables = (None, None)
    if rope is not None:
        if isinstance(rope, torch.Tensor) or not isinstance(rope, (tuple, list)) or len(rope) != 2:
            raise ValueError("rope must be a pair (cos, sin) of float32 [L, head_dim / 2] tensors")
        tables = tuple(rope)
        for name, t in zip(("rope cos", "rope sin"), tables):
            if not isinstance(t, torch.Tensor) or t.dtype != torch.float32 or tuple(t.shape) != (L, head_dim // 2):
                raise ValueError("%s must be a float32 tensor of shape [%d, %d]" % (name, L, head_dim // 2))
    for name, t in (("x", x), ("w", w), ("bias", bias), ("out", out), ("rope cos", tables[0]), ("rope sin", tables[1])):
        if t is None:
            continue
        if name in ("w", "bias", "out") and t.dtype != x.dtype:
            raise TypeError("%s must have the dtype of x (%s), got %s" % (name, x.dtype, t.dtype))
        if not t.is_contiguous():
            raise ValueError("%s must be contiguous" % name)
        if not t.is_cuda or t.device != x.device:
            raise ValueError("%s must be on the GPU of x, got device %s" % (name, t.device))
    flags = FLAG_BF16 if x.dtype == torch.bfloat16 else 0
    with torch.cuda.device(x.device):
        status = load_library().fa_qkv_proj(
            x.data_ptr(), w.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(),
            B, L, f_in, num_heads, head_dim, tables[0].data_ptr() if rope is not None else None,
            tables[1].data_ptr() if rope is not None else None, flags, _current_stream(x) or None)
    _check(status)
    return out
