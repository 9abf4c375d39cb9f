"""Python entry points of the kernels in libgcg_hip.so (C ABI: include/gcg.h).

Two bindings of the same library: the ``torch.ops.gcg`` operators of the PyTorch extension
(``_ops``; used whenever it is built, traceable by ``torch.compile``) and a plain ctypes binding
(``load()``; host-side queries, the entry points that take caller-owned outputs, and every call
when the extension is absent).  There is no CPU or PyTorch fallback: if the library is missing,
or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

from . import _ops

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
# GCG_HIP_LIB points at another build of the same library (e.g. a tuning variant)
LIB_PATH = os.environ.get("GCG_HIP_LIB") or os.path.join(_CSRC, "libgcg_hip.so")

GCG_F32, GCG_BF16, GCG_F16 = 0, 1, 2
ALGO_AUTO, ALGO_DIRECT, ALGO_WINDOW, ALGO_MFMA = 0, 1, 2, 3
ALGO_NAMES = {"auto": ALGO_AUTO, "direct": ALGO_DIRECT, "window": ALGO_WINDOW, "mfma": ALGO_MFMA}

_DTYPES = {torch.float32: GCG_F32, torch.bfloat16: GCG_BF16, torch.float16: GCG_F16}
GCG_BF16_F32, GCG_F16_F32 = 3, 4       # 16-bit tensors, fp32 filter and arithmetic

# every symbol include/gcg.h declares
EXPORTS = (
    "gcg_strerror", "gcg_last_hip_error", "gcg_time_next_kernel", "gcg_version", "gcg_fwd",
    "gcg_bwd_workspace_bytes", "gcg_bwd", "gcg_bwd_static", "gcg_select_algo", "gcg_route_supported",
    "gcg_fwd_interleaved", "gcg_bwd_interleaved", "gcg_fwd_planar", "gcg_bwd_planar",
    "gcg_dwconv_fwd", "gcg_dwconv_bwd_workspace_bytes", "gcg_dwconv_bwd",
    "gcg_mixer_se_fwd", "gcg_mixer_se_bwd_workspace_bytes", "gcg_mixer_se_bwd",
    "gcg_mixer_se_fwd_planar", "gcg_mixer_se_bwd_planar",
    "gcg_filter_decay_fwd", "gcg_filter_decay_bwd",
    "gcg_mixer_mr_fwd", "gcg_mixer_mr_bwd_workspace_bytes", "gcg_mixer_mr_bwd_scratch_bytes", "gcg_mixer_mr_bwd", "gcg_mixer_mr_fwd_decay", "gcg_mixer_mr_bwd_decay",
    "gcg_mixer_mr_fwd_planar", "gcg_mixer_mr_bwd_planar", "gcg_mixer_mr_fwd_planar_decay", "gcg_mixer_mr_bwd_planar_decay", "gcg_fwd_time_major", "gcg_bwd_time_major_workspace_bytes", "gcg_bwd_time_major",
    "gcg_fwd_decay", "gcg_bwd_decay", "gcg_fwd_interleaved_decay", "gcg_bwd_interleaved_decay",
)

_lock = threading.Lock()
_lib = None
TORCH_OPS = _ops.AVAILABLE          # calls go through torch.ops.gcg (else through ctypes)


class GcgError(RuntimeError):
    """A gcg_* entry point returned a negative code (ctypes binding; the torch operators raise a plain
    RuntimeError with the same text)."""


def load() -> ctypes.CDLL:
    """Load the HIP library built in-tree (``make -C savanna_amd/csrc``)."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C savanna_amd/csrc`. There is no fallback path."
            )
        lib = ctypes.CDLL(LIB_PATH)
        vp, i64, i32, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_size_t
        lib.gcg_strerror.argtypes = [ctypes.c_int]
        lib.gcg_strerror.restype = ctypes.c_char_p
        lib.gcg_last_hip_error.argtypes = []
        lib.gcg_last_hip_error.restype = ctypes.c_int
        lib.gcg_time_next_kernel.argtypes = [vp, vp]
        lib.gcg_time_next_kernel.restype = ctypes.c_int
        lib.gcg_version.argtypes = []
        lib.gcg_version.restype = ctypes.c_int
        lib.gcg_fwd.argtypes = [vp] * 7 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_fwd.restype = ctypes.c_int
        lib.gcg_bwd_workspace_bytes.argtypes = [i64, i64, i32, i32, i32, i32, i32]
        lib.gcg_bwd_workspace_bytes.restype = sz
        lib.gcg_bwd.argtypes = [vp] * 10 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_bwd.restype = ctypes.c_int
        lib.gcg_bwd_static.argtypes = [vp] * 9 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_bwd_static.restype = ctypes.c_int
        lib.gcg_select_algo.argtypes = [i64, i64, i32, i32, i32, i32, i32]
        lib.gcg_select_algo.restype = ctypes.c_int
        lib.gcg_route_supported.argtypes = [i32, i64, i64, i32, i32, i32, i32, i32]
        lib.gcg_route_supported.restype = ctypes.c_int
        lib.gcg_fwd_interleaved.argtypes = [vp] * 3 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_fwd_interleaved.restype = ctypes.c_int
        lib.gcg_bwd_interleaved.argtypes = [vp] * 6 + [sz, i64, i64, i32, i32, i32, i32, i32, i32, vp]
        lib.gcg_bwd_interleaved.restype = ctypes.c_int
        lib.gcg_fwd_planar.argtypes = [vp] * 3 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_fwd_planar.restype = ctypes.c_int
        lib.gcg_bwd_planar.argtypes = [vp] * 6 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_bwd_planar.restype = ctypes.c_int
        lib.gcg_dwconv_fwd.argtypes = [vp] * 3 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_dwconv_fwd.restype = ctypes.c_int
        lib.gcg_dwconv_bwd_workspace_bytes.argtypes = [i64, i64, i32, i32, i32, i32]
        lib.gcg_dwconv_bwd_workspace_bytes.restype = sz
        lib.gcg_dwconv_bwd.argtypes = [vp] * 6 + [sz, i64, i64, i32, i32, i32, i32, vp]
        lib.gcg_dwconv_bwd.restype = ctypes.c_int
        lib.gcg_mixer_se_fwd.argtypes = [vp] * 4 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_se_fwd.restype = ctypes.c_int
        lib.gcg_mixer_se_bwd_workspace_bytes.argtypes = [i64, i64, i32, i32, i32, i32, i32]
        lib.gcg_mixer_se_bwd_workspace_bytes.restype = sz
        lib.gcg_mixer_se_bwd.argtypes = [vp] * 8 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_se_bwd.restype = ctypes.c_int
        lib.gcg_mixer_se_fwd_planar.argtypes = lib.gcg_mixer_se_fwd.argtypes
        lib.gcg_mixer_se_fwd_planar.restype = ctypes.c_int
        lib.gcg_mixer_se_bwd_planar.argtypes = lib.gcg_mixer_se_bwd.argtypes
        lib.gcg_mixer_se_bwd_planar.restype = ctypes.c_int
        lib.gcg_filter_decay_fwd.argtypes = [vp] * 3 + [i32, i32, i32, i32, vp]
        lib.gcg_filter_decay_fwd.restype = ctypes.c_int
        lib.gcg_filter_decay_bwd.argtypes = [vp] * 3 + [i32, i32, i32, i32, vp]
        lib.gcg_filter_decay_bwd.restype = ctypes.c_int
        lib.gcg_mixer_mr_fwd.argtypes = [vp] * 4 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_fwd.restype = ctypes.c_int
        lib.gcg_mixer_mr_bwd_workspace_bytes.argtypes = [i64, i64, i32, i32, i32, i32, i32]
        lib.gcg_mixer_mr_bwd_workspace_bytes.restype = sz
        lib.gcg_mixer_mr_bwd_scratch_bytes.argtypes = [i64, i64, i32, i32, i32, i32, i32]
        lib.gcg_mixer_mr_bwd_scratch_bytes.restype = sz
        lib.gcg_mixer_mr_bwd.argtypes = [vp] * 9 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_bwd.restype = ctypes.c_int
        lib.gcg_mixer_mr_fwd_planar_decay.argtypes = [vp] * 4 + [i32, vp, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_fwd_planar_decay.restype = ctypes.c_int
        lib.gcg_mixer_mr_bwd_planar_decay.argtypes = [vp] * 5 + [i32] + [vp] * 4 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_bwd_planar_decay.restype = ctypes.c_int
        lib.gcg_mixer_mr_fwd_planar.argtypes = [vp] * 4 + [i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_fwd_planar.restype = ctypes.c_int
        lib.gcg_mixer_mr_bwd_planar.argtypes = [vp] * 8 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_bwd_planar.restype = ctypes.c_int
        lib.gcg_mixer_mr_fwd_decay.argtypes = [vp] * 4 + [i32, vp, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_fwd_decay.restype = ctypes.c_int
        lib.gcg_mixer_mr_bwd_decay.argtypes = [vp] * 5 + [i32] + [vp] * 5 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_mixer_mr_bwd_decay.restype = ctypes.c_int
        lib.gcg_fwd_time_major.argtypes = [vp] * 5 + [i64, i64, i32, i32, i32, i32, vp]
        lib.gcg_fwd_time_major.restype = ctypes.c_int
        lib.gcg_bwd_time_major_workspace_bytes.argtypes = [i64, i64, i32, i32, i32, i32]
        lib.gcg_bwd_time_major_workspace_bytes.restype = sz
        lib.gcg_bwd_time_major.argtypes = [vp] * 10 + [sz, i64, i64, i32, i32, i32, i32, vp]
        lib.gcg_bwd_time_major.restype = ctypes.c_int
        lib.gcg_fwd_decay.argtypes = [vp] * 5 + [i32, vp, i64, i64, i32, i32, i32, i32, vp]
        lib.gcg_fwd_decay.restype = ctypes.c_int
        lib.gcg_bwd_decay.argtypes = [vp] * 6 + [i32] + [vp] * 5 + [sz, i64, i64, i32, i32, i32, i32, vp]
        lib.gcg_bwd_decay.restype = ctypes.c_int
        lib.gcg_fwd_interleaved_decay.argtypes = [vp] * 3 + [i32, vp, i64, i64, i32, i32, i32, i32, vp]
        lib.gcg_fwd_interleaved_decay.restype = ctypes.c_int
        lib.gcg_bwd_interleaved_decay.argtypes = [vp] * 4 + [i32] + [vp] * 3 + [sz, i64, i64, i32, i32, i32, i32, i32, vp]
        lib.gcg_bwd_interleaved_decay.restype = ctypes.c_int
        _lib = lib
        return lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16") from None


def gated_code(x: torch.Tensor, h: torch.Tensor) -> int:
    """dtype code of the gated operator: the tensors' dtype, or 16-bit tensors with a float32 filter
    (GCG_BF16_F32 / GCG_F16_F32: fp32 arithmetic and an fp32 filter gradient, no casts around the call)."""
    if h.dtype == x.dtype:
        return dtype_code(x.dtype)
    if h.dtype == torch.float32 and x.dtype in (torch.bfloat16, torch.float16):
        return GCG_BF16_F32 if x.dtype == torch.bfloat16 else GCG_F16_F32
    raise TypeError(f"the filter must have the tensors' dtype, or be float32 with bfloat16 / float16 tensors; "
                    f"got {x.dtype} tensors and a {h.dtype} filter")


def algo_code(algo) -> int:
    if isinstance(algo, str):
        return ALGO_NAMES[algo]
    return int(algo)


def time_next_kernel(start_event, stop_event) -> None:
    """Arm two hipEvent_t handles (integers; timing enabled) for the next fwd / bwd / *_interleaved call on
    this thread: the runtime stamps them at the start and the end of that call's main kernel."""
    check(load().gcg_time_next_kernel(start_event, stop_event), "gcg_time_next_kernel")


def check(rc: int, what: str) -> None:
    if rc != 0:
        lib = load()
        msg = lib.gcg_strerror(rc).decode()
        raise GcgError(f"{what}: {msg} (code {rc}, hipError {lib.gcg_last_hip_error()})")


class _on_device:
    """``torch.cuda.device`` that does nothing when the tensor's device is already current (the
    usual case): the context manager costs several microseconds, which shows at small shapes."""

    __slots__ = ("ctx",)

    def __init__(self, device):
        self.ctx = None if device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def _require_gpu(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            "savanna_amd runs on an MI355X (gfx950) device only; got a tensor on "
            f"{t.device}. There is no CPU path."
        )


def fwd(x, B, C, h, return_bx=False, return_y2=False, algo=ALGO_AUTO, out=None):
    """y (and optionally bx, y2) for contiguous (bs, L, g, dg) inputs and (g, 1, hl) filter.
    ``out``: optional pre-allocated contiguous tensor of x's shape, dtype and device for y."""
    _require_gpu(x)
    if out is not None:
        if out.shape != x.shape or out.dtype != x.dtype or out.device != x.device or not out.is_contiguous():
            raise ValueError("out must be a contiguous tensor with the shape, dtype and device of x")
    if TORCH_OPS:
        a = algo_code(algo)
        if out is not None and not (return_bx or return_y2):
            torch.ops.gcg.fwd_out(x, B, C, h, out, a)
            return None, None, out
        if not (return_bx or return_y2):
            return None, None, torch.ops.gcg.fwd(x, B, C, h, a)
        bx, y2, y = torch.ops.gcg.fwd_full(x, B, C, h, return_bx, return_y2, a)
        if out is not None:
            y = out.copy_(y)
        return (bx if return_bx else None), (y2 if return_y2 else None), y
    lib = load()
    bs, L, g, dg = x.shape
    hl = h.shape[-1]
    y = out if out is not None else torch.empty_like(x)
    y2 = torch.empty_like(x) if return_y2 else None
    bx = torch.empty_like(x) if return_bx else None
    if x.numel() == 0:
        return bx, y2, y
    with _on_device(x.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_fwd(
            x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), y.data_ptr(),
            y2.data_ptr() if y2 is not None else None,
            bx.data_ptr() if bx is not None else None,
            bs, L, g, dg, hl, gated_code(x, h), algo_code(algo), st,
        )
    check(rc, "gcg_fwd")
    return bx, y2, y


def bwd(dy, x, B, C, h, algo=ALGO_AUTO):
    """(dx, dB, dC, dh) for contiguous inputs; dh has h's shape and dtype."""
    _require_gpu(x)
    if TORCH_OPS:
        return torch.ops.gcg.bwd(dy, x, B, C, h, algo_code(algo))
    lib = load()
    bs, L, g, dg = x.shape
    hl = h.shape[-1]
    dx, dB, dC = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    dh = torch.empty_like(h)
    if x.numel() == 0:
        return dx, dB, dC, dh.zero_()
    code, a = gated_code(x, h), algo_code(algo)
    nbytes = lib.gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, a)
    if nbytes == 0:
        raise GcgError("gcg_bwd_workspace_bytes: arguments rejected")
    with _on_device(x.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_bwd(
            dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(),
            dx.data_ptr(), dB.data_ptr(), dC.data_ptr(), dh.data_ptr(),
            ws.data_ptr(), nbytes, bs, L, g, dg, hl, code, a, st,
        )
    check(rc, "gcg_bwd")
    return dx, dB, dC, dh


STATIC_SCRATCH_BYTES = 8 << 20      # GCG_BWD_STATIC_SCRATCH_BYTES


def bwd_static(dy, x, B, C, h, dx, dB, dC, dh, algo=ALGO_AUTO):
    """gcg_bwd_static: the backward into the caller's output tensors with the library's built-in scratch
    array instead of a workspace; nothing is allocated by the call (for callers under graph capture).
    Calls that overlap on one GPU share the array and must be ordered by the caller.
    The C entry point sees pointers only, so the tensors are checked here as gcg_bwd's binding checks them:
    a strided or short output would be written out of bounds by the kernels."""
    lib = load()
    _require_gpu(x)
    if x.dim() != 4:
        raise ValueError("x must be (bs, L, g, dg)")
    bs, L, g, dg = x.shape
    for name, t in (("x", x), ("dy", dy), ("B", B), ("C", C), ("dx", dx), ("dB", dB), ("dC", dC)):
        if t.shape != x.shape or t.dtype != x.dtype or t.device != x.device or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous (bs, L, g, dg) tensor with the dtype and device of x")
    if h.dim() != 3 or h.shape[0] != g or h.shape[1] != 1 or h.device != x.device or not h.is_contiguous():
        raise ValueError("h must be a contiguous (g, 1, hl) tensor on the device of x")
    if dh.shape != h.shape or dh.dtype != h.dtype or dh.device != x.device or not dh.is_contiguous():
        raise ValueError("dh must be a contiguous tensor with the shape, dtype and device of h")
    code = gated_code(x, h)             # raises for a filter type that does not go with the tensors'
    if x.numel() == 0:
        dh.zero_()
        return
    with _on_device(x.device):
        rc = lib.gcg_bwd_static(
            dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(),
            dx.data_ptr(), dB.data_ptr(), dC.data_ptr(), dh.data_ptr(),
            bs, L, g, dg, h.shape[-1], code, algo_code(algo),
            torch.cuda.current_stream().cuda_stream,
        )
    check(rc, "gcg_bwd_static")


def _check_feat(feat, h):
    if feat.dim() != 5 or feat.shape[-1] != 3 or not feat.is_contiguous():
        raise ValueError("feat must be a contiguous (bs, L, g, dg, 3) tensor")
    if h.dim() != 3 or h.shape[0] != feat.shape[2] or h.shape[1] != 1 or not h.is_contiguous():
        raise ValueError("h must be a contiguous (g, 1, hl) tensor")
    gated_code(feat, h)
    if h.device != feat.device:
        raise ValueError("feat and h must share dtype and device")


def fwd_interleaved(feat, h, algo=ALGO_AUTO, out=None):
    """y (bs, L, g, dg) for feat (bs, L, g, dg, 3) with feat[..., 0] = C, [..., 1] = B, [..., 2] = x."""
    _require_gpu(feat)
    if TORCH_OPS and out is None:
        return torch.ops.gcg.fwd_interleaved(feat, h, algo_code(algo))
    lib = load()
    _check_feat(feat, h)
    bs, L, g, dg, _ = feat.shape
    hl = h.shape[-1]
    if out is not None:
        if (out.shape != feat.shape[:4] or out.dtype != feat.dtype or out.device != feat.device
                or not out.is_contiguous()):
            raise ValueError("out must be a contiguous (bs, L, g, dg) tensor with the dtype and device of feat")
    y = out if out is not None else torch.empty(feat.shape[:4], dtype=feat.dtype, device=feat.device)
    if y.numel() == 0:
        return y
    with _on_device(feat.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_fwd_interleaved(feat.data_ptr(), h.data_ptr(), y.data_ptr(), bs, L, g, dg, hl,
                                     gated_code(feat, h), algo_code(algo), st)
    check(rc, "gcg_fwd_interleaved")
    return y


KEEP_OUTPUT = 1       # GCG_KEEP_OUTPUT


def bwd_interleaved(dy, feat, h, algo=ALGO_AUTO, keep_output=False):
    """(dfeat, dh): dfeat has feat's layout, dfeat[..., 0] = dC, [..., 1] = dB, [..., 2] = dx.
    ``keep_output``: dfeat goes to dwconv_bwd next, store it through the cache."""
    _require_gpu(feat)
    if TORCH_OPS:
        return torch.ops.gcg.bwd_interleaved(dy, feat, h, algo_code(algo), bool(keep_output))
    lib = load()
    _check_feat(feat, h)
    bs, L, g, dg, _ = feat.shape
    hl = h.shape[-1]
    if dy.shape != feat.shape[:4] or dy.dtype != feat.dtype or not dy.is_contiguous():
        raise ValueError("dy must be a contiguous (bs, L, g, dg) tensor of feat's dtype")
    dfeat = torch.empty_like(feat)
    dh = torch.empty_like(h)
    if dy.numel() == 0:
        return dfeat, dh.zero_()
    code, a = gated_code(feat, h), algo_code(algo)
    nbytes = lib.gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, a)
    if nbytes == 0:
        raise GcgError("gcg_bwd_workspace_bytes: arguments rejected")
    with _on_device(feat.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=feat.device)
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_bwd_interleaved(dy.data_ptr(), feat.data_ptr(), h.data_ptr(), dfeat.data_ptr(), dh.data_ptr(),
                                     ws.data_ptr(), nbytes, bs, L, g, dg, hl, code, a,
                                     KEEP_OUTPUT if keep_output else 0, st)
    check(rc, "gcg_bwd_interleaved")
    return dfeat, dh


def _check_planar(feat, h):
    if feat.dim() != 5 or feat.shape[2] != 3 or not feat.is_contiguous():
        raise ValueError("feat must be a contiguous (bs, L, 3, g, dg) tensor")
    if h.dim() != 3 or h.shape[0] != feat.shape[3] or h.shape[1] != 1 or not h.is_contiguous():
        raise ValueError("h must be a contiguous (g, 1, hl) tensor")
    gated_code(feat, h)
    if h.device != feat.device:
        raise ValueError("feat and h must share dtype and device")


def fwd_planar(feat, h, algo=ALGO_AUTO):
    """y (bs, L, g, dg) for planar features feat (bs, L, 3, g, dg): feat[:, :, 0] = C, [:, :, 1] = B, [:, :, 2] = x,
    the thirds of each row read in place (block.py:881-884, the split without interleaving)."""
    _require_gpu(feat)
    if TORCH_OPS:
        return torch.ops.gcg.fwd_planar(feat, h, algo_code(algo))
    lib = load()
    _check_planar(feat, h)
    bs, L, _, g, dg = feat.shape
    y = torch.empty(bs, L, g, dg, dtype=feat.dtype, device=feat.device)
    if y.numel() == 0:
        return y
    with _on_device(feat.device):
        rc = lib.gcg_fwd_planar(feat.data_ptr(), h.data_ptr(), y.data_ptr(), bs, L, g, dg, h.shape[-1],
                                gated_code(feat, h), algo_code(algo), torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_fwd_planar")
    return y


def bwd_planar(dy, feat, h, algo=ALGO_AUTO):
    """(dfeat, dh): dfeat has feat's layout, dfeat[:, :, 0] = dC, [:, :, 1] = dB, [:, :, 2] = dx."""
    _require_gpu(feat)
    if TORCH_OPS:
        return torch.ops.gcg.bwd_planar(dy, feat, h, algo_code(algo))
    lib = load()
    _check_planar(feat, h)
    bs, L, _, g, dg = feat.shape
    hl = h.shape[-1]
    if dy.shape != (bs, L, g, dg) or dy.dtype != feat.dtype or not dy.is_contiguous():
        raise ValueError("dy must be a contiguous (bs, L, g, dg) tensor of feat's dtype")
    dfeat, dh = torch.empty_like(feat), torch.empty_like(h)
    if dy.numel() == 0:
        return dfeat, dh.zero_()
    code, a = gated_code(feat, h), algo_code(algo)
    nbytes = lib.gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, a)
    if nbytes == 0:
        raise GcgError("gcg_bwd_workspace_bytes: arguments rejected")
    with _on_device(feat.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=feat.device)
        rc = lib.gcg_bwd_planar(dy.data_ptr(), feat.data_ptr(), h.data_ptr(), dfeat.data_ptr(), dh.data_ptr(),
                                ws.data_ptr(), nbytes, bs, L, g, dg, hl, code, a,
                                torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_bwd_planar")
    return dfeat, dh


def _check_dwconv(x, w):
    if x.dim() != 4 or not x.is_contiguous():
        raise ValueError("x must be a contiguous (bs, L, g, dg) tensor")
    if w.dim() != 3 or w.shape[0] != x.shape[2] or w.shape[1] != 1 or not w.is_contiguous():
        raise ValueError("w must be a contiguous (g, 1, hl) tensor")
    if w.dtype != x.dtype or w.device != x.device:
        raise ValueError("x and w must share dtype and device")


def dwconv_fwd(x, w, keep_output=False):
    """y = causal depthwise convolution of x (bs, L, g, dg) with w (g, 1, hl), no gates.
    ``keep_output``: y goes to fwd_interleaved next, store it through the cache."""
    _require_gpu(x)
    if TORCH_OPS:
        return torch.ops.gcg.dwconv_fwd(x, w, bool(keep_output))
    lib = load()
    _check_dwconv(x, w)
    bs, L, g, dg = x.shape
    y = torch.empty_like(x)
    if x.numel() == 0:
        return y
    with _on_device(x.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_dwconv_fwd(x.data_ptr(), w.data_ptr(), y.data_ptr(), bs, L, g, dg, w.shape[-1],
                                dtype_code(x.dtype), KEEP_OUTPUT if keep_output else 0, st)
    check(rc, "gcg_dwconv_fwd")
    return y


def dwconv_bwd(dy, x, w):
    """(dx, dw) of dwconv_fwd."""
    _require_gpu(x)
    if TORCH_OPS:
        return torch.ops.gcg.dwconv_bwd(dy, x, w)
    lib = load()
    _check_dwconv(x, w)
    if dy.shape != x.shape or dy.dtype != x.dtype or not dy.is_contiguous():
        raise ValueError("dy must be a contiguous tensor of x's shape and dtype")
    bs, L, g, dg = x.shape
    hl = w.shape[-1]
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    if x.numel() == 0:
        return dx, dw.zero_()
    code = dtype_code(x.dtype)
    nbytes = lib.gcg_dwconv_bwd_workspace_bytes(bs, L, g, dg, hl, code)
    if nbytes == 0:
        check(-2, "gcg_dwconv_bwd_workspace_bytes")     # GCG_ERR_UNSUPPORTED
    with _on_device(x.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_dwconv_bwd(dy.data_ptr(), x.data_ptr(), w.data_ptr(), dx.data_ptr(), dw.data_ptr(),
                                ws.data_ptr(), nbytes, bs, L, g, dg, hl, code, st)
    check(rc, "gcg_dwconv_bwd")
    return dx, dw


def _check_mixer_se(raw, wf, h, planar=False):
    if raw.dim() != 5 or raw.shape[2 if planar else 4] != 3 or not raw.is_contiguous():
        raise ValueError("raw must be a contiguous (bs, L, 3, g, dg) tensor" if planar
                         else "raw must be a contiguous (bs, L, g, dg, 3) tensor")
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    if wf.dim() != 3 or wf.shape[0] != 3 * g * dg or wf.shape[1] != 1 or not wf.is_contiguous():
        raise ValueError("wf must be a contiguous (3 * g * dg, 1, kf) tensor")
    if h.dim() != 3 or h.shape[0] != g or h.shape[1] != 1 or not h.is_contiguous():
        raise ValueError("h must be a contiguous (g, 1, hl) tensor")
    if wf.dtype != raw.dtype or wf.device != raw.device or h.device != raw.device:
        raise ValueError("raw and wf must share dtype, and raw, wf and h their device")
    gated_code(raw, h)          # h of raw's dtype, or fp32 with 16-bit raw (fp32 arithmetic)


def mixer_se_fwd(raw, wf, h, planar=False):
    """y (bs, L, g, dg) = fwd_interleaved(dwconv_fwd(raw, wf), h) in one pass over raw (bs, L, g, dg, 3);
    ``planar``: raw is (bs, L, 3, g, dg), the split without interleaving (block.py:881-884)."""
    _require_gpu(raw)
    if TORCH_OPS:
        return torch.ops.gcg.mixer_se_fwd(raw, wf, h, bool(planar))
    lib = load()
    _check_mixer_se(raw, wf, h, planar)
    bs, L = raw.shape[:2]
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    y = torch.empty(bs, L, g, dg, dtype=raw.dtype, device=raw.device)
    if y.numel() == 0:
        return y
    fn = lib.gcg_mixer_se_fwd_planar if planar else lib.gcg_mixer_se_fwd
    with _on_device(raw.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = fn(raw.data_ptr(), wf.data_ptr(), h.data_ptr(), y.data_ptr(), bs, L, g, dg,
                h.shape[-1], wf.shape[-1], gated_code(raw, h), st)
    check(rc, "gcg_mixer_se_fwd_planar" if planar else "gcg_mixer_se_fwd")
    return y


def mixer_se_bwd(dy, raw, wf, h, planar=False):
    """(draw, dwf, dh) of mixer_se_fwd."""
    _require_gpu(raw)
    if TORCH_OPS:
        return torch.ops.gcg.mixer_se_bwd(dy, raw, wf, h, bool(planar))
    lib = load()
    _check_mixer_se(raw, wf, h, planar)
    bs, L = raw.shape[:2]
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    if dy.shape != (bs, L, g, dg) or dy.dtype != raw.dtype or not dy.is_contiguous() or dy.device != raw.device:
        raise ValueError("dy must be a contiguous (bs, L, g, dg) tensor of raw's dtype and device")
    hl, kf = h.shape[-1], wf.shape[-1]
    draw, dwf, dh = torch.empty_like(raw), torch.empty_like(wf), torch.empty_like(h)
    if raw.numel() == 0:
        return draw, dwf.zero_(), dh.zero_()
    code = gated_code(raw, h)
    nbytes = lib.gcg_mixer_se_bwd_workspace_bytes(bs, L, g, dg, hl, kf, code)
    if nbytes == 0:
        check(-2, "gcg_mixer_se_bwd_workspace_bytes")     # GCG_ERR_UNSUPPORTED
    with _on_device(raw.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=raw.device)
        st = torch.cuda.current_stream().cuda_stream
        fn = lib.gcg_mixer_se_bwd_planar if planar else lib.gcg_mixer_se_bwd
        rc = fn(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), h.data_ptr(), draw.data_ptr(),
                dwf.data_ptr(), dh.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl, kf, code, st)
    check(rc, "gcg_mixer_se_bwd_planar" if planar else "gcg_mixer_se_bwd")
    return draw, dwf, dh


def _check_filter_params(w, decay):
    for t in (w, decay):
        if t.dim() != 2 or t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError("w and decay must be contiguous fp32 (g, L_cache) tensors")
    if w.shape != decay.shape or w.device != decay.device:
        raise ValueError("w and decay must share shape and device")


def filter_decay_fwd(w, decay, hl: int, dtype: torch.dtype):
    """h (g, 1, hl) in ``dtype`` = w[:, :hl] * decay[:, :hl]."""
    _require_gpu(w)
    if TORCH_OPS:
        return torch.ops.gcg.filter_decay_fwd(w, decay, hl, dtype)
    lib = load()
    _check_filter_params(w, decay)
    g, l_cache = w.shape
    if not 0 < hl <= l_cache:
        raise ValueError("hl must be in 1..L_cache")
    h = torch.empty(g, 1, hl, dtype=dtype, device=w.device)
    with _on_device(w.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_filter_decay_fwd(w.data_ptr(), decay.data_ptr(), h.data_ptr(), g, l_cache, hl, dtype_code(dtype), st)
    check(rc, "gcg_filter_decay_fwd")
    return h


def filter_decay_bwd(dh, decay):
    """dw (g, L_cache) fp32 from dh (g, 1, hl)."""
    _require_gpu(dh)
    if TORCH_OPS:
        return torch.ops.gcg.filter_decay_bwd(dh, decay)
    lib = load()
    _check_filter_params(decay, decay)
    g, l_cache = decay.shape
    if dh.dim() != 3 or dh.shape[0] != g or dh.shape[1] != 1 or dh.shape[2] > l_cache or not dh.is_contiguous():
        raise ValueError("dh must be a contiguous (g, 1, hl) tensor with hl <= L_cache")
    dw = torch.empty(g, l_cache, dtype=torch.float32, device=dh.device)
    with _on_device(dh.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.gcg_filter_decay_bwd(dh.data_ptr(), decay.data_ptr(), dw.data_ptr(), g, l_cache, dh.shape[2],
                                      dtype_code(dh.dtype), st)
    check(rc, "gcg_filter_decay_bwd")
    return dw



def _check_mixer_mr(raw, wf, h, planar=False):
    if raw.dim() != 5 or raw.shape[2 if planar else 4] != 3 or not raw.is_contiguous():
        raise ValueError("raw must be a contiguous (bs, L, 3, g, dg) tensor" if planar
                         else "raw must be a contiguous (bs, L, g, dg, 3) tensor")
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    if wf.dim() != 3 or wf.shape[0] != 3 * g * dg or wf.shape[1] != 1 or not wf.is_contiguous() or wf.dtype != raw.dtype:
        raise ValueError("wf must be a contiguous (3 * g * dg, 1, kf) tensor of raw's dtype")
    if h.dim() != 3 or h.shape[0] != g or h.shape[1] != 1 or not h.is_contiguous():
        raise ValueError("h must be a contiguous (g, 1, hl) tensor")
    if wf.device != raw.device or h.device != raw.device:
        raise ValueError("raw, wf and h must be on one device")


def _aligned16(t) -> bool:
    """16-byte alignment of a tensor's first element.  While torch.compile traces there is no address to look at
    and the answer is yes: the choice of kernels is then part of the graph, and the entry points themselves
    refuse a misaligned tensor with an error."""
    if torch.compiler.is_compiling():
        return True
    return t.data_ptr() % 16 == 0


def _all_aligned16(tensors, skip_strided=False) -> bool:
    for t in tensors:                      # (a plain loop: torch.compile traces it)
        if skip_strided and not t.is_contiguous():
            continue
        if not _aligned16(t):
            return False
    return True


ROUTE_DECAY, ROUTE_TIME_MAJOR, ROUTE_MIXER_SE, ROUTE_MIXER_MR, ROUTE_MIXER_MR_PLANAR = 1, 2, 3, 4, 5


@torch.compiler.assume_constant_result      # sizes in, a bool out: torch.compile evaluates it while tracing
def route_supported(route: int, bs: int, L: int, g: int, dg: int, hl: int, kf: int, code: int) -> bool:
    """gcg_route_supported: whether the entry points of a route take these sizes (every limit the library checks
    apart from the tensors' alignment: filter lengths, group widths, what a tensor window can span)."""
    if min(bs, L, g, dg, hl) <= 0:
        return False
    return load().gcg_route_supported(route, bs, L, g, dg, hl, kf, code) == 1


def mixer_mr_supported(dg: int, hl: int, kf: int, *tensors, planar: bool = False, sizes=None) -> bool:
    """Whether gcg_mixer_mr_fwd / _bwd take these sizes (matrix-core kernels, filters of up to 128 taps
    -- those of at most 8 are the fused Hyena-SE kernels' -- and a featurizer of at most 3).  ``planar``: the
    planar entry points, which exist in the one-kernel form only (16-bit arithmetic).
    ``sizes`` = (bs, L, g, dtype code): with them the library is asked as well (gcg_route_supported), which also
    knows how far its tensor windows reach; without them only the shape rules above are applied."""
    if not (9 <= hl <= 128 and dg % 16 == 0 and 1 <= kf <= 3 and _all_aligned16(tensors)):
        return False
    if sizes is None:
        return True
    bs, L, g, code = sizes
    return route_supported(ROUTE_MIXER_MR_PLANAR if planar else ROUTE_MIXER_MR, bs, L, g, dg, hl, kf, code)


def mixer_mr_fwd(raw, wf, h, planar=False):
    """Featurizer conv and Hyena-MR operator in one pass: y (bs, L, g, dg) from the projection output
    raw (bs, L, g, dg, 3), without the featurized tensor; the same values as dwconv_fwd followed by fwd_interleaved.
    ``planar``: raw is (bs, L, 3, g, dg), the split without interleaving (block.py:881-884); 16-bit arithmetic only."""
    _require_gpu(raw)
    if TORCH_OPS:
        return torch.ops.gcg.mixer_mr_fwd(raw, wf, h, bool(planar))
    lib = load()
    _check_mixer_mr(raw, wf, h, planar)
    bs, L = raw.shape[:2]
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    y = torch.empty(bs, L, g, dg, dtype=raw.dtype, device=raw.device)
    if y.numel() == 0:
        return y
    fn = lib.gcg_mixer_mr_fwd_planar if planar else lib.gcg_mixer_mr_fwd
    with _on_device(raw.device):
        rc = fn(raw.data_ptr(), wf.data_ptr(), h.data_ptr(), y.data_ptr(), bs, L, g, dg,
                h.shape[-1], wf.shape[-1], gated_code(raw, h), torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_mixer_mr_fwd_planar" if planar else "gcg_mixer_mr_fwd")
    return y


def mixer_mr_bwd(dy, raw, wf, h, planar=False):
    """(draw, dwf, dh) of mixer_mr_fwd from the projection output alone: the features are recomputed; their
    gradient stays inside the kernel (16-bit arithmetic) or lives in a scratch tensor for the duration of the call."""
    _require_gpu(raw)
    if TORCH_OPS:
        return torch.ops.gcg.mixer_mr_bwd(dy, raw, wf, h, bool(planar))
    lib = load()
    _check_mixer_mr(raw, wf, h, planar)
    bs, L = raw.shape[:2]
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    hl, kf = h.shape[-1], wf.shape[-1]
    draw, dwf, dh = torch.empty_like(raw), torch.empty_like(wf), torch.empty_like(h)
    if dy.numel() == 0:
        return draw, dwf.zero_(), dh.zero_()
    code = gated_code(raw, h)
    nbytes = lib.gcg_mixer_mr_bwd_workspace_bytes(bs, L, g, dg, hl, kf, code)
    if nbytes == 0:
        check(-2, "gcg_mixer_mr_bwd_workspace_bytes")
    if planar:
        with _on_device(raw.device):
            ws = torch.empty(nbytes, dtype=torch.uint8, device=raw.device)
            rc = lib.gcg_mixer_mr_bwd_planar(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), h.data_ptr(), draw.data_ptr(),
                                             dwf.data_ptr(), dh.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl, kf,
                                             code, torch.cuda.current_stream().cuda_stream)
        check(rc, "gcg_mixer_mr_bwd_planar")
        return draw, dwf, dh
    with _on_device(raw.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=raw.device)
        sbytes = lib.gcg_mixer_mr_bwd_scratch_bytes(bs, L, g, dg, hl, kf, code)
        scratch = torch.empty(sbytes, dtype=torch.uint8, device=raw.device)
        rc = lib.gcg_mixer_mr_bwd(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), h.data_ptr(), draw.data_ptr(),
                                  dwf.data_ptr(), dh.data_ptr(), scratch.data_ptr() if sbytes else None, ws.data_ptr(),
                                  nbytes, bs, L, g, dg,
                                  hl, kf, code, torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_mixer_mr_bwd")
    return draw, dwf, dh


def mixer_mr_fwd_decay(raw, wf, w, decay, hl: int, filt: torch.dtype, planar=False):
    """mixer_mr_fwd with the filter F(w * decay)[:, :hl] formed inside the kernel (w, decay: (g, l_cache) fp32)."""
    _require_gpu(raw)
    if TORCH_OPS:
        return torch.ops.gcg.mixer_mr_fwd_decay(raw, wf, w, decay, hl, filt, bool(planar))
    lib = load()
    _check_filter_params(w, decay)
    bs, L = raw.shape[:2]
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    y = torch.empty(bs, L, g, dg, dtype=raw.dtype, device=raw.device)
    if y.numel() == 0:
        return y
    fn = lib.gcg_mixer_mr_fwd_planar_decay if planar else lib.gcg_mixer_mr_fwd_decay
    with _on_device(raw.device):
        rc = fn(raw.data_ptr(), wf.data_ptr(), w.data_ptr(), decay.data_ptr(), w.shape[1], y.data_ptr(), bs, L, g, dg,
                hl, wf.shape[-1], _decay_code(raw, filt), torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_mixer_mr_fwd_planar_decay" if planar else "gcg_mixer_mr_fwd_decay")
    return y


def mixer_mr_bwd_decay(dy, raw, wf, w, decay, hl: int, filt: torch.dtype, planar=False):
    """(draw, dwf, dw) of mixer_mr_fwd_decay; dw is the gradient of the filter parameter w."""
    _require_gpu(raw)
    if TORCH_OPS:
        return torch.ops.gcg.mixer_mr_bwd_decay(dy, raw, wf, w, decay, hl, filt, bool(planar))
    lib = load()
    _check_filter_params(w, decay)
    bs, L = raw.shape[:2]
    g, dg = (raw.shape[3], raw.shape[4]) if planar else (raw.shape[2], raw.shape[3])
    kf = wf.shape[-1]
    draw, dwf, dw = torch.empty_like(raw), torch.empty_like(wf), torch.empty_like(w)
    if dy.numel() == 0:
        return draw, dwf.zero_(), dw.zero_()
    code = _decay_code(raw, filt)
    nbytes = lib.gcg_mixer_mr_bwd_workspace_bytes(bs, L, g, dg, hl, kf, code)
    if nbytes == 0:
        check(-2, "gcg_mixer_mr_bwd_workspace_bytes")
    with _on_device(raw.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=raw.device)
        st = torch.cuda.current_stream().cuda_stream
        if planar:
            rc = lib.gcg_mixer_mr_bwd_planar_decay(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), w.data_ptr(),
                                                   decay.data_ptr(), w.shape[1], draw.data_ptr(), dwf.data_ptr(),
                                                   dw.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl, kf, code, st)
        else:
            sbytes = lib.gcg_mixer_mr_bwd_scratch_bytes(bs, L, g, dg, hl, kf, code)
            scratch = torch.empty(sbytes, dtype=torch.uint8, device=raw.device)
            rc = lib.gcg_mixer_mr_bwd_decay(dy.data_ptr(), raw.data_ptr(), wf.data_ptr(), w.data_ptr(), decay.data_ptr(),
                                            w.shape[1], draw.data_ptr(), dwf.data_ptr(), dw.data_ptr(),
                                            scratch.data_ptr() if sbytes else None, ws.data_ptr(), nbytes, bs, L, g, dg, hl,
                                            kf, code, st)
    check(rc, "gcg_mixer_mr_bwd_planar_decay" if planar else "gcg_mixer_mr_bwd_decay")
    return draw, dwf, dw


# ---- the short-filter operator on time-major operands (seqlen, bs, g, dg) ------------------------

def time_major_supported(dg: int, hl: int, *tensors) -> bool:
    """Whether gcg_fwd_time_major / gcg_bwd_time_major take these tensors (register-window kernels): the shape
    rules, and the library's own answer for the sizes of the first tensor, (seqlen, bs, g, dg) -- its windows span
    bs rows of memory per time row, so a large batch of wide rows is beyond them."""
    if not (hl <= 8 and dg % 4 == 0 and all(t.is_contiguous() for t in tensors) and _all_aligned16(tensors)):
        return False
    if not tensors:
        return True
    L, bs, g, _ = tensors[0].shape
    return route_supported(ROUTE_TIME_MAJOR, bs, L, g, dg, hl, 0, dtype_code(tensors[0].dtype))


def fwd_time_major(x, B, C, h):
    """y (bs, seqlen, g, dg) for x, B, C of shape (seqlen, bs, g, dg), read where they lie."""
    _require_gpu(x)
    if TORCH_OPS:
        return torch.ops.gcg.fwd_time_major(x, B, C, h)
    lib = load()
    L, bs, g, dg = x.shape
    y = torch.empty(bs, L, g, dg, dtype=x.dtype, device=x.device)
    if x.numel() == 0:
        return y
    with _on_device(x.device):
        rc = lib.gcg_fwd_time_major(x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), y.data_ptr(), bs, L, g, dg,
                                    h.shape[-1], gated_code(x, h), torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_fwd_time_major")
    return y


def bwd_time_major(dy, x, B, C, h):
    """(dx, dB, dC, dh) with dx, dB, dC in the operands' (seqlen, bs, g, dg) layout; dy is (bs, seqlen, g, dg)."""
    _require_gpu(x)
    if TORCH_OPS:
        return torch.ops.gcg.bwd_time_major(dy, x, B, C, h)
    lib = load()
    L, bs, g, dg = x.shape
    hl = h.shape[-1]
    dx, dB, dC, dh = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x), torch.empty_like(h)
    if x.numel() == 0:
        return dx, dB, dC, dh.zero_()
    code = gated_code(x, h)
    nbytes = lib.gcg_bwd_time_major_workspace_bytes(bs, L, g, dg, hl, code)
    if nbytes == 0:
        raise GcgError("gcg_bwd_time_major_workspace_bytes: arguments rejected")
    with _on_device(x.device):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        rc = lib.gcg_bwd_time_major(dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(), dx.data_ptr(),
                                    dB.data_ptr(), dC.data_ptr(), dh.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg,
                                    hl, code, torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_bwd_time_major")
    return dx, dB, dC, dh


# ---- the gated convolution with the decayed explicit filter built inside the kernels -------------

def decay_supported(g: int, dg: int, hl: int, *tensors) -> bool:
    """Whether the *_decay entry points take these sizes: matrix-core kernels only
    (hl <= 128, dg a multiple of 16, 16-byte aligned tensors; a tensor that is not contiguous is
    copied or read through its interleaved source before it reaches them), rows no wider than a tensor window
    of those kernels holds (the library's answer for the first tensor's (bs, L, g, dg))."""
    if not (hl <= 128 and dg % 16 == 0 and _all_aligned16(tensors, skip_strided=True)):
        return False
    if not tensors or tensors[0].dim() != 4:
        return True
    bs, L = tensors[0].shape[:2]
    return route_supported(ROUTE_DECAY, bs, L, g, dg, hl, 0, dtype_code(tensors[0].dtype))


def _decay_code(t: torch.Tensor, filt: torch.dtype) -> int:
    if filt == t.dtype:
        return dtype_code(t.dtype)
    if filt == torch.float32 and t.dtype in (torch.bfloat16, torch.float16):
        return GCG_BF16_F32 if t.dtype == torch.bfloat16 else GCG_F16_F32
    raise TypeError(f"filter type {filt} with {t.dtype} tensors")


def fwd_decay(x, B, C, w, decay, hl: int, filt: torch.dtype):
    """gcg_fwd with h = filt(w[:, :hl] * decay[:, :hl]) formed inside the kernel; w, decay: (g, L_cache) fp32."""
    _require_gpu(x)
    if TORCH_OPS:
        return torch.ops.gcg.fwd_decay(x, B, C, w, decay, hl, filt)
    lib = load()
    _check_filter_params(w, decay)
    bs, L, g, dg = x.shape
    y = torch.empty_like(x)
    if x.numel() == 0:
        return y
    with _on_device(x.device):
        rc = lib.gcg_fwd_decay(x.data_ptr(), B.data_ptr(), C.data_ptr(), w.data_ptr(), decay.data_ptr(), w.shape[1],
                               y.data_ptr(), bs, L, g, dg, hl, _decay_code(x, filt),
                               torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_fwd_decay")
    return y


def bwd_decay(dy, x, B, C, w, decay, hl: int, filt: torch.dtype):
    """(dx, dB, dC, dw): gcg_bwd whose filter-gradient reduction writes the (g, L_cache) fp32 gradient of w."""
    _require_gpu(x)
    if TORCH_OPS:
        return torch.ops.gcg.bwd_decay(dy, x, B, C, w, decay, hl, filt)
    lib = load()
    _check_filter_params(w, decay)
    bs, L, g, dg = x.shape
    dx, dB, dC, dw = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x), torch.empty_like(w)
    if x.numel() == 0:
        return dx, dB, dC, dw.zero_()
    code = _decay_code(x, filt)
    # zero bytes: the shape is outside these kernels or the arguments are wrong; the call below says which
    nbytes = lib.gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, ALGO_NAMES["mfma"])
    with _on_device(x.device):
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=x.device)
        rc = lib.gcg_bwd_decay(dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), w.data_ptr(), decay.data_ptr(),
                               w.shape[1], dx.data_ptr(), dB.data_ptr(), dC.data_ptr(), dw.data_ptr(), ws.data_ptr(),
                               nbytes, bs, L, g, dg, hl, code, torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_bwd_decay")
    return dx, dB, dC, dw


def fwd_interleaved_decay(feat, w, decay, hl: int, filt: torch.dtype):
    _require_gpu(feat)
    if TORCH_OPS:
        return torch.ops.gcg.fwd_interleaved_decay(feat, w, decay, hl, filt)
    lib = load()
    _check_filter_params(w, decay)
    bs, L, g, dg, _ = feat.shape
    y = torch.empty(bs, L, g, dg, dtype=feat.dtype, device=feat.device)
    if y.numel() == 0:
        return y
    with _on_device(feat.device):
        rc = lib.gcg_fwd_interleaved_decay(feat.data_ptr(), w.data_ptr(), decay.data_ptr(), w.shape[1], y.data_ptr(),
                                           bs, L, g, dg, hl, _decay_code(feat, filt),
                                           torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_fwd_interleaved_decay")
    return y


def bwd_interleaved_decay(dy, feat, w, decay, hl: int, filt: torch.dtype, keep_output=False):
    _require_gpu(feat)
    if TORCH_OPS:
        return torch.ops.gcg.bwd_interleaved_decay(dy, feat, w, decay, hl, filt, keep_output)
    lib = load()
    _check_filter_params(w, decay)
    bs, L, g, dg, _ = feat.shape
    dfeat, dw = torch.empty_like(feat), torch.empty_like(w)
    if dy.numel() == 0:
        return dfeat, dw.zero_()
    code = _decay_code(feat, filt)
    # zero bytes: the shape is outside these kernels or the arguments are wrong; the call below says which
    nbytes = lib.gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, ALGO_NAMES["mfma"])
    with _on_device(feat.device):
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=feat.device)
        rc = lib.gcg_bwd_interleaved_decay(dy.data_ptr(), feat.data_ptr(), w.data_ptr(), decay.data_ptr(), w.shape[1],
                                           dfeat.data_ptr(), dw.data_ptr(), ws.data_ptr(), nbytes, bs, L, g, dg, hl,
                                           code, KEEP_OUTPUT if keep_output else 0,
                                           torch.cuda.current_stream().cuda_stream)
    check(rc, "gcg_bwd_interleaved_decay")
    return dfeat, dw


def select_algo(bs, L, g, dg, hl, dtype: torch.dtype, backward=False) -> str:
    rc = load().gcg_select_algo(bs, L, g, dg, hl, dtype_code(dtype), int(backward))
    if rc < 0:
        check(rc, "gcg_select_algo")
    return {v: k for k, v in ALGO_NAMES.items()}[rc]
