"""Forward entry point, call-compatible with
savanna/kernels/triton_src/cgcg/src/fwd.py:13-233 (``two_pass_fwd_grouped``)."""
from __future__ import annotations

import torch

from .... import _lib


def two_pass_fwd_grouped(
    x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, h: torch.Tensor,
    y: torch.Tensor = None, return_bx: bool = True, return_y2: bool = True,
    verbose: bool = False, schedule: str = "default", autotune: bool = True,
    # Triton tiling arguments of the reference signature, accepted and ignored
    CHUNK_SIZE: int = None, BLOCK_D: int = None, CHUNK_TILES_PER_PROGRAM: int = 1,
    THREADBLOCK_SWIZZLE: str = "row", num_warps: int = 4, num_stages: int = 3, num_ctas: int = 1,
    maxnreg: int = None, warmup: bool = False,
    algo="auto",
):
    """Gated causal convolution y = C * conv(B * x, h) on the GPU.

    x, B, C: (bs, L, g, dg) contiguous; h: (g, 1, hl).  Returns ``(bx, y2, y)`` like
    the reference (fwd.py:228-233), with ``bx``/``y2`` None when not requested.

    The Triton tiling arguments (CHUNK_SIZE ... maxnreg) are accepted so existing
    call sites keep working; they do not affect the result.  ``algo`` forces a kernel
    family ("direct", "window", "mfma") and is what the parity tests use.
    """
    bs, seqlen, g, dg = x.shape
    # the reference's argument checks (fwd.py:79-99, 125-131) that are about the data
    assert x.shape == B.shape == C.shape, "x, B, C must share one shape"
    assert h.dim() == 3 and h.shape[0] == g and h.shape[1] == 1, "h must be (g, 1, hl)"
    assert x.is_contiguous() and B.is_contiguous() and C.is_contiguous() and h.is_contiguous()
    assert x.dtype == B.dtype == C.dtype, "x, B, C must share one dtype"
    _lib.gated_code(x, h)       # h: the same dtype, or float32 with 16-bit tensors (fp32 arithmetic, no casts)
    if schedule == "persistent":
        raise NotImplementedError("Skip persistent for now")
    if schedule != "default":
        raise ValueError(f"schedule {schedule} not implemented")
    if warmup:
        raise NotImplementedError("ahead-of-time warmup is a Triton notion; the HIP library is prebuilt")
    if verbose:
        name = _lib.select_algo(bs, seqlen, g, dg, h.shape[-1], x.dtype) if algo in ("auto", 0) else algo
        print(f"gcg fwd: {bs=} {seqlen=} {g=} {dg=} hl={h.shape[-1]} dtype={x.dtype} kernel={name}")
    if y is not None:
        y = y.reshape(x.shape)      # the reference takes a (bs, L, d) or (bs, L, g, dg) buffer (fwd.py:155-156)
    return _lib.fwd(x, B, C, h, return_bx=return_bx, return_y2=return_y2, algo=algo, out=y)
