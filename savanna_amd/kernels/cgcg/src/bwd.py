"""Backward entry point, call-compatible with
savanna/kernels/triton_src/cgcg/src/bwd.py:347-474 (``two_pass_bwd_refactor``)."""
from __future__ import annotations

import torch

from .... import _lib


def two_pass_bwd_refactor(
    dy: torch.Tensor,
    Bx: torch.Tensor = None,
    y2: torch.Tensor = None,
    x: torch.Tensor = None,
    B: torch.Tensor = None,
    C: torch.Tensor = None,
    h: torch.Tensor = None,
    bs=None,
    seqlen=None,
    g=None,
    dg=None,
    fused=False,
    autotune=True,
    kernel_config=None,
    algo="auto",
):
    """(dx, dB, dC, dh) of y = C * conv(B * x, h).

    ``Bx`` and ``y2`` (the activations the reference saves in the forward and reads here,
    bwd.py:349-350) are accepted for call compatibility and not read: one fused kernel
    recomputes both on chip from x, B and h.  ``fused``, ``autotune`` and
    ``kernel_config`` select between Triton paths in the reference and have no effect.
    """
    assert x.shape == B.shape == C.shape == dy.shape
    if Bx is not None:
        assert Bx.shape == x.shape
    if y2 is not None:
        assert y2.shape == x.shape
    if None not in (bs, seqlen, g, dg):
        assert dy.shape == (bs, seqlen, g, dg)
    assert h.dim() == 3 and h.shape[0] == x.shape[2] and h.shape[1] == 1
    assert all(t.is_contiguous() for t in (dy, x, B, C, h))
    assert dy.dtype == x.dtype == B.dtype == C.dtype
    _lib.gated_code(x, h)       # h: the same dtype, or float32 with 16-bit tensors
    return _lib.bwd(dy, x, B, C, h, algo=algo)
