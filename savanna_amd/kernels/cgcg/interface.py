"""Autograd boundary of the gated chunked causal convolution.

Mirrors savanna/kernels/triton_src/cgcg/interface.py:27-176: same function name,
positional and keyword arguments, preconditions and return value, so that
savanna/model/operators/hyena/hyena.py:517-531 and :825-840 can call it unchanged.
"""
from __future__ import annotations

import warnings

import torch

from .src.bwd import two_pass_bwd_refactor
from .src.fwd import two_pass_fwd_grouped
from .src.kernel_utils import BwdKernelConfigRefactor, FwdKernelConfigRefactor  # noqa: F401


def _contig(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


class TwoPassChunkedGateConvGate(torch.autograd.Function):
    """y = C * conv(B * x, h); saves only the four inputs (the reference also saves
    Bx and y2, interface.py:79 -- here they are recomputed in the backward kernel)."""

    @staticmethod
    def forward(ctx, x, B, C, h, bs, seqlen, g, dg, schedule="default", fwd_autotune=False,
                fwd_kernel_cfg=None, fused_bwd=False, bwd_autotune=False, bwd_kernel_cfg=None):
        schedule = schedule if fwd_autotune else fwd_kernel_cfg.schedule
        assert x.shape == torch.Size([bs, seqlen, g, dg])
        assert x.shape == B.shape == C.shape
        x, B, C, h = _contig(x), _contig(B), _contig(C), _contig(h)
        _, _, y = two_pass_fwd_grouped(x, B, C, h, autotune=fwd_autotune, schedule=schedule,
                                       return_bx=False, return_y2=False)
        ctx.save_for_backward(x, B, C, h)
        ctx.input_shape = (bs, seqlen, g, dg)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, B, C, h = ctx.saved_tensors
        bs, seqlen, g, dg = ctx.input_shape
        dx, dB, dC, dh = two_pass_bwd_refactor(dy=_contig(dy), x=x, B=B, C=C, h=h,
                                               bs=bs, seqlen=seqlen, g=g, dg=dg)
        return (dx, dB, dC, dh) + (None,) * 10


def two_pass_chunked_gate_conv_gate(
    x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, h: torch.Tensor,
    bs: int, seqlen: int, g: int, dg: int,
    schedule: str = "default",
    fwd_autotune: bool = False, bwd_autotune: bool = True, fused_bwd: bool = True,
    fwd_kernel_cfg: FwdKernelConfigRefactor = None, bwd_kernel_cfg: BwdKernelConfigRefactor = None,
):
    """Gate -> causal FIR convolution -> gate, differentiable in x, B, C and h.

    x, B (pre-gate pair) and C (post-gate): (bs, seqlen, g, dg); h: (g, 1, hl).
    Preconditions follow interface.py:148-159 of the reference.
    """
    assert fwd_autotune or (fwd_kernel_cfg is not None), "Must specify fwd_kernel_cfg if not autotuning fwd"
    if fused_bwd:
        assert bwd_autotune or (bwd_kernel_cfg is not None), "Must specify bwd_kernel_cfg if not autotuning bwd"
        if bwd_autotune and (bwd_kernel_cfg is not None):
            warnings.warn("WARNING: Both autotune and bwd_kernel_cfg specified, using bwd_kernel_cfg")
            bwd_autotune = False
    if fwd_autotune and (fwd_kernel_cfg is not None):
        warnings.warn("WARNING: Both autotune and fwd_kernel_cfg specified, using fwd_kernel_cfg")
        fwd_autotune = False
    return TwoPassChunkedGateConvGate.apply(
        x, B, C, h, bs, seqlen, g, dg, schedule, fwd_autotune, fwd_kernel_cfg,
        fused_bwd, bwd_autotune, bwd_kernel_cfg,
    )
