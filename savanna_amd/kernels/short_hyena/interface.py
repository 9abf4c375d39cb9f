"""``run_short_hyena``: the entry point of the reference's other short-filter kernel family
(savanna/kernels/triton_src/short_hyena/interface.py:96-119), kept call-compatible.

That family computes the same operator, ``out = q * conv(k * v, w)`` with a causal
cross-correlation (short_hyena/utils.py:14-28, ref_hyena_mlp :36-66), on another layout: inputs
``(seqlen, bs, g, dg)``, output ``(bs, g, seqlen, dg)`` (short_hyena/fwd.py:245-247).  Here it maps
onto the gated convolution kernels (C = q, B = k, x = v).  With one filter per group of at most 8 taps
the register-window kernels read q, k, v where they lie -- rows of one batch entry ``bs * g * dg``
elements apart -- and write dq, dk, dv in that layout, so nothing is permuted on the way in
(gcg_fwd_time_major / gcg_bwd_time_major); the result is computed as (bs, seqlen, g, dg) and returned as the
permuted view the reference's shape asks for.  Other shapes take two layout changes around the general kernels.
"""
from __future__ import annotations

import torch

from ... import _lib
from ..cgcg.interface import two_pass_chunked_gate_conv_gate
from ..cgcg.src.kernel_utils import FwdKernelConfigRefactor

_FWD_CFG = FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row")


class _TimeMajorShortHyena(torch.autograd.Function):
    """q * conv(k * v, w) on (seqlen, bs, g, dg) operands in place -> (bs, seqlen, g, dg); saves the inputs only
    (ShortHyenaOperator also saves three permuted intermediates, interface.py:47)."""

    @staticmethod
    def forward(ctx, q, k, v, w):
        ctx.save_for_backward(q, k, v, w)
        return _lib.fwd_time_major(v, k, q, w)

    @staticmethod
    def backward(ctx, dy):
        q, k, v, w = ctx.saved_tensors
        dv, dk, dq, dw = _lib.bwd_time_major(dy if dy.is_contiguous() else dy.contiguous(), v, k, q, w)
        return dq, dk, dv, dw


def run_short_hyena(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, w: torch.Tensor,
                    repeat_interleave: bool = True, use_causal_conv: bool = False, autotune: bool = False,
                    fwd_kernel_cfg=None, bwd_kernel_cfg=None) -> torch.Tensor:
    """q, k, v: (seqlen, bs, g, dg); w: (g, 1, hl) with ``repeat_interleave`` (one filter per group,
    short_hyena/fwd.py:292-294) or (g*dg, 1, hl) without.  Returns (bs, g, seqlen, dg).

    ``use_causal_conv`` selects a library in the reference (filters of at most 4 taps,
    interface.py:31-33) and has no effect on the result; the kernel-config arguments are Triton
    tiles, required unless ``autotune`` as in the reference (interface.py:109-111) and otherwise unused.
    """
    assert autotune or (fwd_kernel_cfg is not None and bwd_kernel_cfg is not None), \
        "Must specify fwd_kernel_cfg and bwd_kernel_cfg if not autotuning"
    seqlen, bs, g, dg = q.shape
    assert k.shape == q.shape == v.shape
    hl = w.shape[-1]
    if use_causal_conv:
        assert hl <= 4, "causal conv only works with filter_len <= 4"
    if repeat_interleave:
        assert w.shape[0] == g
        groups, width = g, dg
    else:
        assert w.shape[0] == g * dg
        groups, width = g * dg, 1
    if repeat_interleave and q.is_cuda and _lib.time_major_supported(dg, hl, q, k, v):
        w3 = w.reshape(g, 1, hl)
        y = _TimeMajorShortHyena.apply(q, k, v, w3 if w3.is_contiguous() else w3.contiguous())
        return y.permute(0, 2, 1, 3)
    to_blgd = lambda t: t.permute(1, 0, 2, 3).reshape(bs, seqlen, groups, width)
    y = two_pass_chunked_gate_conv_gate(to_blgd(v), to_blgd(k), to_blgd(q), w.reshape(groups, 1, hl),
                                        bs, seqlen, groups, width, fwd_kernel_cfg=_FWD_CFG, bwd_autotune=True)
    return y.reshape(bs, seqlen, g, dg).permute(0, 2, 1, 3)
