"""``run_short_hyena``: the entry point of the reference's other short-filter kernel family
(savanna/kernels/triton_src/short_hyena/interface.py:96-119), kept call-compatible.

That family computes the same operator, ``out = q * conv(k * v, w)`` with a causal
cross-correlation (short_hyena/utils.py:14-28, ref_hyena_mlp :36-66), on another layout: inputs
``(seqlen, bs, g, dg)``, output ``(bs, g, seqlen, dg)`` (short_hyena/fwd.py:245-247).  Here it maps
onto the gated convolution kernels (C = q, B = k, x = v); the two layout changes are views on the
way in (made contiguous by the autograd boundary) and a permuted view of the result on the way out.
"""
from __future__ import annotations

import torch

from ..cgcg.interface import two_pass_chunked_gate_conv_gate
from ..cgcg.src.kernel_utils import FwdKernelConfigRefactor

_FWD_CFG = FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row")


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
    to_blgd = lambda t: t.permute(1, 0, 2, 3).reshape(bs, seqlen, groups, width)
    y = two_pass_chunked_gate_conv_gate(to_blgd(v), to_blgd(k), to_blgd(q), w.reshape(groups, 1, hl),
                                        bs, seqlen, groups, width, fwd_kernel_cfg=_FWD_CFG, bwd_autotune=True)
    return y.reshape(bs, seqlen, g, dg).permute(0, 2, 1, 3)
