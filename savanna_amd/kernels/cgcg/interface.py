"""Autograd boundary of the gated chunked causal convolution.

Mirrors savanna/kernels/triton_src/cgcg/interface.py:27-176: same function name,
positional and keyword arguments, preconditions and return value, so that
savanna/model/operators/hyena/hyena.py:517-531 and :825-840 can call it unchanged.
"""
from __future__ import annotations

import warnings

import torch

from ... import _lib
from .src.bwd import two_pass_bwd_refactor
from .src.fwd import two_pass_fwd_grouped
from .src.kernel_utils import BwdKernelConfigRefactor, FwdKernelConfigRefactor  # noqa: F401


def _contig(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


def interleaved_source(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor):
    """The (bs, L, g, dg, 3) tensor whose thirds [..., 0], [..., 1], [..., 2] are C, B, x, or None.

    The interleaved split of the projected features (savanna/model/block.py:886-890,
    ``rearrange(features, "b l (g dg p) -> b l g p dg", p=3).unbind(dim=3)`` -> x1, x2, v, passed on
    as C, B, x) hands the operator three views of one buffer with element stride 3.  The reference
    gathers each into its own tensor (interface.py:51-54); the HIP kernels read the buffer as it is.
    """
    if not (x.shape == B.shape == C.shape and x.dim() == 4 and x.dtype == B.dtype == C.dtype):
        return None
    if not (x.device == B.device == C.device):
        return None
    bs, L, g, dg = x.shape
    want = (L * g * dg * 3, g * dg * 3, dg * 3, 3)
    for t in (x, B, C):
        if any(n > 1 and st != w for n, st, w in zip(t.shape, t.stride(), want)):
            return None
    base = C.untyped_storage().data_ptr()
    if x.untyped_storage().data_ptr() != base or B.untyped_storage().data_ptr() != base:
        return None
    o = C.storage_offset()
    if B.storage_offset() != o + 1 or x.storage_offset() != o + 2:
        return None
    return torch.as_strided(C, (bs, L, g, dg, 3), want + (1,), o)


def planar_source(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor):
    """The (bs, L, 3, g, dg) tensor whose thirds [:, :, 0], [:, :, 1], [:, :, 2] are C, B, x, or None.

    The split without interleaving (savanna/model/block.py:881-884,
    ``rearrange(features, "b l (p g dg) -> b l p g dg", p=3).unbind(dim=2)`` -> x1, x2, v, passed on as C, B, x;
    interleave_projections = false) hands the operator three views whose rows lie 3 * g * dg elements apart.
    """
    if not (x.shape == B.shape == C.shape and x.dim() == 4 and x.dtype == B.dtype == C.dtype):
        return None
    if not (x.device == B.device == C.device):
        return None
    bs, L, g, dg = x.shape
    d = g * dg
    want = (L * 3 * d, 3 * d, dg, 1)
    for t in (x, B, C):
        if any(n > 1 and st != w for n, st, w in zip(t.shape, t.stride(), want)):
            return None
    base = C.untyped_storage().data_ptr()
    if x.untyped_storage().data_ptr() != base or B.untyped_storage().data_ptr() != base:
        return None
    o = C.storage_offset()
    if B.storage_offset() != o + d or x.storage_offset() != o + 2 * d:
        return None
    return torch.as_strided(C, (bs, L, 3, g, dg), (L * 3 * d, 3 * d, d, dg, 1), o)


class TwoPassChunkedGateConvGate(torch.autograd.Function):
    """y = C * conv(B * x, h); saves only the four inputs (the reference also saves
    Bx and y2, interface.py:79 -- here they are recomputed in the backward kernel)."""

    @staticmethod
    def forward(ctx, x, B, C, h, bs, seqlen, g, dg, schedule="default", fwd_autotune=False,
                fwd_kernel_cfg=None, fused_bwd=False, bwd_autotune=False, bwd_kernel_cfg=None):
        schedule = schedule if fwd_autotune else fwd_kernel_cfg.schedule
        assert x.shape == torch.Size([bs, seqlen, g, dg])
        assert x.shape == B.shape == C.shape
        ctx.input_shape = (bs, seqlen, g, dg)
        # (under torch.compile the storage test cannot be traced: compiled callers that hold the features tensor
        # call two_pass_chunked_gate_conv_gate_interleaved)
        tracing = torch.compiler.is_compiling()
        feat = interleaved_source(x, B, C) if x.numel() > 0 and not tracing else None
        ctx.interleaved = feat is not None
        planar = planar_source(x, B, C) if feat is None and x.numel() > 0 and g * dg > 1 and not tracing else None
        ctx.planar = planar is not None
        if feat is not None or planar is not None:
            # three views of one buffer (interleaved elements, or the thirds of its rows): no gathers
            assert h.dim() == 3 and h.shape[0] == g and h.shape[1] == 1, "h must be (g, 1, hl)"
            if schedule != "default":
                raise NotImplementedError("Skip persistent for now") if schedule == "persistent" else \
                    ValueError(f"schedule {schedule} not implemented")
            h = _contig(h)
            y = _lib.fwd_interleaved(feat, h) if feat is not None else _lib.fwd_planar(planar, h)
            ctx.save_for_backward(feat if feat is not None else planar, h)
            return y
        x, B, C, h = _contig(x), _contig(B), _contig(C), _contig(h)
        _, _, y = two_pass_fwd_grouped(x, B, C, h, autotune=fwd_autotune, schedule=schedule,
                                       return_bx=False, return_y2=False)
        ctx.save_for_backward(x, B, C, h)
        return y

    @staticmethod
    def backward(ctx, dy):
        if ctx.interleaved:
            feat, h = ctx.saved_tensors
            dfeat, dh = _lib.bwd_interleaved(_contig(dy), feat, h)
            return (dfeat[..., 2], dfeat[..., 1], dfeat[..., 0], dh) + (None,) * 10
        if ctx.planar:
            feat, h = ctx.saved_tensors
            dfeat, dh = _lib.bwd_planar(_contig(dy), feat, h)
            return (dfeat[:, :, 2], dfeat[:, :, 1], dfeat[:, :, 0], dh) + (None,) * 10
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


class InterleavedGateConvGate(torch.autograd.Function):
    """The same operator on the interleaved features tensor itself, so that the gradient is
    produced in the features' layout and autograd has nothing to re-assemble."""

    @staticmethod
    def forward(ctx, feat, h, keep_dfeatures=False):
        feat, h = _contig(feat), _contig(h)
        y = _lib.fwd_interleaved(feat, h)
        ctx.save_for_backward(feat, h)
        ctx.keep_dfeatures = keep_dfeatures
        return y

    @staticmethod
    def backward(ctx, dy):
        feat, h = ctx.saved_tensors
        dfeat, dh = _lib.bwd_interleaved(_contig(dy), feat, h, keep_output=ctx.keep_dfeatures)
        return dfeat, dh, None


def two_pass_chunked_gate_conv_gate_interleaved(features: torch.Tensor, h: torch.Tensor,
                                                bs: int, seqlen: int, g: int, dg: int,
                                                keep_dfeatures: bool = False) -> torch.Tensor:
    """y = x1 * conv(x2 * v, h) for projected features laid out "(g dg p)" with p = (x1, x2, v)
    fastest, i.e. the tensor savanna/model/block.py:886-890 splits before calling the mixer.

    features: (bs, seqlen, 3*g*dg) or (bs, seqlen, g, dg, 3); h: (g, 1, hl).  Returns (bs, seqlen, g, dg).
    Equivalent to ``two_pass_chunked_gate_conv_gate(x=v, B=x2, C=x1, h=h, ...)`` on the split views.
    ``keep_dfeatures``: the gradient of the features is read at once by the backward of the op that
    produced them (the featurizer conv); it is then stored through the cache.  Same values either way.
    """
    assert features.numel() == bs * seqlen * g * dg * 3, "features must hold 3*g*dg values per position"
    assert h.dim() == 3 and h.shape[0] == g and h.shape[1] == 1, "h must be (g, 1, hl)"
    return InterleavedGateConvGate.apply(features.reshape(bs, seqlen, g, dg, 3), h, keep_dfeatures)


class PlanarGateConvGate(torch.autograd.Function):
    """The same operator on the planar features tensor (bs, L, 3, g, dg) itself: the kernels read the thirds of each
    row in place and the backward writes the gradient in the same layout."""

    @staticmethod
    def forward(ctx, feat, h):
        feat, h = _contig(feat), _contig(h)
        ctx.save_for_backward(feat, h)
        return _lib.fwd_planar(feat, h)

    @staticmethod
    def backward(ctx, dy):
        feat, h = ctx.saved_tensors
        return _lib.bwd_planar(_contig(dy), feat, h)


def two_pass_chunked_gate_conv_gate_planar(features: torch.Tensor, h: torch.Tensor,
                                           bs: int, seqlen: int, g: int, dg: int) -> torch.Tensor:
    """y = x1 * conv(x2 * v, h) for projected features laid out "(p g dg)" with p = (x1, x2, v) slowest, i.e. the
    tensor savanna/model/block.py:881-884 splits when interleave_projections is off.

    features: (bs, seqlen, 3*g*dg) or (bs, seqlen, 3, g, dg); h: (g, 1, hl).  Returns (bs, seqlen, g, dg).
    Equivalent to ``two_pass_chunked_gate_conv_gate(x=v, B=x2, C=x1, h=h, ...)`` on the split views.
    """
    assert features.numel() == bs * seqlen * g * dg * 3, "features must hold 3*g*dg values per position"
    assert h.dim() == 3 and h.shape[0] == g and h.shape[1] == 1, "h must be (g, 1, hl)"
    return PlanarGateConvGate.apply(features.reshape(bs, seqlen, 3, g, dg), h)


class DecayedGateConvGate(torch.autograd.Function):
    """y = C * conv(B * x, h) with the Hyena-MR filter h = filt(w[:, :hl] * decay[:, :hl]) formed inside the
    convolution kernels, and the gradient of w written by the backward kernel's own filter-gradient
    reduction: neither h nor dh exists in memory and the layer launches nothing besides the convolution.
    Counterpart of ExplicitSingleDecayFilter.filter (savanna/model/operators/hyena/parametrization/
    explicit.py:68-75), the slice and cast of savanna/model/operators/hyena/hyena.py:440-441, :499-503 and
    TwoPassChunkedGateConvGate (cgcg/interface.py:27-127) taken together.  Matrix-core shapes only
    (``_lib.decay_supported``).  Three views of one interleaved features tensor are read in place."""

    @staticmethod
    def forward(ctx, x, B, C, w, decay, hl, filt):
        w, decay = _contig(w), _contig(decay)
        feat = interleaved_source(x, B, C) if x.numel() > 0 and not torch.compiler.is_compiling() else None
        ctx.interleaved = feat is not None
        ctx.hl, ctx.filt = hl, filt
        if feat is not None:
            ctx.save_for_backward(feat, w, decay)
            return _lib.fwd_interleaved_decay(feat, w, decay, hl, filt)
        x, B, C = _contig(x), _contig(B), _contig(C)
        ctx.save_for_backward(x, B, C, w, decay)
        return _lib.fwd_decay(x, B, C, w, decay, hl, filt)

    @staticmethod
    def backward(ctx, dy):
        if ctx.interleaved:
            feat, w, decay = ctx.saved_tensors
            dfeat, dw = _lib.bwd_interleaved_decay(_contig(dy), feat, w, decay, ctx.hl, ctx.filt)
            return dfeat[..., 2], dfeat[..., 1], dfeat[..., 0], dw, None, None, None
        x, B, C, w, decay = ctx.saved_tensors
        dx, dB, dC, dw = _lib.bwd_decay(_contig(dy), x, B, C, w, decay, ctx.hl, ctx.filt)
        return dx, dB, dC, dw, None, None, None


class InterleavedDecayedGateConvGate(torch.autograd.Function):
    """The same on the interleaved features tensor itself (gradient in the features' layout)."""

    @staticmethod
    def forward(ctx, feat, w, decay, hl, filt, keep_dfeatures=False):
        feat, w, decay = _contig(feat), _contig(w), _contig(decay)
        ctx.save_for_backward(feat, w, decay)
        ctx.hl, ctx.filt, ctx.keep_dfeatures = hl, filt, keep_dfeatures
        return _lib.fwd_interleaved_decay(feat, w, decay, hl, filt)

    @staticmethod
    def backward(ctx, dy):
        feat, w, decay = ctx.saved_tensors
        dfeat, dw = _lib.bwd_interleaved_decay(_contig(dy), feat, w, decay, ctx.hl, ctx.filt,
                                               keep_output=ctx.keep_dfeatures)
        return dfeat, dw, None, None, None, None
