"""The ``torch.ops.gcg`` operators: loads the PyTorch extension built from csrc/gcg_torch.cpp.

The extension registers every kernel entry point of the C ABI as a torch operator with a device
implementation (allocates the outputs, enqueues on torch's current stream) and a meta
implementation (shapes only), so the Python layers above can be traced by ``torch.compile`` and the
per-call cost is one dispatcher hop instead of a ctypes call with Python-side allocation.  It is
the binding the reference's Triton launch wrappers correspond to
(savanna/kernels/triton_src/cgcg/src/fwd.py:13-233, src/bwd.py:347-474).

``AVAILABLE`` is False when gcg_torch.so has not been built or ``GCG_BINDING=ctypes`` is set; the
ctypes binding in ``_lib`` then carries the calls (same library, same kernels).
"""
from __future__ import annotations

import os

import torch

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
EXT_PATH = os.path.join(_CSRC, "gcg_torch.so")

AVAILABLE = False
LOAD_ERROR = None

if os.environ.get("GCG_BINDING", "torch") != "ctypes" and not os.environ.get("GCG_HIP_LIB"):
    if os.path.exists(EXT_PATH):
        try:
            torch.ops.load_library(EXT_PATH)
            AVAILABLE = True
        except OSError as e:          # e.g. built against another torch: say so, the ctypes binding still works
            LOAD_ERROR = str(e)
    else:
        LOAD_ERROR = f"{EXT_PATH} is not built"

OP_NAMES = (
    "fwd", "fwd_full", "fwd_out", "bwd", "fwd_interleaved", "bwd_interleaved", "dwconv_fwd", "dwconv_bwd",
    "mixer_se_fwd", "mixer_se_bwd", "filter_decay_fwd", "filter_decay_bwd",
    "mixer_mr_fwd", "mixer_mr_bwd", "mixer_mr_fwd_decay", "mixer_mr_bwd_decay", "fwd_time_major", "bwd_time_major", "fwd_decay", "bwd_decay", "fwd_interleaved_decay", "bwd_interleaved_decay",
    "fwd_planar", "bwd_planar",
)


# ---- autograd --------------------------------------------------------------------------------------------
# Every forward operator has its backward formula registered, so that a call of torch.ops.gcg.* on tensors that
# require grad is part of the autograd graph like any other operator (the autograd.Function wrappers in
# savanna_amd/kernels and savanna_amd/operators call the same operators inside their own forward / backward,
# where autograd is off, and are not affected).  The backward operators are differentiated no further: as in the
# reference, whose backward runs under torch.no_grad (savanna/kernels/triton_src/cgcg/src/bwd.py:5, :414-417).
# fwd_full (optional Bx and y2 outputs) and fwd_out (writes into its argument) refuse tensors that require grad.

def _register_autograd():
    ops = torch.ops.gcg
    reg = torch.library.register_autograd

    def save(*names):
        """setup_context that keeps the named tensor inputs and every non-tensor input."""
        def setup(ctx, inputs, output):
            ctx.save_for_backward(*[inputs[i] for i in names])
            ctx.rest = inputs
        return setup

    def gated(ctx, dy):              # fwd(x, B, C, h, algo)
        x, B, C, h = ctx.saved_tensors
        dx, dB, dC, dh = ops.bwd(dy.contiguous(), x, B, C, h, ctx.rest[4])
        return dx, dB, dC, dh, None
    reg("gcg::fwd", gated, setup_context=save(0, 1, 2, 3))

    def interleaved(ctx, dy):        # fwd_interleaved(feat, h, algo)
        feat, h = ctx.saved_tensors
        dfeat, dh = ops.bwd_interleaved(dy.contiguous(), feat, h, ctx.rest[2], False)
        return dfeat, dh, None
    reg("gcg::fwd_interleaved", interleaved, setup_context=save(0, 1))

    def planar(ctx, dy):             # fwd_planar(feat, h, algo)
        feat, h = ctx.saved_tensors
        dfeat, dh = ops.bwd_planar(dy.contiguous(), feat, h, ctx.rest[2])
        return dfeat, dh, None
    reg("gcg::fwd_planar", planar, setup_context=save(0, 1))

    def dwconv(ctx, dy):             # dwconv_fwd(x, w, keep_output)
        x, w = ctx.saved_tensors
        dx, dw = ops.dwconv_bwd(dy.contiguous(), x, w)
        return dx, dw, None
    reg("gcg::dwconv_fwd", dwconv, setup_context=save(0, 1))

    def mixer(bwd_op):
        def backward(ctx, dy):       # mixer_*_fwd(raw, wf, h, planar)
            raw, wf, h = ctx.saved_tensors
            draw, dwf, dh = bwd_op(dy.contiguous(), raw, wf, h, ctx.rest[3])
            return draw, dwf, dh, None
        return backward
    reg("gcg::mixer_se_fwd", mixer(ops.mixer_se_bwd), setup_context=save(0, 1, 2))
    reg("gcg::mixer_mr_fwd", mixer(ops.mixer_mr_bwd), setup_context=save(0, 1, 2))

    def filter_decay(ctx, dh):       # filter_decay_fwd(w, decay, hl, dtype): decay is a buffer (explicit.py:46, :64)
        (decay,) = ctx.saved_tensors
        return ops.filter_decay_bwd(dh.contiguous(), decay), None, None, None
    reg("gcg::filter_decay_fwd", filter_decay, setup_context=save(1))

    def mixer_mr_decay(ctx, dy):     # mixer_mr_fwd_decay(raw, wf, w, decay, hl, filt, planar)
        raw, wf, w, decay = ctx.saved_tensors
        draw, dwf, dw = ops.mixer_mr_bwd_decay(dy.contiguous(), raw, wf, w, decay, *ctx.rest[4:7])
        return draw, dwf, dw, None, None, None, None
    reg("gcg::mixer_mr_fwd_decay", mixer_mr_decay, setup_context=save(0, 1, 2, 3))

    def time_major(ctx, dy):         # fwd_time_major(x, B, C, h)
        x, B, C, h = ctx.saved_tensors
        return ops.bwd_time_major(dy.contiguous(), x, B, C, h)
    reg("gcg::fwd_time_major", time_major, setup_context=save(0, 1, 2, 3))

    def gated_decay(ctx, dy):        # fwd_decay(x, B, C, w, decay, hl, filt)
        x, B, C, w, decay = ctx.saved_tensors
        dx, dB, dC, dw = ops.bwd_decay(dy.contiguous(), x, B, C, w, decay, *ctx.rest[5:7])
        return dx, dB, dC, dw, None, None, None
    reg("gcg::fwd_decay", gated_decay, setup_context=save(0, 1, 2, 3, 4))

    def interleaved_decay(ctx, dy):  # fwd_interleaved_decay(feat, w, decay, hl, filt)
        feat, w, decay = ctx.saved_tensors
        dfeat, dw = ops.bwd_interleaved_decay(dy.contiguous(), feat, w, decay, *ctx.rest[3:5], False)
        return dfeat, dw, None, None, None
    reg("gcg::fwd_interleaved_decay", interleaved_decay, setup_context=save(0, 1, 2))

    def refuse(name, hint):
        def backward(ctx, *grads):
            raise RuntimeError(f"torch.ops.gcg.{name} is not differentiable; {hint}")
        return backward
    reg("gcg::fwd_full", refuse("fwd_full", "use torch.ops.gcg.fwd for a differentiable y"), setup_context=lambda ctx, inputs, output: None)


if AVAILABLE:
    _register_autograd()
