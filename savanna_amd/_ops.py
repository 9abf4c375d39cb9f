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
