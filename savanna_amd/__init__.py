"""MI355X-native gated chunked causal convolution (Hyena-SE / Hyena-MR).

A drop-in for savanna's ``gcg_two_pass`` path: the hand-written HIP kernels live in
``csrc/`` behind the C ABI of ``include/gcg.h``; ``kernels/cgcg`` mirrors the
reference's Python entry points (savanna/kernels/triton_src/cgcg) and
``operators/hyena.py`` the operator dispatch that calls them.
"""
from .kernels.cgcg.interface import two_pass_chunked_gate_conv_gate  # noqa: F401

__version__ = "0.1.0"
