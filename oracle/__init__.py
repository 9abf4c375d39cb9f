"""CPU oracle for the gated chunked causal convolution (test infrastructure only).

Only tests/, the smoke check and the CPU-baseline leg of the benchmark may import
this package; the shipped code under savanna_amd/ never does.
"""
from .gcg_ref import (  # noqa: F401
    bf16_round,
    brute_force_fwd,
    correction_toeplitz,
    gcg_bwd_oracle,
    gcg_bwd_ref_torch,
    gcg_fwd_oracle,
    gcg_fwd_ref_torch,
    gcg_two_pass_chunked_bwd,
    gcg_two_pass_chunked_fwd,
    load_c_oracle,
    toeplitz,
)
