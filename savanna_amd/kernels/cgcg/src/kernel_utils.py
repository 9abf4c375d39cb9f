"""Kernel-config records accepted at the operator boundary.

savanna's hyena operator builds ``FwdKernelConfigRefactor`` / ``BwdKernelConfigRefactor``
objects from its YAML flags and passes them to the convolution entry point
(savanna/model/operators/hyena/hyena.py:277-293, 657-697; classes at
savanna/kernels/triton_src/cgcg/src/kernel_utils.py:268-352).  Their fields are Triton
tuning knobs.  The HIP kernels choose their own tiling, so the records are validated the
way the reference validates them, carried through, and otherwise ignored: no field
changes a result.
"""
from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Optional

_SCHEDULES = ("default", "persistent")
_SWIZZLES = ("row", "col")


@dataclass
class KernelConfig:
    CHUNK_SIZE: int                       # Triton: time rows per program
    BLOCK_D: int                          # Triton: channels per program
    THREADBLOCK_SWIZZLE: str              # "row" or "col" program ordering
    schedule: str = "default"             # "default" or "persistent"
    USE_TMA: bool = False                 # Hopper tensor-memory-accelerator variants
    FLUSH_TMA: bool = False
    NUM_PIPELINE_STAGES: int = 0          # tl.range pipelining, 0 or 1
    CHUNK_TILES_PER_PROGRAM: int = 1
    num_warps: int = 4                    # Triton launch knobs from here on
    num_stages: int = 3
    num_ctas: int = 1
    maxnreg: Optional[int] = None

    def __post_init__(self):
        # same three checks as kernel_utils.py:289-294 of the reference
        assert self.schedule in _SCHEDULES, f"schedule must be one of {_SCHEDULES}"
        assert self.THREADBLOCK_SWIZZLE in _SWIZZLES, f"THREADBLOCK_SWIZZLE must be one of {_SWIZZLES}"
        assert 0 <= self.NUM_PIPELINE_STAGES < 2, "NUM_PIPELINE_STAGES must be 0 or 1"

    def _key(self):
        return tuple(getattr(self, f.name) for f in fields(self))

    def __eq__(self, other):
        if not isinstance(other, KernelConfig):
            return NotImplemented
        return type(self) is type(other) and self._key() == other._key()

    def __hash__(self):
        return hash(self._key())

    def __str__(self):
        body = ", ".join(f"{f.name}={getattr(self, f.name)}" for f in fields(self))
        return f"{type(self).__name__}: {body}"


@dataclass(eq=False)
class FwdKernelConfigRefactor(KernelConfig):
    name: str = "fwd"
    version: str = "refactor"
    RETURN_BX: bool = True                # the reference forward also returns B*x ...
    RETURN_Y2: bool = True                # ... and the convolution before the post-gate


@dataclass
class BwdKernelConfigRefactor:
    name: str = "bwd-refactor"
    pre_conv_BLOCK_X: int = 128           # tiles of the reference's gate-and-transpose kernels
    pre_conv_BLOCK_Y: int = 128
    pre_conv_num_warps: int = 4
    post_conv_BLOCK_X: int = 128
    post_conv_BLOCK_Y: int = 128
    post_conv_num_warps: int = 4
