"""gcg_bwd_static -- the backward that allocates nothing (its filter-gradient scratch is a device array inside
the library) -- against gcg_bwd with a caller's workspace, through the C ABI.  Both run the same kernels with
the same order of summation, so every output must agree bit for bit.  Each case makes two calls in a row, the
second on a smaller input, because all calls on a GPU share the one array, which keeps the last call's contents.
The file's name makes pytest collect it last.
"""
import pytest
import torch

from helpers import inputs
from savanna_amd import _lib

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def both_ways(shape, dtype, algo, seed):
    bs, L, g, dg, hl = shape
    x, B, C, h, dy = (t.to(DEV) for t in inputs(bs, L, g, dg, hl, dtype, seed=seed))
    ref = _lib.bwd(dy, x, B, C, h, algo=algo)
    # poisoned outputs: whatever the call leaves unwritten shows
    outs = [torch.full_like(x, float("nan")) for _ in range(3)] + [torch.full_like(h, float("nan"))]
    _lib.bwd_static(dy, x, B, C, h, *outs, algo=algo)
    torch.cuda.synchronize()
    for name, got, want in zip(("dx", "dB", "dC", "dh"), outs, ref):
        assert torch.equal(got, want), f"{name} differs from gcg_bwd for {shape} {dtype} {algo}"


# (first call, second and smaller call) per kernel family
PAIRS = [
    ("mfma", torch.bfloat16, (2, 1500, 6, 16, 128), (1, 300, 3, 16, 128)),
    ("mfma", torch.float32, (1, 700, 4, 16, 100), (1, 96, 2, 16, 33)),
    ("window", torch.bfloat16, (2, 2000, 8, 16, 7), (1, 130, 2, 16, 7)),
    ("window", torch.float32, (1, 900, 4, 8, 4), (1, 64, 1, 8, 3)),
    ("direct", torch.float16, (1, 700, 2, 16, 200), (1, 150, 1, 16, 150)),
    ("auto", torch.bfloat16, (3, 1111, 5, 16, 65), (1, 40, 1, 16, 65)),
]


@pytest.mark.parametrize("algo,dtype,big,small", PAIRS)
def test_static_scratch_matches_workspace(gcg_lib, algo, dtype, big, small):
    both_ways(big, dtype, algo, seed=1)
    both_ways(small, dtype, algo, seed=2)


def test_headline_shape_fits_and_matches(gcg_lib):
    """The Evo2-7B layer shape of the headline workload, then a smaller call straight after it."""
    both_ways((2, 8192, 256, 16, 128), torch.bfloat16, "auto", seed=3)
    both_ways((1, 512, 8, 16, 128), torch.bfloat16, "auto", seed=4)


def test_sizes_beyond_the_scratch_are_rejected(gcg_lib):
    """A shape whose partials need more than the built-in array is refused with its own error code and message,
    before anything is launched."""
    bs, L, g, dg, hl = 4, 1 << 17, 512, 16, 7
    code = _lib.dtype_code(torch.bfloat16)
    need = gcg_lib.gcg_bwd_workspace_bytes(bs, L, g, dg, hl, code, _lib.ALGO_AUTO)
    assert need > _lib.STATIC_SCRATCH_BYTES
    one = torch.zeros(64, device=DEV)       # never dereferenced: the size check comes first
    p = one.data_ptr()
    rc = gcg_lib.gcg_bwd_static(p, p, p, p, p, p, p, p, p, bs, L, g, dg, hl, code, _lib.ALGO_AUTO, None)
    assert rc == -6
    assert b"gcg_bwd_static" in gcg_lib.gcg_strerror(rc)
