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


def test_outputs_are_checked(gcg_lib):
    """A strided, short or mistyped output is refused by the binding before the kernels could write past it."""
    x, B, C, h, dy = (t.to(DEV) for t in inputs(1, 64, 2, 16, 7, torch.bfloat16, seed=5))
    good = [torch.empty_like(x) for _ in range(3)] + [torch.empty_like(h)]
    _lib.bwd_static(dy, x, B, C, h, *good)
    strided = torch.empty(1, 64, 2, 32, dtype=x.dtype, device=DEV)[..., ::2]
    short = torch.empty(1, 32, 2, 16, dtype=x.dtype, device=DEV)
    for bad_dx in (strided, short, torch.empty_like(x, dtype=torch.float32), torch.empty_like(x, device="cpu")):
        with pytest.raises(ValueError, match="dx"):
            _lib.bwd_static(dy, x, B, C, h, bad_dx, *good[1:])
    with pytest.raises(ValueError, match="dh"):
        _lib.bwd_static(dy, x, B, C, h, *good[:3], torch.empty(2, 1, 8, dtype=h.dtype, device=DEV))


@pytest.mark.parametrize("algo,dtype,shape", [("mfma", torch.bfloat16, (2, 1500, 6, 16, 128)),
                                               ("window", torch.bfloat16, (2, 2000, 8, 16, 7))])
def test_static_backward_in_a_captured_graph(gcg_lib, algo, dtype, shape):
    """The use the entry point is for: a first call outside the capture (it looks the scratch array up), then a call
    recorded into a HIP graph and replayed, with eager work of the same library between the replays; every replay
    must give gcg_bwd's bits.  Under capture the matrix-core backward adds its filter-gradient partials with a
    second kernel instead of its ticket scheme, in the same order."""
    bs, L, g, dg, hl = shape
    x, B, C, h, dy = (t.to(DEV) for t in inputs(bs, L, g, dg, hl, dtype, seed=6))
    ref = _lib.bwd(dy, x, B, C, h, algo=algo)
    outs = [torch.full_like(x, float("nan")) for _ in range(3)] + [torch.full_like(h, float("nan"))]
    _lib.bwd_static(dy, x, B, C, h, *outs, algo=algo)           # outside the capture, as the header asks
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _lib.bwd_static(dy, x, B, C, h, *outs, algo=algo)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        for o in outs:
            o.fill_(float("nan"))
        other = _lib.bwd(dy, x, B, C, h, algo=algo)              # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, want, again in zip(("dx", "dB", "dC", "dh"), outs, ref, other):
            assert torch.equal(got, want), f"replay {replay}: {name} differs from gcg_bwd"
            assert torch.equal(again, want)


def test_more_streams_than_ticket_sets(gcg_lib):
    """The matrix-core backward keeps one set of arrival tickets per stream, for 64 streams; launches on further
    streams add their filter-gradient partials with a second kernel.  Same bits either way."""
    x, B, C, h, dy = (t.to(DEV) for t in inputs(2, 700, 4, 16, 128, torch.bfloat16, seed=7))
    ref = _lib.bwd(dy, x, B, C, h, algo="mfma")
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(70)]
    results = []
    for st in streams:
        st.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(st):
            results.append(_lib.bwd(dy, x, B, C, h, algo="mfma"))
    torch.cuda.synchronize()
    for got in results:
        for a, b in zip(got, ref):
            assert torch.equal(a, b)
