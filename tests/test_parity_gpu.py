"""Parity of the HIP kernels with the CPU oracle, through the C ABI (ctypes binding in
savanna_amd/_lib.py).  Modelled on the reference's tests/test_fwd_refactor.py:53-114 and
tests/test_bwd_refactor.py:70-143: same quantities (Bx, y2, y; dx, dB, dC, dh), same
parameter grid style, seeded CPU inputs so checker and kernel see identical values.
"""
import pytest
import torch

from helpers import TOL, TOL_DH, assert_close, inputs, oracle_bwd, oracle_fwd
from savanna_amd import _lib

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]
MFMA_BWD = True


def algos_for(hl, dg, dtype):
    out = ["direct"]
    if hl <= 8 and dg % 4 == 0:
        out.append("window")
    if hl <= 128 and dg % 16 == 0:
        out.append("mfma")
    return out


# (bs, L, g, dg, hl): ragged lengths, partial channel tiles, one-tap and full-length filters
SMALL = [
    (1, 32, 1, 16, 4),
    (2, 32, 2, 32, 4),       # the reference's debug configs (tests/test_fwd_refactor.py:33-36)
    (2, 128, 2, 16, 128),
    (1, 256, 4, 16, 128),
    (2, 300, 3, 16, 128),    # L not a multiple of the chunk
    (1, 1000, 5, 16, 100),   # filter shorter than the chunk, d = 80 (partial 64-channel tile)
    (1, 513, 2, 48, 33),
    (2, 200, 4, 16, 7),
    (1, 77, 8, 4, 7),        # dg below the matrix-core width
    (3, 130, 2, 20, 3),
    (1, 64, 6, 1, 5),        # one channel per filter
    (1, 70, 2, 24, 1),       # single tap
    (1, 400, 1, 64, 8),
    (1, 700, 2, 16, 200),    # filter longer than a chunk (direct kernel only)
    (1, 200, 17, 16, 64),    # d = 272: a 256-channel workgroup plus a block with one live wave
    (1, 100, 9, 16, 128),    # d = 144: partial 128-channel block
    (2, 5, 2, 16, 128),      # sequence shorter than one step and than the filter
    (1, 1, 1, 16, 7),        # a single row
    (1, 2049, 20, 16, 97),   # odd length, odd filter, d = 320
    (3, 2500, 10, 16, 128),  # odd batch, ragged length: several runs per column and more than one round of workgroups
    (5, 1111, 3, 16, 65),
]


def _cases(backward=False):
    for shape in SMALL:
        bs, L, g, dg, hl = shape
        for dtype in DTYPES:
            for algo in algos_for(hl, dg, dtype):
                if backward and algo == "mfma" and not MFMA_BWD:
                    continue
                yield pytest.param(*shape, dtype, algo, id=f"{bs}x{L}x{g}x{dg}-hl{hl}-{str(dtype)[6:]}-{algo}")


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype,algo", list(_cases()))
def test_fwd_small(gcg_lib, bs, L, g, dg, hl, dtype, algo):
    x, B, C, h, _ = inputs(bs, L, g, dg, hl, dtype)
    bx_ref, y2_ref, y_ref = oracle_fwd(x, B, C, h)
    bx, y2, y = _lib.fwd(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), return_bx=True, return_y2=True, algo=algo)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == (bs, L, g, dg)
    assert_close(bx, bx_ref, TOL[dtype], "Bx")
    assert_close(y2, y2_ref, TOL[dtype], "y2")
    assert_close(y, y_ref, TOL[dtype], "y")
    # outputs that were not requested must not be needed
    _, _, y_only = _lib.fwd(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), algo=algo)
    assert torch.equal(y_only, y)


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype,algo", list(_cases(backward=True)))
def test_bwd_small(gcg_lib, bs, L, g, dg, hl, dtype, algo):
    x, B, C, h, dy = inputs(bs, L, g, dg, hl, dtype, seed=1, dy_scale=0.1)  # dy = 0.1*randn as in test_bwd_refactor.py:98
    ref = oracle_bwd(dy, x, B, C, h)
    got = _lib.bwd(dy.to(DEV), x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), algo=algo)
    torch.cuda.synchronize()
    few_terms = algo == "mfma" and bs * L * dg < 256
    for o, r, n in zip(got, ref, ("dx", "dB", "dC", "dh")):
        assert o.dtype == dtype
        if n == "dh" and few_terms:
            continue
        assert_close(o, r, TOL_DH[dtype] if n == "dh" else TOL[dtype], n)
    if few_terms:
        # The matrix cores take u = B*x and g2 = dy*C rounded to the I/O type (as the reference's
        # tl.dot on bf16 Bx and its bf16 dy2 buffer do).  With only a handful of products per tap
        # nothing averages that rounding out and a tap's sum can cancel, so dh is checked against
        # the oracle fed with the rounded products: dh depends on the inputs only through u and g2.
        u = (B.float() * x.float()).to(dtype)
        g2 = (dy.float() * C.float()).to(dtype)
        one = torch.ones_like(u)
        dh_ref = oracle_bwd(g2, u, one, one, h)[3]
        assert_close(got[3], dh_ref, TOL_DH[dtype], "dh (rounded products)")


@pytest.mark.parametrize("algo", ["direct", "window"])
def test_bwd_is_deterministic(gcg_lib, algo):
    x, B, C, h, dy = (t.to(DEV) for t in inputs(2, 512, 4, 16, 7, torch.float32, seed=3))
    a = _lib.bwd(dy, x, B, C, h, algo=algo)
    b = _lib.bwd(dy, x, B, C, h, algo=algo)
    for u, v in zip(a, b):
        assert torch.equal(u, v)


def test_error_codes(gcg_lib):
    x, B, C, h, dy = (t.to(DEV) for t in inputs(1, 64, 2, 16, 200, torch.bfloat16))
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.fwd(x, B, C, h, algo="mfma")        # hl > 128
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.fwd(x, B, C, h, algo="window")      # hl > 8
    with pytest.raises(RuntimeError, match="no CPU path"):
        _lib.fwd(x.cpu(), B.cpu(), C.cpu(), h.cpu())
    lib = _lib.load()
    assert lib.gcg_fwd(None, B.data_ptr(), C.data_ptr(), h.data_ptr(), x.data_ptr(), None, None,
                       1, 64, 2, 16, 200, 1, 0, None) == -1
    assert lib.gcg_bwd(dy.data_ptr(), x.data_ptr(), B.data_ptr(), C.data_ptr(), h.data_ptr(),
                       x.data_ptr(), x.data_ptr(), x.data_ptr(), h.data_ptr(), None, 0,
                       1, 64, 2, 16, 200, 1, 0, None) == -3


@pytest.mark.parametrize("dtype,hl", [(torch.bfloat16, 128), (torch.float32, 7)])
def test_misaligned_tensors_take_the_direct_kernels(gcg_lib, dtype, hl):
    """The vector kernels need 16-byte aligned tensors; a view that starts one element into its
    storage is re-routed to the element-wise direct kernels under automatic selection and is
    refused when a vector family is forced."""
    bs, L, g, dg = 1, 200, 2, 16
    x, B, C, h, dy = inputs(bs, L, g, dg, hl, dtype, seed=7, dy_scale=0.1)
    n = bs * L * g * dg

    def shifted(t):
        buf = torch.empty(n + 1, dtype=dtype, device=DEV)
        v = buf[1:].view(bs, L, g, dg)
        v.copy_(t)
        assert v.data_ptr() % 16 != 0 and v.is_contiguous()
        return v

    xs, Bs, Cs, dys = shifted(x), shifted(B), shifted(C), shifted(dy)
    hd = h.to(DEV)
    _, _, y = _lib.fwd(xs, Bs, Cs, hd)
    assert_close(y, oracle_fwd(x, B, C, h)[2], TOL[dtype], "y")
    got = _lib.bwd(dys, xs, Bs, Cs, hd)
    for o, r_, n_ in zip(got, oracle_bwd(dy, x, B, C, h), ("dx", "dB", "dC", "dh")):
        assert_close(o, r_, TOL_DH[dtype] if n_ == "dh" else TOL[dtype], n_)
    forced = "mfma" if hl > 8 else "window"
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.fwd(xs, Bs, Cs, hd, algo=forced)


def test_kernel_timer_hook(gcg_lib):
    """gcg_time_next_kernel: the armed events are stamped by the next call's main kernel only, the arming lasts
    one call, and results are what they are without it."""
    import ctypes

    hip = None
    with open("/proc/self/maps") as f:
        for line in f:
            if "libamdhip64" in line:
                hip = ctypes.CDLL(line.split()[-1])
                break
    assert hip is not None
    hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
    hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipEventCreate(ctypes.byref(a)) == 0 and hip.hipEventCreate(ctypes.byref(b)) == 0
    x, B, C, h, dy = (t.to(DEV) for t in inputs(2, 2048, 16, 16, 128, torch.bfloat16, seed=3, dy_scale=0.1))
    want = _lib.bwd(dy, x, B, C, h)
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    assert gcg_lib.gcg_time_next_kernel(a, None) == -1             # one null pointer
    _lib.time_next_kernel(a, b)
    t0.record()
    got = _lib.bwd(dy, x, B, C, h)
    t1.record()
    torch.cuda.synchronize()
    ms = ctypes.c_float()
    assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
    assert 0.0 < ms.value <= t0.elapsed_time(t1)                   # inside the bracket around the whole call
    for g_, w_ in zip(got, want):
        assert torch.equal(g_, w_)
    # one call per arming: the next call leaves the events alone, and a forward takes them when armed again
    before = ms.value
    _lib.bwd(dy, x, B, C, h)
    torch.cuda.synchronize()
    assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0 and ms.value == before
    _lib.time_next_kernel(a, b)
    _lib.fwd(x, B, C, h)
    torch.cuda.synchronize()
    assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0 and ms.value > 0.0
    hip.hipEventDestroy(a)
    hip.hipEventDestroy(b)
