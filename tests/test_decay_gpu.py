"""The Hyena-MR operator with its decayed explicit filter formed inside the convolution kernels
(gcg_fwd_decay, gcg_bwd_decay and the interleaved pair): h = F(w[:, :hl] * decay[:, :hl]) as
ExplicitSingleDecayFilter.filter computes it (savanna/model/operators/hyena/parametrization/explicit.py:68-75,
sliced and cast as savanna/model/operators/hyena/hyena.py:440-441, :499-503), and the gradient of w as autograd
derives it.  Checked against the oracle fed with that expression, and bit for bit against the chain of entry
points (filter launch, convolution, filter-gradient launch) that the fused calls replace."""
import pytest
import torch

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# (bs, L, g, dg, hl, l_cache)
SHAPES = [
    (2, 300, 3, 16, 128, 128),
    (1, 1000, 5, 16, 100, 128),     # filter shorter than the parameter: the rest of dw is zero
    (1, 2049, 20, 16, 97, 200),
    (2, 200, 2, 32, 64, 64),        # two 16-channel blocks per group
    (1, 260, 2, 128, 128, 128),     # a group wider than a 4-wave workgroup: separate filter-gradient reduction
    (3, 2500, 10, 16, 128, 128),
    (2, 40, 2, 16, 33, 128),        # sequence shorter than hyena_mr_len
]
# tensors' dtype, filter dtype
TYPES = [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16), (torch.float32, torch.float32),
         (torch.bfloat16, torch.float32)]


def make(bs, L, g, dg, hl, lc, dtype, seed=0):
    gen = torch.Generator().manual_seed(seed)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(3))
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    w = torch.randn(g, lc, generator=gen) / lc ** 0.5
    rates = torch.logspace(0, 2, g)[:, None]
    decay = torch.exp(-rates * torch.linspace(0, 1, lc)[None])
    return x, B, C, dy, w, decay


def _cases():
    for shape in SHAPES:
        for dtype, filt in TYPES:
            yield pytest.param(*shape, dtype, filt, id="x".join(map(str, shape)) + f"-{str(dtype)[6:]}-{str(filt)[6:]}")


@pytest.mark.parametrize("bs,L,g,dg,hl,lc,dtype,filt", list(_cases()))
def test_against_oracle_and_chain(gcg_lib, bs, L, g, dg, hl, lc, dtype, filt):
    x, B, C, dy, w, decay = make(bs, L, g, dg, hl, lc, dtype)
    xd, Bd, Cd, dyd, wd, dd = (t.to(DEV) for t in (x, B, C, dy, w, decay))
    # explicit.py:68-75 and hyena.py:440-441, :499-503 spelled out
    h = (w[:, :hl] * decay[:, :hl])[:, None].to(filt)
    tol = TOL[dtype] if filt == dtype else 1.1 * 2.0 ** -8
    y = _lib.fwd_decay(xd, Bd, Cd, wd, dd, hl, filt)
    dx, dB, dC, dw = _lib.bwd_decay(dyd, xd, Bd, Cd, wd, dd, hl, filt)
    torch.cuda.synchronize()
    assert_close(y, oracle.gcg_fwd_oracle(x.float(), B.float(), C.float(), h.float()), tol, "y")
    ref = oracle.gcg_bwd_oracle(dy.float(), x.float(), B.float(), C.float(), h.float())
    for o, r, n in zip((dx, dB, dC), ref, ("dx", "dB", "dC")):
        assert_close(o, r, tol, n)
    dw_ref = torch.zeros(g, lc)
    dw_ref[:, :hl] = ref[3][:, 0].to(filt).float() * decay[:, :hl]       # autograd of the cast, product and slice
    assert dw.dtype == torch.float32 and dw.shape == (g, lc)
    assert_close(dw, dw_ref, TOL_DH[filt], "dw")
    assert torch.count_nonzero(dw[:, hl:]).item() == 0
    # the chain the fused calls replace: same kernels around a filter in memory, hence the same bits
    hd = _lib.filter_decay_fwd(wd, dd, hl, filt)
    _, _, y2 = _lib.fwd(xd, Bd, Cd, hd, algo="mfma")
    dx2, dB2, dC2, dh2 = _lib.bwd(dyd, xd, Bd, Cd, hd, algo="mfma")
    dw2 = _lib.filter_decay_bwd(dh2, dd)
    for a, b, n in ((y, y2, "y"), (dx, dx2, "dx"), (dB, dB2, "dB"), (dC, dC2, "dC"), (dw, dw2, "dw")):
        assert torch.equal(a, b), n


@pytest.mark.parametrize("dtype,filt", TYPES)
def test_interleaved(gcg_lib, dtype, filt):
    bs, L, g, dg, hl, lc = 2, 700, 6, 16, 128, 160
    x, B, C, dy, w, decay = make(bs, L, g, dg, hl, lc, dtype, seed=2)
    feat = torch.stack([C, B, x], dim=-1).contiguous().to(DEV)
    wd, dd, dyd = w.to(DEV), decay.to(DEV), dy.to(DEV)
    y = _lib.fwd_interleaved_decay(feat, wd, dd, hl, filt)
    dfeat, dw = _lib.bwd_interleaved_decay(dyd, feat, wd, dd, hl, filt)
    hd = _lib.filter_decay_fwd(wd, dd, hl, filt)
    assert torch.equal(y, _lib.fwd_interleaved(feat, hd, algo="mfma"))
    dfeat2, dh2 = _lib.bwd_interleaved(dyd, feat, hd, algo="mfma")
    assert torch.equal(dfeat, dfeat2)
    assert torch.equal(dw, _lib.filter_decay_bwd(dh2, dd))
    # and the separate-tensor fused calls on the same values
    assert torch.equal(y, _lib.fwd_decay(x.to(DEV), B.to(DEV), C.to(DEV), wd, dd, hl, filt))


def test_shapes_outside_the_matrix_core_kernels_are_refused(gcg_lib):
    x, B, C, dy, w, decay = (t.to(DEV) for t in make(1, 64, 2, 8, 7, 16, torch.bfloat16))
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.fwd_decay(x, B, C, w, decay, 7, torch.bfloat16)                # dg = 8
    x, B, C, dy, w, decay = (t.to(DEV) for t in make(1, 64, 2, 16, 200, 256, torch.bfloat16))
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.bwd_decay(dy, x, B, C, w, decay, 200, torch.bfloat16)          # hl > 128
    assert not _lib.decay_supported(2, 8, 7) and not _lib.decay_supported(2, 16, 200) and _lib.decay_supported(2, 16, 128)


@pytest.mark.parametrize("act,cgcg", [(torch.bfloat16, "bfloat16"), (torch.float32, "float32"),
                                      (torch.bfloat16, "float32")])
@pytest.mark.parametrize("interleaved", [False, True])
def test_operator_launches_nothing_but_the_convolution(gcg_lib, act, cgcg, interleaved):
    """HyenaMROperator with the filter formed in the kernels: same output and gradients, bit for bit, as with
    the filter made by its own launches, and a kernel trace that holds the two convolution kernels only."""
    from savanna_amd.operators.hyena import CgcgConfig, HyenaMROperator

    torch.manual_seed(0)
    bs, L, g, dg = 2, 384, 4, 16
    op = HyenaMROperator(g * dg, g, 128, CgcgConfig(cgcg_dtype=cgcg), small_init=False, device=DEV)
    feats = torch.randn(bs, L, g, dg, 3, device=DEV).to(act).requires_grad_(True)
    dz = (0.1 * torch.randn(bs, L, g * dg, device=DEV)).to(act)

    def run(fuse):
        op.fuse_filter = fuse
        feats.grad = op.filter.h.grad = None
        if interleaved:
            z = op.forward_features(feats.reshape(bs, L, 3 * g * dg))
        else:
            x1, x2, v = feats.unbind(dim=-1)
            z = op(x1, x2, v)
        z.backward(dz)
        return z.detach(), feats.grad.clone(), op.filter.h.grad.clone()

    want = run(False)
    from torch.profiler import ProfilerActivity, profile
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        got = run(True)
        torch.cuda.synchronize()
    for a, b, n in zip(got, want, ("z", "dfeatures", "dw")):
        assert a.dtype == b.dtype and torch.equal(a, b), n
    kernels = [e.key for e in prof.key_averages() if e.device_time_total > 0 and "Memcpy" not in e.key
               and "Memset" not in e.key]
    ours = [k for k in kernels if "gcg::" in k]
    assert len(ours) == 2 and all("mfma" in k for k in ours), kernels
    if interleaved:       # (on the split views autograd itself re-assembles the gradient of the features)
        assert len(kernels) == 2, kernels
