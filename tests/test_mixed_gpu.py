"""16-bit tensors with an fp32 filter and fp32 arithmetic (GCG_BF16_F32 / GCG_F16_F32): the operator as the
reference runs it when ``cgcg_dtype`` is float32 (its default, savanna/arguments/global_config.py:404) and the
activations are bf16 -- tensors cast up before the call, the result cast down after it
(savanna/model/operators/hyena/hyena.py:499-503, :533-534) -- without those casts.

The oracle is fed the 16-bit tensors widened to fp32 and the unrounded fp32 filter.  Outputs are 16-bit, so
besides the error bar (half a unit in the last place of the largest value) the tests count how many elements
equal the oracle's result rounded once: arithmetic or a filter rounded to 16 bits anywhere inside would leave
about half of them different.  The filter gradient is fp32 and meets the fp32 bar.
"""
import pytest
import torch

import oracle
from helpers import TOL_DH, assert_close, rel_err
from savanna_amd import _lib

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
HALF_ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}     # of the largest value, relative to it

SHAPES = [
    (2, 128, 2, 16, 128),
    (2, 300, 3, 16, 128),     # ragged length
    (1, 1000, 5, 16, 100),    # partial channel tile
    (1, 513, 2, 48, 33),
    (2, 200, 4, 16, 7),
    (1, 77, 8, 4, 7),
    (3, 130, 2, 20, 3),
    (1, 200, 17, 16, 64),
    (2, 5, 2, 16, 128),
    (3, 2500, 10, 16, 128),   # several runs per column
    (1, 700, 2, 16, 200),     # direct kernels only
]


def algos_for(hl, dg):
    out = ["direct"]
    if hl <= 8 and dg % 4 == 0:
        out.append("window")
    if hl <= 128 and dg % 16 == 0:
        out.append("mfma")
    return out


def mixed_inputs(bs, L, g, dg, hl, dtype, seed=0):
    gen = torch.Generator().manual_seed(seed)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(3))
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    h = torch.randn(g, 1, hl, generator=gen) / max(1.0, hl ** 0.5)          # fp32, not representable in 16 bits
    return x, B, C, h, dy


def check_rounded_once(out, ref, dtype, what, min_equal=0.98):
    assert out.dtype == dtype
    assert_close(out, ref, 1.1 * HALF_ULP[dtype], what)
    equal = (out.cpu() == ref.to(dtype)).float().mean().item()
    assert equal >= min_equal, f"{what}: only {equal:.3f} of the elements equal the fp32 result rounded once"


def _cases():
    for shape in SHAPES:
        bs, L, g, dg, hl = shape
        for dtype in (torch.bfloat16, torch.float16):
            for algo in algos_for(hl, dg):
                yield pytest.param(*shape, dtype, algo, id=f"{bs}x{L}x{g}x{dg}-hl{hl}-{str(dtype)[6:]}-{algo}")


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype,algo", list(_cases()))
def test_fwd(gcg_lib, bs, L, g, dg, hl, dtype, algo):
    x, B, C, h, _ = mixed_inputs(bs, L, g, dg, hl, dtype)
    bx_ref, y2_ref, y_ref = oracle.gcg_fwd_oracle(x.float(), B.float(), C.float(), h, return_intermediates=True)
    bx, y2, y = _lib.fwd(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), return_bx=True, return_y2=True, algo=algo)
    torch.cuda.synchronize()
    check_rounded_once(y, y_ref, dtype, "y")
    check_rounded_once(y2, y2_ref, dtype, "y2")
    check_rounded_once(bx, bx_ref, dtype, "Bx", min_equal=1.0)          # one product, rounded once
    _, _, y_only = _lib.fwd(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), algo=algo)
    assert torch.equal(y_only, y)


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype,algo", list(_cases()))
def test_bwd(gcg_lib, bs, L, g, dg, hl, dtype, algo):
    x, B, C, h, dy = mixed_inputs(bs, L, g, dg, hl, dtype, seed=1)
    ref = oracle.gcg_bwd_oracle(dy.float(), x.float(), B.float(), C.float(), h)
    got = _lib.bwd(dy.to(DEV), x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), algo=algo)
    torch.cuda.synchronize()
    for o, r, n in zip(got[:3], ref[:3], ("dx", "dB", "dC")):
        check_rounded_once(o, r, dtype, n)
    assert got[3].dtype == torch.float32 and got[3].shape == h.shape
    assert_close(got[3], ref[3], TOL_DH[torch.float32], "dh")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("bs,L", [(2, 8192), (1, 8192 + 77)], ids=["7b", "ragged"])
def test_full_size_runs(gcg_lib, bs, L, dtype):
    """fp32 arithmetic at the Evo2-7B layer shape (runs of 128 steps: every phase of the kernels' rings, the
    lead-in of a run that starts mid-sequence, the ragged last step), four filter groups against the oracle."""
    g, dg, hl = 256, 16, 128
    gen = torch.Generator(device=DEV).manual_seed(17)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen, device=DEV).to(dtype) for _ in range(3))
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=DEV)).to(dtype)
    h = torch.randn(g, 1, hl, generator=gen, device=DEV) / hl ** 0.5
    _, _, y = _lib.fwd(x, B, C, h)
    dx, dB, dC, dh = _lib.bwd(dy, x, B, C, h)
    torch.cuda.synchronize()
    assert _lib.select_algo(bs, L, g, dg, hl, dtype, True) == "mfma"
    idx = torch.tensor([0, 3, 130, 255], device=DEV)
    xs, Bs, Cs, dys = (t.index_select(2, idx).float().cpu() for t in (x, B, C, dy))
    hs = h.index_select(0, idx).cpu()
    y_ref = oracle.gcg_fwd_oracle(xs, Bs, Cs, hs)
    ref = oracle.gcg_bwd_oracle(dys, xs, Bs, Cs, hs)
    check_rounded_once(y.index_select(2, idx), y_ref, dtype, "y")
    for o, r, n in zip((dx, dB, dC), ref[:3], ("dx", "dB", "dC")):
        check_rounded_once(o.index_select(2, idx), r, dtype, n)
    assert_close(dh.index_select(0, idx), ref[3], TOL_DH[torch.float32], "dh")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hl", [7, 128])
def test_interleaved(gcg_lib, dtype, hl):
    bs, L, g, dg = 2, 700, 6, 16
    x, B, C, h, dy = mixed_inputs(bs, L, g, dg, hl, dtype, seed=2)
    feat = torch.stack([C, B, x], dim=-1).contiguous().to(DEV)
    y = _lib.fwd_interleaved(feat, h.to(DEV))
    dfeat, dh = _lib.bwd_interleaved(dy.to(DEV), feat, h.to(DEV))
    torch.cuda.synchronize()
    # the separate-tensor kernels on the same values: same arithmetic, so the same bits (dh up to summation order)
    _, _, y_sep = _lib.fwd(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV))
    dx, dB, dC, dh_sep = _lib.bwd(dy.to(DEV), x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV))
    if hl > 8:      # matrix-core kernels: the two layouts share the product side bit for bit
        assert torch.equal(y, y_sep)
        assert torch.equal(dfeat[..., 0], dC) and torch.equal(dfeat[..., 1], dB) and torch.equal(dfeat[..., 2], dx)
    else:           # register-window kernels: other lane widths, fp32 sums in another order
        for a, b in ((y, y_sep), (dfeat[..., 0], dC), (dfeat[..., 1], dB), (dfeat[..., 2], dx)):
            assert (a == b).float().mean().item() >= 0.98
    assert_close(dh, dh_sep, 1e-6, "dh against the separate-tensor kernels")
    ref = oracle.gcg_bwd_oracle(dy.float(), x.float(), B.float(), C.float(), h)
    check_rounded_once(y, oracle.gcg_fwd_oracle(x.float(), B.float(), C.float(), h), dtype, "y")
    check_rounded_once(dfeat[..., 2], ref[0], dtype, "dx")
    assert dh.dtype == torch.float32
    assert_close(dh, ref[3], TOL_DH[torch.float32], "dh")


def test_long_sequence_fp32_arithmetic(gcg_lib):
    """A quarter of a million tokens: long runs (256 steps and more per workgroup), window offsets in the hundreds of
    megabytes; two filter groups against the oracle, interleaved against separate."""
    bs, L, g, dg, hl, dtype = 1, 262144 + 19, 32, 16, 128, torch.bfloat16
    gen = torch.Generator(device=DEV).manual_seed(23)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen, device=DEV).to(dtype) for _ in range(3))
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=DEV)).to(dtype)
    h = torch.randn(g, 1, hl, generator=gen, device=DEV) / hl ** 0.5
    _, _, y = _lib.fwd(x, B, C, h)
    dx, dB, dC, dh = _lib.bwd(dy, x, B, C, h)
    feat = torch.stack([C, B, x], dim=-1).contiguous()
    dfeat, dh_i = _lib.bwd_interleaved(dy, feat, h)
    torch.cuda.synchronize()
    assert torch.equal(dfeat[..., 0], dC) and torch.equal(dfeat[..., 1], dB) and torch.equal(dfeat[..., 2], dx)
    assert_close(dh_i, dh, 1e-6, "dh interleaved against separate")
    idx = torch.tensor([0, 31], device=DEV)
    xs, Bs, Cs, dys = (t.index_select(2, idx).float().cpu() for t in (x, B, C, dy))
    hs = h.index_select(0, idx).cpu()
    ref = oracle.gcg_bwd_oracle(dys, xs, Bs, Cs, hs)
    check_rounded_once(y.index_select(2, idx), oracle.gcg_fwd_oracle(xs, Bs, Cs, hs), dtype, "y")
    for o, r, n in zip((dx, dB, dC), ref[:3], ("dx", "dB", "dC")):
        check_rounded_once(o.index_select(2, idx), r, dtype, n)
    assert_close(dh.index_select(0, idx), ref[3], TOL_DH[torch.float32], "dh")


def _random_shapes(n=24, seed=5):
    """Shapes around the limits of the five-slice kernels: filter lengths 97..128, ragged lengths from less than one
    step to several runs, channel counts that leave waves or lanes of a workgroup without work."""
    import random
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        dg = rnd.choice([16, 16, 32, 48])
        g = rnd.choice([1, 2, 3, 5, 8, 20])
        L = rnd.choice([rnd.randint(1, 40), rnd.randint(41, 400), rnd.randint(401, 3000)])
        out.append((rnd.choice([1, 2, 3]), L, g, dg, rnd.randint(97, 128)))
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("bs,L,g,dg,hl", _random_shapes(), ids=lambda v: str(v))
def test_random_shapes_fp32_arithmetic(gcg_lib, bs, L, g, dg, hl, dtype):
    """16-bit tensors in fp32 arithmetic on separate and on interleaved tensors against the oracle, and against
    each other bit for bit (the two layouts add the same plane products in the same order, whichever kernel
    runs them: for f16 the separate tensors take the kernel with product waves and row waves, the interleaved
    ones the 4-wave kernel)."""
    x, B, C, h, dy = mixed_inputs(bs, L, g, dg, hl, dtype, seed=bs * 1000 + L)
    xd, Bd, Cd, hd, dyd = (t.to(DEV) for t in (x, B, C, h, dy))
    _, _, y = _lib.fwd(xd, Bd, Cd, hd, algo="mfma")
    dx, dB, dC, dh = _lib.bwd(dyd, xd, Bd, Cd, hd, algo="mfma")
    feat = torch.stack([Cd, Bd, xd], dim=-1).contiguous()
    y_i = _lib.fwd_interleaved(feat, hd)
    dfeat, dh_i = _lib.bwd_interleaved(dyd, feat, hd)
    torch.cuda.synchronize()
    ref = oracle.gcg_bwd_oracle(dy.float(), x.float(), B.float(), C.float(), h)
    check_rounded_once(y, oracle.gcg_fwd_oracle(x.float(), B.float(), C.float(), h), dtype, "y", min_equal=0.97)
    for o, r, n in zip((dx, dB, dC), ref[:3], ("dx", "dB", "dC")):
        check_rounded_once(o, r, dtype, n, min_equal=0.97)
    assert_close(dh, ref[3], TOL_DH[torch.float32], "dh")
    assert torch.equal(y_i, y)
    assert torch.equal(dfeat[..., 0], dC) and torch.equal(dfeat[..., 1], dB) and torch.equal(dfeat[..., 2], dx)
    assert_close(dh_i, dh, 1e-6, "dh interleaved against separate")


def test_fp32_filter_needs_16_bit_tensors(gcg_lib):
    x, B, C, h, _ = mixed_inputs(1, 64, 2, 16, 7, torch.bfloat16)
    with pytest.raises((TypeError, RuntimeError), match="filter"):
        _lib.fwd(x.float().to(DEV), B.float().to(DEV), C.float().to(DEV), h.to(torch.bfloat16).to(DEV))
    # the featurizer entry points have no such mode
    lib = _lib.load()
    t = x.to(DEV)
    assert lib.gcg_dwconv_fwd(t.data_ptr(), t.data_ptr(), t.data_ptr(), 1, 64, 2, 16, 3, _lib.GCG_BF16_F32, 0, None) == -1


@pytest.mark.parametrize("kind", ["mr", "se"])
def test_operator_with_fp32_cgcg_dtype(gcg_lib, kind):
    """HyenaMROperator / HyenaSEOperator with cgcg_dtype float32 (the reference's default) on bf16 activations:
    the same values as casting the tensors up, running the fp32 kernels and casting the result down
    (hyena.py:499-503, :533-534), gradients included, from one kernel each way."""
    from savanna_amd.operators.hyena import CgcgConfig, HyenaMROperator, HyenaSEOperator

    torch.manual_seed(0)
    bs, L, g, dg = 2, 384, 4, 16
    cfg = CgcgConfig(cgcg_dtype="float32")
    op = (HyenaMROperator(g * dg, g, 128, cfg, small_init=False, device=DEV) if kind == "mr"
          else HyenaSEOperator(g * dg, g, 7, cfg, device=DEV))
    x1, x2, v = (torch.randn(bs, L, g, dg, device=DEV).to(torch.bfloat16).requires_grad_(True) for _ in range(3))
    dz = (0.1 * torch.randn(bs, L, g * dg, device=DEV)).to(torch.bfloat16)
    z = op(x1, x2, v)
    assert z.dtype == torch.bfloat16
    z.backward(dz)
    got = [z.detach()] + [t.grad.clone() for t in (x1, x2, v)] + [p.grad.clone() for p in op.parameters()]
    for t in (x1, x2, v, *op.parameters()):
        t.grad = None
    # the reference's flow, spelled out
    h = op._filter(L).to(torch.float32)
    z2 = op.cgcg_fn(x=v.float(), B=x2.float(), C=x1.float(), h=h, bs=bs, seqlen=L, g=g, dg=dg, fwd_autotune=False,
                    bwd_autotune=True, fused_bwd=True, fwd_kernel_cfg=op.cgcg_fwd_config)
    z2 = z2.reshape(bs, L, g * dg).to(torch.bfloat16)
    z2.backward(dz)
    want = [z2.detach()] + [t.grad for t in (x1, x2, v)] + [p.grad for p in op.parameters()]
    for a, b, n in zip(got, want, ("z", "dx1", "dx2", "dv", "dparam")):
        assert a.dtype == b.dtype, n
        if n == "dparam":
            assert_close(a, b, 2e-5, n)
        else:
            # both round an fp32 result once; the two fp32 results differ in the last bits only
            assert (a == b).float().mean().item() >= 0.98, n
            assert rel_err(a, b.float()) <= 2.2 * HALF_ULP[torch.bfloat16], n
