"""Element-wise parity in the reference's own terms.

The reference's tests compare every element with ``torch.allclose``: ``atol = rtol = 1e-4`` in fp32 and
``atol = 1e-3, rtol = 1e-2`` in bf16 (savanna/kernels/triton_src/cgcg/tests/test_bwd_refactor.py:172-177,
tests/test_fwd_refactor.py:103-114).  The bars of the other parity tests (largest error over the largest
value) cannot see a wrong output of small magnitude; this file adds the element-wise statement for every
kernel family, on the small grid and at the reference's benchmark shape.

What the kernels are compared with.  The matrix-core kernels feed the matrix instructions with
u = B*x and g2 = dy*C rounded to the tensors' 16-bit type, as the reference's Triton kernel rounds Bx
before ``tl.dot`` and stores dy2 in the I/O type (fwd_kernels.py:703-721, bwd.py:391-400).  So that this
rounding of an operand is not mistaken for an error of the kernel, the oracle is given the same rounded
operands (the convolution is linear in u and in g2, and the gates are applied outside it):

    y2 = conv(u_r),  y = C * y2,  dC = dy * y2,  du = conv^T(g2_r),  dx = du * B,  dB = du * x,
    dh = sum over (b, t, c) of g2_r[t] u_r[t - lag]

The register-window and direct kernels keep u and g2 in fp32 and are compared with the oracle on the
unrounded products.  Beside the allclose bars, the fraction of outputs that equal the oracle's value rounded
once to the I/O type is checked (the kernels round once, after fp32 accumulation).
"""
import pytest
import torch

import oracle
from helpers import inputs
from savanna_amd import _lib
from savanna_amd.synthetic import make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# test_bwd_refactor.py:172-177 (fp16 takes the bf16 bars: same I/O width, more mantissa)
BARS = {torch.float32: dict(atol=1e-4, rtol=1e-4), torch.bfloat16: dict(atol=1e-3, rtol=1e-2),
        torch.float16: dict(atol=1e-3, rtol=1e-2)}
# dh has bars of its own there: atol = rtol = 1e-3 (test_bwd_refactor.py:83-87); a dh stored in a 16-bit type
# is rounded by up to 2^-9 of its value, so those types keep rtol 1e-2
BARS_DH = {torch.float32: dict(atol=1e-3, rtol=1e-3), torch.bfloat16: dict(atol=1e-3, rtol=1e-2),
           torch.float16: dict(atol=1e-3, rtol=1e-2)}

SHAPES = [
    (2, 32, 2, 32, 4),       # the reference's debug configs (tests/test_fwd_refactor.py:33-36)
    (2, 128, 2, 16, 128),
    (2, 300, 3, 16, 128),    # L not a multiple of the chunk
    (1, 1000, 5, 16, 100),
    (1, 513, 2, 48, 33),
    (2, 200, 4, 16, 7),
    (1, 77, 8, 4, 7),
    (1, 2049, 20, 16, 97),
    (3, 2500, 10, 16, 128),  # several runs per column, more than one round of workgroups
]


def algos_for(hl, dg):
    out = ["direct"]
    if hl <= 8 and dg % 4 == 0:
        out.append("window")
    if hl <= 128 and dg % 16 == 0:
        out.append("mfma")
    return out


def reference(x, B, C, h, dy, dtype, rounded_operands):
    """(y, dx, dB, dC, dh) in fp32 from the C oracle; with ``rounded_operands`` the convolutions take
    u = B*x and g2 = dy*C rounded to ``dtype`` (what the matrix cores are fed)."""
    xf, Bf, Cf, hf, dyf = (t.float() for t in (x, B, C, h, dy))
    if not rounded_operands or dtype == torch.float32:
        y = oracle.gcg_fwd_oracle(xf, Bf, Cf, hf)
        dx, dB, dC, dh = oracle.gcg_bwd_oracle(dyf, xf, Bf, Cf, hf)
        return y, dx, dB, dC, dh
    u = (Bf * xf).to(dtype).float()
    g2 = (dyf * Cf).to(dtype).float()
    one = torch.ones_like(u)
    _, y2, _ = oracle.gcg_fwd_oracle(u, one, one, hf, return_intermediates=True)
    du, _, _, dh = oracle.gcg_bwd_oracle(g2, u, one, one, hf)
    return Cf * y2, du * Bf, du * xf, dyf * y2, dh


def check(out, ref, dtype, what, min_equal=None):
    out = out.detach().float().cpu()
    assert torch.isfinite(out).all(), f"{what}: non-finite values"
    bars = (BARS_DH if what == "dh" else BARS)[dtype]
    bad = ~torch.isclose(out, ref, **bars)
    if bad.any():
        i = (out - ref).abs().mul(bad).argmax()
        raise AssertionError(f"{what}: {int(bad.sum())} of {out.numel()} elements outside atol {bars['atol']} / rtol "
                             f"{bars['rtol']}; worst: got {out.flatten()[i].item()!r}, reference {ref.flatten()[i].item()!r}")
    if min_equal is not None and dtype != torch.float32:
        equal = (out == ref.to(dtype).float()).float().mean().item()
        assert equal >= min_equal, f"{what}: only {equal:.4f} of the outputs equal the reference rounded once"
        return equal
    return None


def _cases():
    for shape in SHAPES:
        bs, L, g, dg, hl = shape
        for dtype in (torch.float32, torch.bfloat16, torch.float16):
            for algo in algos_for(hl, dg):
                yield pytest.param(*shape, dtype, algo, id=f"{bs}x{L}x{g}x{dg}-hl{hl}-{str(dtype)[6:]}-{algo}")


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype,algo", list(_cases()))
def test_allclose_small(gcg_lib, bs, L, g, dg, hl, dtype, algo):
    x, B, C, h, dy = inputs(bs, L, g, dg, hl, dtype, seed=11, dy_scale=0.1)   # dy = 0.1 * randn, test_bwd_refactor.py:98
    y_ref, dx_ref, dB_ref, dC_ref, dh_ref = reference(x, B, C, h, dy, dtype, rounded_operands=(algo == "mfma"))
    _, _, y = _lib.fwd(x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), algo=algo)
    dx, dB, dC, dh = _lib.bwd(dy.to(DEV), x.to(DEV), B.to(DEV), C.to(DEV), h.to(DEV), algo=algo)
    torch.cuda.synchronize()
    # y and dC are one product of an fp32 sum with a gate, rounded once: all but the ties of the fp32 accumulation
    # order land on the reference's rounded value; dx and dB go through the same and a second gate
    check(y, y_ref, dtype, "y", min_equal=0.995)
    check(dC, dC_ref, dtype, "dC", min_equal=0.995)
    check(dx, dx_ref, dtype, "dx", min_equal=0.995)
    check(dB, dB_ref, dtype, "dB", min_equal=0.995)
    check(dh, dh_ref, dtype, "dh")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("hl", [4, 32, 128])
def test_allclose_reference_grid(gcg_lib, hl, dtype):
    """The reference's benchmark shape (bs 2, L 8192, d 4096 in 256 groups; tests/test_fwd_refactor.py:22-31), every
    element of four filter groups against the oracle, forward and backward, with the family the library selects."""
    bs, L, g, dg = 2, 8192, 256, 16
    inp = make_inputs(bs, L, g, dg, hl, dtype, seed=3 * hl, device=DEV)
    inp["dy"] = (0.1 * inp["dy"].float()).to(dtype)
    _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
    dx, dB, dC, dh = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"])
    torch.cuda.synchronize()
    algo = _lib.select_algo(bs, L, g, dg, hl, dtype, True)
    idx = torch.tensor([0, 1, 127, 255], device=DEV)
    x, B, C, dyv = (inp[n].index_select(2, idx).cpu() for n in ("k", "q", "v", "dy"))
    h = inp["h"].index_select(0, idx).cpu()
    y_ref, dx_ref, dB_ref, dC_ref, dh_ref = reference(x, B, C, h, dyv, dtype, rounded_operands=(algo == "mfma"))
    fractions = {}
    for name, got, ref in (("y", y, y_ref), ("dC", dC, dC_ref), ("dx", dx, dx_ref), ("dB", dB, dB_ref)):
        fractions[name] = check(got.index_select(2, idx), ref, dtype, name, min_equal=0.995)
    check(dh.index_select(0, idx), dh_ref, dtype, "dh")
    print(f"hl={hl} {str(dtype)[6:]} ({algo}): fraction of outputs equal to the reference rounded once: {fractions}")
