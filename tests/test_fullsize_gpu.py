"""Parity at the benchmark shapes, where a full CPU pass is too slow: the oracle is run on
whole filter groups picked from the tensor (the operator is independent across groups, dh
included), closed forms are checked bit-exactly over the whole tensor, and the kernel
families are compared with each other on every element."""
import pytest
import torch

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib
from savanna_amd.synthetic import WORKLOADS, make_inputs, make_inputs_device

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def group_slice(t, groups):
    return t[:, :, groups].contiguous()


def check_groups_against_oracle(inp, outs, grads, groups, dtype):
    """inp: dict q,k,v,h,dy on the device; outs = y; grads = (dx, dB, dC, dh) or None."""
    idx = torch.tensor(groups, device=inp["q"].device)
    x, B, C = (inp[n].index_select(2, idx).float().cpu() for n in ("k", "q", "v"))
    h = inp["h"].index_select(0, idx).float().cpu()
    y_ref = oracle.gcg_fwd_oracle(x, B, C, h)
    assert_close(outs.index_select(2, idx), y_ref, TOL[dtype], "y")
    if grads is not None:
        dy = inp["dy"].index_select(2, idx).float().cpu()
        ref = oracle.gcg_bwd_oracle(dy, x, B, C, h)
        for got, want, n in zip(grads[:3], ref[:3], ("dx", "dB", "dC")):
            assert_close(got.index_select(2, idx), want, TOL[dtype], n)
        assert_close(grads[3].index_select(0, idx), ref[3], TOL_DH[dtype], "dh")


# ---- reference test grid (tests/test_fwd_refactor.py:22-31, tests/test_bwd_refactor.py) -------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("hl", [4, 32, 128])
@pytest.mark.parametrize("L", [1024, 8192])
def test_reference_grid_fwd_bwd(gcg_lib, L, hl, dtype):
    bs, g, dg = 2, 256, 16
    inp = make_inputs(bs, L, g, dg, hl, dtype, seed=L + hl, device=DEV)
    _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
    grads = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"])
    check_groups_against_oracle(inp, y, grads, [0, 1, 127, 255], dtype)


@pytest.mark.parametrize("g", [1, 4])
@pytest.mark.parametrize("hl", [4, 128])
def test_wide_groups(gcg_lib, g, hl):
    """Few filters shared by many channels (tests/test_two_pass_ref.py:14-21: d=4096, g in {1,2,4})."""
    bs, L, d = 1, 1024, 4096
    for dtype in (torch.float32, torch.bfloat16):
        inp = make_inputs(bs, L, g, d // g, hl, dtype, seed=g, device=DEV)
        _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
        grads = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"])
        check_groups_against_oracle(inp, y, grads, list(range(g)), dtype)


@pytest.mark.parametrize("bs,L", [(3, 8192), (5, 4000)], ids=["b3", "b5-ragged"])
def test_more_workgroups_than_fit_at_once(gcg_lib, bs, L):
    """Batch sizes whose columns do not divide the CU count: the matrix-core kernels then cut the sequence so
    that the launch takes several rounds of workgroups (768 and 1280 in the backward here).  Separate and
    interleaved operands, groups against the oracle and dx against the other kernel family on every element."""
    g, dg, hl, dtype = 256, 16, 128, torch.bfloat16
    inp = make_inputs(bs, L, g, dg, hl, dtype, seed=bs, device=DEV)
    _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
    grads = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"])
    check_groups_against_oracle(inp, y, grads, [0, 77, 255], dtype)
    feat = torch.stack([inp["v"], inp["q"], inp["k"]], dim=-1).contiguous()
    y_i = _lib.fwd_interleaved(feat, inp["h"])
    dfeat, dh_i = _lib.bwd_interleaved(inp["dy"], feat, inp["h"])
    assert torch.equal(y_i, y)
    assert torch.equal(dfeat[..., 2], grads[0]) and torch.equal(dfeat[..., 1], grads[1]) and torch.equal(dfeat[..., 0], grads[2])
    assert_close(dh_i, grads[3], TOL_DH[dtype], "dh interleaved")
    direct = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"], algo="direct")
    assert_close(grads[0], direct[0], TOL[dtype], "dx, matrix cores against vector ALUs")


# ---- the benchmark configurations ------------------------------------------------------------------
def test_mr_7b_delta_filter_bit_exact(gcg_lib):
    """h = e_{hl-1-s}: y[t] = C[t] * bf16(B*x)[t-s], every bit, at B=2 L=8192 D=4096."""
    wl = WORKLOADS["mr_fwd_7b"]
    inp = make_inputs(wl.bs, wl.L, wl.g, wl.dg, 128, wl.dtype, device=DEV, with_dy=False)
    u = (inp["q"].float() * inp["k"].float()).to(torch.bfloat16)
    for s in (0, 37, 127):
        h = torch.zeros(wl.g, 1, 128, dtype=wl.dtype, device=DEV)
        h[:, 0, 127 - s] = 1.0
        _, y2, y = _lib.fwd(inp["k"], inp["q"], inp["v"], h, return_y2=True, algo="mfma")
        shifted = torch.zeros_like(u)
        shifted[:, s:] = u[:, : wl.L - s]
        assert torch.equal(y2, shifted), f"y2, shift {s}"
        assert torch.equal(y, (inp["v"].float() * shifted.float()).to(torch.bfloat16)), f"y, shift {s}"


def test_mr_7b_fwd_bwd(gcg_lib):
    wl = WORKLOADS["mr_fwdbwd_7b"]
    inp = make_inputs(wl.bs, wl.L, wl.g, wl.dg, 128, wl.dtype, device=DEV)
    _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
    grads = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"])
    check_groups_against_oracle(inp, y, grads, [0, 3, 64, 200, 255], wl.dtype)
    # every element, against the vector-ALU family (independent code, fp32 u)
    _, _, y_d = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"], algo="direct")
    grads_d = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"], algo="direct")
    assert_close(y, y_d.float(), 1e-2, "y mfma vs direct")
    for a, b_, n in zip(grads, grads_d, ("dx", "dB", "dC", "dh")):
        assert_close(a, b_.float(), 1e-2, f"{n} mfma vs direct")
    # bitwise reproducible
    again = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"])
    for a, b_ in zip(grads, again):
        assert torch.equal(a, b_)


def test_se_fp32_config(gcg_lib):
    wl = WORKLOADS["se_fwd_fp32"]
    inp = make_inputs(wl.bs, wl.L, wl.g, wl.dg, 7, wl.dtype, device=DEV)
    _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
    ref = oracle.gcg_fwd_oracle(inp["k"].cpu(), inp["q"].cpu(), inp["v"].cpu(), inp["h"].cpu())
    assert_close(y, ref, 1e-5, "y")
    # the library formulation in fp32 on the CPU agrees to the reference's own tolerance
    torch.testing.assert_close(y.cpu(), oracle.gcg_fwd_ref_torch(inp["k"].cpu(), inp["q"].cpu(), inp["v"].cpu(),
                                                                 inp["h"].cpu()), atol=1e-4, rtol=1e-4)


def test_40b_pair_fwd_bwd(gcg_lib):
    """SE (hl 7) then MR (hl 128) on the same activations, B=1 L=32768 D=8192."""
    wl = WORKLOADS["se_mr_fwdbwd_40b"]
    for hl in wl.filters:
        inp = make_inputs(wl.bs, wl.L, wl.g, wl.dg, hl, wl.dtype, device=DEV)
        _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
        grads = _lib.bwd(inp["dy"], inp["k"], inp["q"], inp["v"], inp["h"])
        check_groups_against_oracle(inp, y, grads, [0, 257, 511], wl.dtype)
        del inp, y, grads
        torch.cuda.empty_cache()


def test_long_context_64bit_offsets(gcg_lib):
    """B=1 L=2^20 D=4096: 2^32 elements per tensor.  A shift filter is checked on every
    element (an offset that wrapped at 2^31 or 2^32 would move data), and the decayed filter
    against the oracle on windows at the start, across flat offsets 2^31 and 2^32, and at the end."""
    wl = WORKLOADS["mr_fwd_1m"]
    inp = make_inputs_device(wl.bs, wl.L, wl.g, wl.dg, 128, wl.dtype, DEV, with_dy=False)
    L, d = wl.L, wl.d
    h = torch.zeros(wl.g, 1, 128, dtype=wl.dtype, device=DEV)
    h[:, 0, 126] = 1.0                                        # one-row shift
    _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], h)
    rows = 65536
    for t0 in range(0, L, rows):
        t1 = min(L, t0 + rows)
        lo = max(t0 - 1, 0)
        u = (inp["q"][:, lo:t1].float() * inp["k"][:, lo:t1].float()).to(torch.bfloat16)
        if t0 == 0:
            u = torch.cat([torch.zeros_like(u[:, :1]), u], dim=1)
        want = (inp["v"][:, t0:t1].float() * u[:, : t1 - t0].float()).to(torch.bfloat16)
        assert torch.equal(y[:, t0:t1], want), f"rows {t0}..{t1}"
    del y
    _, _, y = _lib.fwd(inp["k"], inp["q"], inp["v"], inp["h"])
    groups = [0, 131, 255]
    idx = torch.tensor(groups, device=DEV)
    row31, row32 = (1 << 31) // d, L                          # rows holding flat offsets 2^31 and 2^32 (= end)
    for t0, t1 in [(0, 300), (row31 - 200, row31 + 200), (row32 - 300, row32)]:
        lo = max(0, t0 - 127)
        x, B, C = (inp[n][:, lo:t1].index_select(2, idx).float().cpu() for n in ("k", "q", "v"))
        ref = oracle.gcg_fwd_oracle(x, B, C, inp["h"].index_select(0, idx).float().cpu())
        assert_close(y[:, t0:t1].index_select(2, idx), ref[:, t0 - lo:], TOL[wl.dtype], f"y rows {t0}..{t1}")


@pytest.mark.parametrize("layout", ["separate", "interleaved", "direct"])
def test_short_filter_64bit_offsets(gcg_lib, layout):
    """The register-window kernels (Hyena-SE, 7 taps) on B=1, L=2^19, D=4096 in bf16: 2^31 elements per tensor,
    3 * 2^31 in the interleaved one.  A filter that delays by two rows makes every output a product of input
    elements (these kernels keep B*x and dy*C in fp32), compared exactly on the whole tensors."""
    bs, L, g, dg, hl, s_ = 1, 1 << 19, 256, 16, 7, 2
    dt = torch.bfloat16
    gen = torch.Generator(device=DEV)
    feat = torch.empty(bs, L, g, dg, 3, dtype=dt, device=DEV)
    dy = torch.empty(bs, L, g, dg, dtype=dt, device=DEV)
    for k, t0 in enumerate(range(0, L, 1 << 16)):
        gen.manual_seed(700 + k)
        feat[:, t0:t0 + (1 << 16)].normal_(generator=gen)
        dy[:, t0:t0 + (1 << 16)].normal_(generator=gen)
    h = torch.zeros(g, 1, hl, dtype=dt, device=DEV)
    h[:, 0, hl - 1 - s_] = 1.0
    C, B, x = feat.unbind(-1)
    if layout != "interleaved":
        algo = "window" if layout == "separate" else "direct"      # direct: the general fallback kernels
        x, B, C = x.contiguous(), B.contiguous(), C.contiguous()
        _, _, y = _lib.fwd(x, B, C, h, algo=algo)
        dx, dB, dC, dh = _lib.bwd(dy, x, B, C, h, algo=algo)
    else:
        y = _lib.fwd_interleaved(feat, h)
        dfeat, dh = _lib.bwd_interleaved(dy, feat, h)
        dC, dB, dx = dfeat.unbind(-1)
    torch.cuda.synchronize()
    assert torch.isfinite(dh.float()).all()
    u = x.float() * B.float()
    want = torch.zeros_like(dy)
    want[:, s_:] = (C[:, s_:].float() * u[:, :-s_]).to(dt)
    assert torch.equal(y, want), "y"
    want.zero_()
    want[:, s_:] = (dy[:, s_:].float() * u[:, :-s_]).to(dt)
    assert torch.equal(dC, want), "dC"
    del u
    g2 = dy.float() * C.float()
    want.zero_()
    want[:, :-s_] = (g2[:, s_:] * x[:, :-s_].float()).to(dt)
    assert torch.equal(dB, want), "dB"
    want.zero_()
    want[:, :-s_] = (g2[:, s_:] * B[:, :-s_].float()).to(dt)
    assert torch.equal(dx, want), "dx"
