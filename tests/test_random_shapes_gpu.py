"""Seeded random shapes through every entry point with the kernel family chosen by the library,
against the CPU oracle: ragged lengths, odd group widths, filters from one tap to beyond the
matrix-core limit -- the combinations the hand-picked lists do not enumerate."""
import random

import pytest
import torch

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _shapes(n, seed, dgs, max_hl):
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        bs, L = rnd.randint(1, 3), rnd.choice([1, 2, 7, 31, 32, 33, 64, 127, 129, 200, 511, 700])
        g, dg = rnd.randint(1, 6), rnd.choice(dgs)
        hl = rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 16, 31, 32, 33, 64, 100, 128, 129, 140])
        out.append((bs, L, g, dg, min(hl, max_hl), DTYPES[rnd.randrange(3)]))
    return out


def _id(p):
    bs, L, g, dg, hl, dtype = p
    return f"{bs}x{L}x{g}x{dg}-hl{hl}-{str(dtype)[6:]}"


def _inputs(bs, L, g, dg, hl, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(3))
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype)
    return x, B, C, dy, h


GATED = _shapes(48, 1, [1, 2, 4, 8, 16, 20, 32, 48], 140)


@pytest.mark.parametrize("p", GATED, ids=[_id(p) for p in GATED])
def test_gated_operator_random(gcg_lib, p):
    bs, L, g, dg, hl, dtype = p
    x, B, C, dy, h = _inputs(bs, L, g, dg, hl, dtype, seed=hash(p[:5]) & 0xffff)
    y_ref = oracle.gcg_fwd_oracle(x.float(), B.float(), C.float(), h.float())
    ref = oracle.gcg_bwd_oracle(dy.float(), x.float(), B.float(), C.float(), h.float())
    xd, Bd, Cd, dyd, hd = (t.to(DEV) for t in (x, B, C, dy, h))
    _, _, y = _lib.fwd(xd, Bd, Cd, hd)
    got = _lib.bwd(dyd, xd, Bd, Cd, hd)
    feat = torch.stack([Cd, Bd, xd], dim=-1).contiguous()
    y_i = _lib.fwd_interleaved(feat, hd)
    dfeat, dh_i = _lib.bwd_interleaved(dyd, feat, hd)
    torch.cuda.synchronize()
    few = bs * L * dg < 256          # a tap summed from a handful of rounded products can cancel
    assert_close(y, y_ref, TOL[dtype], "y")
    assert_close(y_i, y_ref, TOL[dtype], "y interleaved")
    for o, oi, r, n in zip(got[:3], (dfeat[..., 2], dfeat[..., 1], dfeat[..., 0]), ref[:3], ("dx", "dB", "dC")):
        assert_close(o, r, TOL[dtype], n)
        assert_close(oi, r, TOL[dtype], n + " interleaved")
    if not few or dtype == torch.float32:
        assert_close(got[3], ref[3], TOL_DH[dtype], "dh")
        assert_close(dh_i, ref[3], TOL_DH[dtype], "dh interleaved")


FEAT = _shapes(24, 2, [1, 4, 8, 16], 8)


@pytest.mark.parametrize("p", FEAT, ids=[_id(p) for p in FEAT])
def test_featurizer_random(gcg_lib, p):
    bs, L, g, dg, hl, dtype = p
    if (g * dg) % 4:
        g *= 4                        # the featurizer kernels take channel counts that are multiples of 4
    x, _, _, dy, w = _inputs(bs, L, g, dg, hl, dtype, seed=hash(p[:5]) & 0xffff)
    one = torch.ones(bs, L, g, dg)
    y_ref = oracle.gcg_fwd_oracle(x.float(), one, one, w.float())
    dx_ref, _, _, dw_ref = oracle.gcg_bwd_oracle(dy.float(), x.float(), one, one, w.float())
    y = _lib.dwconv_fwd(x.to(DEV), w.to(DEV))
    dx, dw = _lib.dwconv_bwd(dy.to(DEV), x.to(DEV), w.to(DEV))
    torch.cuda.synchronize()
    assert_close(y, y_ref, TOL[dtype], "y")
    assert_close(dx, dx_ref, TOL[dtype], "dx")
    if bs * L * dg >= 256 or dtype == torch.float32:
        assert_close(dw, dw_ref, TOL_DH[dtype], "dw")


MIX = _shapes(24, 3, [2, 4, 6, 8, 16, 20, 32], 8)


@pytest.mark.parametrize("p", MIX, ids=[_id(p) for p in MIX])
def test_fused_mixer_random(gcg_lib, p):
    from test_mixer_se_gpu import data, oracle_chain

    bs, L, g, dg, hl, dtype = p
    kf = 1 + (hash(p[:5]) % 4)
    raw, dy, wf, h = data(bs, L, g, dg, hl, kf, dtype, seed=hash(p[:5]) & 0xffff)
    ref = oracle_chain(raw, dy, wf, h, dtype)
    rawd, dyd, wfd, hd = (t.to(DEV) for t in (raw, dy, wf, h))
    y = _lib.mixer_se_fwd(rawd, wfd, hd)
    draw, dwf, dh = _lib.mixer_se_bwd(dyd, rawd, wfd, hd)
    torch.cuda.synchronize()
    assert_close(y, ref[0], TOL[dtype], "y")
    assert_close(draw, ref[1], 2 * TOL[dtype], "d raw")
    if bs * L * dg >= 256 or dtype == torch.float32:
        assert_close(dwf, ref[2], 2 * TOL_DH[dtype], "dwf")
        assert_close(dh, ref[3], TOL_DH[dtype], "dh")


def _mr_shapes(n, seed):
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        bs, L = rnd.randint(1, 3), rnd.choice([9, 31, 32, 33, 64, 127, 129, 200, 511, 700, 1500, 2600])
        g, dg = rnd.randint(1, 9), rnd.choice([16, 16, 32, 48, 64])
        hl = min(L, rnd.choice([9, 16, 31, 32, 33, 64, 65, 97, 100, 127, 128]))
        types = [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16), (torch.float32, torch.float32),
                 (torch.bfloat16, torch.float32)]
        out.append((bs, L, g, dg, max(hl, 9), rnd.randint(1, 3)) + types[rnd.randrange(4)])
    return out


MIX_MR = _mr_shapes(64, 4)


@pytest.mark.parametrize("p", MIX_MR, ids=["x".join(map(str, p[:6])) + f"-{str(p[6])[6:]}-{str(p[7])[6:]}" for p in MIX_MR])
def test_fused_mr_mixer_random(gcg_lib, p):
    """gcg_mixer_mr_* on random shapes against the chain of featurizer and interleaved operator (bit for bit at
    bf16 and in fp32-inside arithmetic), the planar layout against the interleaved one, and the filter formed in
    the kernels against the explicit one."""
    from test_mixer_mr_gpu import chain, make

    bs, L, g, dg, hl, kf, dtype, filt = p
    raw, wf, h, dy = (t.to(DEV) for t in make(bs, L, g, dg, hl, kf, dtype, filt, seed=hash(p[:6]) & 0xffff))
    y = _lib.mixer_mr_fwd(raw, wf, h)
    draw, dwf, dh = _lib.mixer_mr_bwd(dy, raw, wf, h)
    y_c, draw_c, dwf_c, dh_c = chain(raw, wf, h, dy)
    torch.cuda.synchronize()
    if dtype == torch.float16 and filt == dtype:
        # the featurizer's three taps are grouped differently in different kernels at f16: last-place differences
        assert_close(y, y_c, TOL[dtype], "y")
        assert_close(draw, draw_c, TOL[dtype], "d raw")
    else:
        assert torch.equal(y, y_c), "y"
        assert torch.equal(draw, draw_c), "d raw"
    if bs * L * dg >= 256 or dtype == torch.float32:
        assert_close(dh, dh_c, TOL_DH[filt], "dh")
        assert_close(dwf, dwf_c, 2 * TOL_DH[dtype], "dwf")
    # the filter formed in the kernels: w * decay cut to hl taps
    lc = max(hl, 128)
    gen = torch.Generator().manual_seed(hash(p[:6]) & 0xfff)
    w = (torch.randn(g, lc, generator=gen) / lc ** 0.5).to(DEV)
    decay = torch.exp(-torch.logspace(0, 2, g)[:, None] * torch.linspace(0, 1, lc)[None]).to(DEV)
    hd = _lib.filter_decay_fwd(w, decay, hl, filt)
    y_d = _lib.mixer_mr_fwd_decay(raw, wf, w, decay, hl, filt)
    draw_d, dwf_d, dw = _lib.mixer_mr_bwd_decay(dy, raw, wf, w, decay, hl, filt)
    draw_e, dwf_e, dh_e = _lib.mixer_mr_bwd(dy, raw, wf, hd)
    assert torch.equal(y_d, _lib.mixer_mr_fwd(raw, wf, hd)), "y, filter in the kernel"
    assert torch.equal(draw_d, draw_e) and torch.equal(dwf_d, dwf_e), "d raw / dwf, filter in the kernel"
    assert torch.equal(dw, _lib.filter_decay_bwd(dh_e, decay)), "dw"
    if dtype == filt and dtype != torch.float32:
        d = g * dg
        raw_pl = raw.permute(0, 1, 4, 2, 3).contiguous()
        wf_pl = wf.view(d, 3, 1, kf).permute(1, 0, 2, 3).reshape(3 * d, 1, kf).contiguous()
        y_p = _lib.mixer_mr_fwd(raw_pl, wf_pl, h, planar=True)
        draw_p, dwf_p, dh_p = _lib.mixer_mr_bwd(dy, raw_pl, wf_pl, h, planar=True)
        torch.cuda.synchronize()
        assert torch.equal(y_p, y) and torch.equal(draw_p, draw.permute(0, 1, 4, 2, 3)) and torch.equal(dh_p, dh), "planar"
        assert torch.equal(dwf_p.view(3, d, 1, kf), dwf.view(d, 3, 1, kf).permute(1, 0, 2, 3)), "planar dwf"
