"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU: the C oracle reproduces them.  GPU: every kernel family that takes the shape
reproduces them through the C ABI."""
import glob
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib

HERE = os.path.dirname(os.path.abspath(__file__))
ALL = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
FEAT = [f for f in ALL if os.path.basename(f).startswith("featurizer")]           # the ungated featurizer conv
MIXER = [f for f in ALL if os.path.basename(f).startswith("mixer_se")]            # featurizer + Hyena-SE operator
MIXER_MR = [f for f in ALL if os.path.basename(f).startswith("mixer_mr")]         # featurizer + Hyena-MR operator, decayed filter
FILES = [f for f in ALL if f not in FEAT and f not in MIXER and f not in MIXER_MR]   # the gated operator
DT = {"torch.float32": torch.float32, "torch.bfloat16": torch.bfloat16, "torch.float16": torch.float16}


def load(path):
    z = np.load(path, allow_pickle=False)
    t = {k: torch.from_numpy(z[k]) for k in z.files if k != "dtype"}     # (0-d arrays, e.g. hl, become 0-d tensors)
    return t, DT[str(z["dtype"])]


def test_fixtures_present():
    assert len(FILES) >= 4 and len(FEAT) >= 1 and len(MIXER) >= 1 and len(MIXER_MR) >= 1


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_c_oracle_reproduces_golden(path):
    t, _ = load(path)
    bx, y2, y = oracle.gcg_fwd_oracle(t["x"], t["B"], t["C"], t["h"], return_intermediates=True)
    for got, name in ((bx, "bx"), (y2, "y2"), (y, "y")):
        assert_close(got, t[name], 2e-6, name)
    for got, name in zip(oracle.gcg_bwd_oracle(t["dy"], t["x"], t["B"], t["C"], t["h"]), ("dx", "dB", "dC", "dh")):
        assert_close(got, t[name], 2e-6, name)


@pytest.mark.gpu
@pytest.mark.parametrize("algo", ["auto", "direct", "window", "mfma"])
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_hip_reproduces_golden(gcg_lib, path, algo):
    t, dtype = load(path)
    bs, L, g, dg = t["x"].shape
    hl = t["h"].shape[-1]
    if algo == "window" and hl > 8:
        pytest.skip("register-window family takes hl <= 8")
    if algo == "mfma" and (hl > 128 or dg % 16):
        pytest.skip("matrix-core family takes hl <= 128 and 16-channel groups")
    dev = {k: v.to(dtype).to("cuda:0") for k, v in t.items()}
    bx, y2, y = _lib.fwd(dev["x"], dev["B"], dev["C"], dev["h"], return_bx=True, return_y2=True, algo=algo)
    for got, name in ((bx, "bx"), (y2, "y2"), (y, "y")):
        assert_close(got, t[name], TOL[dtype], f"{name} [{algo}]")
    grads = _lib.bwd(dev["dy"], dev["x"], dev["B"], dev["C"], dev["h"], algo=algo)
    for got, name in zip(grads, ("dx", "dB", "dC", "dh")):
        assert_close(got, t[name], TOL_DH[dtype] if name == "dh" else TOL[dtype], f"{name} [{algo}]")


@pytest.mark.gpu
@pytest.mark.parametrize("algo", ["auto", "direct"])
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_hip_interleaved_reproduces_golden(gcg_lib, path, algo):
    """The same vectors through the interleaved entry points: x, B, C packed into one
    (bs, L, g, dg, 3) tensor, the three input gradients read back from one."""
    t, dtype = load(path)
    dev = {k: v.to(dtype).to("cuda:0") for k, v in t.items()}
    feat = torch.stack([dev["C"], dev["B"], dev["x"]], dim=-1).contiguous()
    y = _lib.fwd_interleaved(feat, dev["h"], algo=algo)
    assert_close(y, t["y"], TOL[dtype], f"y [{algo}]")
    dfeat, dh = _lib.bwd_interleaved(dev["dy"], feat, dev["h"], algo=algo)
    for i, name in enumerate(("dC", "dB", "dx")):
        assert_close(dfeat[..., i], t[name], TOL[dtype], f"{name} [{algo}]")
    assert_close(dh, t["dh"], TOL_DH[dtype], f"dh [{algo}]")


@pytest.mark.parametrize("path", FEAT, ids=[os.path.basename(f) for f in FEAT])
def test_c_oracle_reproduces_featurizer_golden(path):
    """The featurizer is the gated operator with both gates at one."""
    t, _ = load(path)
    one = torch.ones_like(t["x"])
    assert_close(oracle.gcg_fwd_oracle(t["x"], one, one, t["w"]), t["y"], 2e-6, "y")
    dx, _, _, dw = oracle.gcg_bwd_oracle(t["dy"], t["x"], one, one, t["w"])
    assert_close(dx, t["dx"], 2e-6, "dx")
    assert_close(dw, t["dw"], 2e-6, "dw")


@pytest.mark.gpu
@pytest.mark.parametrize("path", FEAT, ids=[os.path.basename(f) for f in FEAT])
def test_hip_featurizer_reproduces_golden(gcg_lib, path):
    t, dtype = load(path)
    dev = {k: v.to(dtype).to("cuda:0") for k, v in t.items()}
    assert_close(_lib.dwconv_fwd(dev["x"], dev["w"]), t["y"], TOL[dtype], "y")
    dx, dw = _lib.dwconv_bwd(dev["dy"], dev["x"], dev["w"])
    assert_close(dx, t["dx"], TOL[dtype], "dx")
    assert_close(dw, t["dw"], TOL_DH[dtype], "dw")


def _chain_with_oracle(t, dtype):
    """The two C-oracle applications that make up the chain, with the tensors that the chain holds
    in `dtype` rounded to it."""
    bs, L, g, dg, _ = t["raw"].shape
    r4 = t["raw"].reshape(bs, L, 3 * g * dg, 1)
    one = torch.ones_like(r4)
    f = oracle.gcg_fwd_oracle(r4, one, one, t["wf"]).to(dtype).float().reshape(bs, L, g, dg, 3)
    C, B, x = (f[..., i].contiguous() for i in range(3))
    y = oracle.gcg_fwd_oracle(x, B, C, t["h"])
    dx, dB, dC, dh = oracle.gcg_bwd_oracle(t["dy"], x, B, C, t["h"])
    df = torch.stack([dC, dB, dx], dim=-1).to(dtype).float().reshape(bs, L, 3 * g * dg, 1)
    draw, _, _, dwf = oracle.gcg_bwd_oracle(df, r4, one, one, t["wf"])
    return y, draw.reshape(t["raw"].shape), dwf, dh


@pytest.mark.parametrize("path", MIXER, ids=[os.path.basename(f) for f in MIXER])
def test_c_oracle_chain_reproduces_mixer_golden(path):
    """The oracle applied twice (featurizer, then operator) against the reference's chain written
    with F.conv1d, rearrange / unbind and autograd in float64.  Where the float64 value of the
    featurized tensor sits next to a bf16 rounding boundary the fp32 oracle may round it the other
    way (one bf16 ulp in that element), hence the tolerance of a rounded stage."""
    t, dtype = load(path)
    y, draw, dwf, dh = _chain_with_oracle(t, dtype)
    assert_close(y, t["y"], TOL[dtype], "y")
    assert_close(draw, t["draw"], TOL[dtype], "d raw")
    assert_close(dwf, t["dwf"], TOL_DH[dtype], "dwf")
    assert_close(dh, t["dh"], TOL_DH[dtype], "dh")


@pytest.mark.gpu
@pytest.mark.parametrize("path", MIXER, ids=[os.path.basename(f) for f in MIXER])
def test_hip_mixer_reproduces_golden(gcg_lib, path):
    t, dtype = load(path)
    dev = {k: v.to(dtype).to("cuda:0") for k, v in t.items()}
    y = _lib.mixer_se_fwd(dev["raw"], dev["wf"], dev["h"])
    draw, dwf, dh = _lib.mixer_se_bwd(dev["dy"], dev["raw"], dev["wf"], dev["h"])
    assert_close(y, t["y"], TOL[dtype], "y")
    assert_close(draw, t["draw"], 2 * TOL[dtype], "d raw")
    assert_close(dwf, t["dwf"], 2 * TOL_DH[dtype], "dwf")
    assert_close(dh, t["dh"], TOL_DH[dtype], "dh")


def _dw_from_dh(dh, t, dtype):
    """Gradient of the filter parameter from the gradient of the filter: through the cast to the tensors' type
    (stored in that type) and the product with the decay, zero beyond the taps in use."""
    hl = int(t["hl"])
    dw = torch.zeros_like(t["w"])
    dw[:, :hl] = dh[:, 0].to(dtype).float() * t["decay"][:, :hl]
    return dw


@pytest.mark.parametrize("path", MIXER_MR, ids=[os.path.basename(f) for f in MIXER_MR])
def test_c_oracle_chain_reproduces_mixer_mr_golden(path):
    """The Hyena-MR layer's chain written with F.conv1d, rearrange / unbind and autograd in float64 (decayed filter,
    featurizer, operator) against the oracle applied twice on the fixture's filter, and the filter as
    (w * decay)[:, :hl] rounded to the tensors' type."""
    t, dtype = load(path)
    hl = int(t["hl"])
    h = (t["w"] * t["decay"])[:, :hl].to(dtype).float()[:, None]
    assert torch.equal(h, t["h"])
    y, draw, dwf, dh = _chain_with_oracle(t, dtype)
    assert_close(y, t["y"], TOL[dtype], "y")
    assert_close(draw, t["draw"], TOL[dtype], "d raw")
    assert_close(dwf, t["dwf"], TOL_DH[dtype], "dwf")
    assert_close(_dw_from_dh(dh, t, dtype), t["dw"], TOL_DH[dtype], "dw")


@pytest.mark.gpu
@pytest.mark.parametrize("layout", ["interleaved", "planar"])
@pytest.mark.parametrize("path", MIXER_MR, ids=[os.path.basename(f) for f in MIXER_MR])
def test_hip_mixer_mr_reproduces_golden(gcg_lib, path, layout):
    """gcg_mixer_mr_fwd_decay / _bwd_decay (filter formed in the kernels) and, on the planar layout of the same
    values, gcg_mixer_mr_fwd_planar / _bwd_planar with the fixture's filter."""
    t, dtype = load(path)
    hl = int(t["hl"])
    dev = {k: (v.to(dtype) if k not in ("w", "decay", "hl") else v).to("cuda:0") for k, v in t.items()}
    if layout == "interleaved":
        y = _lib.mixer_mr_fwd_decay(dev["raw"], dev["wf"], dev["w"], dev["decay"], hl, dtype)
        draw, dwf, dw = _lib.mixer_mr_bwd_decay(dev["dy"], dev["raw"], dev["wf"], dev["w"], dev["decay"], hl, dtype)
    else:
        bs, L, g, dg, _ = t["raw"].shape
        d = g * dg
        raw_pl = dev["raw"].permute(0, 1, 4, 2, 3).contiguous()
        wf_pl = dev["wf"].view(d, 3, 1, -1).permute(1, 0, 2, 3).reshape(3 * d, 1, -1).contiguous()
        y = _lib.mixer_mr_fwd(raw_pl, wf_pl, dev["h"], planar=True)
        draw_pl, dwf_pl, dh = _lib.mixer_mr_bwd(dev["dy"], raw_pl, wf_pl, dev["h"], planar=True)
        draw = draw_pl.permute(0, 1, 3, 4, 2)
        dwf = dwf_pl.view(3, d, 1, -1).permute(1, 0, 2, 3).reshape(3 * d, 1, -1)
        dw = _dw_from_dh(dh.float().cpu(), t, dtype)
    assert_close(y, t["y"], TOL[dtype], "y")
    assert_close(draw, t["draw"], 2 * TOL[dtype], "d raw")
    assert_close(dwf, t["dwf"], 2 * TOL_DH[dtype], "dwf")
    assert_close(dw, t["dw"], TOL_DH[dtype], "dw")
