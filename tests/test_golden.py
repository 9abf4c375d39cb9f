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
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
DT = {"torch.float32": torch.float32, "torch.bfloat16": torch.bfloat16, "torch.float16": torch.float16}


def load(path):
    z = np.load(path, allow_pickle=False)
    t = {k: torch.from_numpy(z[k]) for k in z.files if k != "dtype"}
    return t, DT[str(z["dtype"])]


def test_fixtures_present():
    assert len(FILES) >= 4


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
