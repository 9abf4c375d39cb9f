"""Pins the CPU oracle (oracle/) before anything is compared with it.

Every check below is chosen so that a plausible mistake -- a flipped filter, an
off-by-one in the causal pad, a dropped carry term, blocked vs striped filter groups,
a wrong sign or index in a gradient -- fails at least one of them.  None of them
restates the oracle's own formula.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import gcg_ref

torch.manual_seed(0)


def rand(bs, L, g, dg, hl, dtype=torch.float64, seed=0):
    gen = torch.Generator().manual_seed(seed)
    x, B, C, dy = (torch.randn(bs, L, g, dg, generator=gen, dtype=dtype) for _ in range(4))
    h = torch.randn(g, 1, hl, generator=gen, dtype=dtype)
    return x, B, C, h, dy


SHAPES = [(1, 5, 1, 1, 1), (2, 17, 3, 2, 4), (1, 40, 2, 4, 7), (2, 33, 2, 3, 40), (1, 300, 2, 16, 128)]


# ---- the library routine the reference calls --------------------------------------------
@pytest.mark.parametrize("bs,L,g,dg,hl", SHAPES)
def test_c_oracle_matches_conv1d(bs, L, g, dg, hl):
    """Independent phrasing of ref_fwd.py:109-129: pad both sides, trim the tail,
    per-channel loop over F.conv1d with groups=1."""
    x, B, C, h, _ = rand(bs, L, g, dg, hl)
    u = (B * x).reshape(bs, L, g * dg)
    y2 = torch.empty_like(u)
    for c in range(g * dg):
        w = h[c // dg].reshape(1, 1, hl)
        full = F.conv1d(u[:, :, c].unsqueeze(1), w, padding=hl - 1)
        y2[:, :, c] = full[:, 0, :L]
    want = C * y2.reshape(bs, L, g, dg)
    got = oracle.gcg_fwd_oracle(x, B, C, h)
    torch.testing.assert_close(got.double(), want, atol=2e-6, rtol=2e-6)
    torch.testing.assert_close(oracle.gcg_fwd_ref_torch(x, B, C, h), want, atol=1e-12, rtol=1e-12)


@pytest.mark.parametrize("bs,L,g,dg,hl", SHAPES[:4])
def test_brute_force(bs, L, g, dg, hl):
    x, B, C, h, _ = rand(bs, L, g, dg, hl, dtype=torch.float32)
    want = oracle.brute_force_fwd(x, B, C, h)
    torch.testing.assert_close(oracle.gcg_fwd_oracle(x, B, C, h).double(), want, atol=1e-5, rtol=1e-5)


# ---- closed forms ---------------------------------------------------------------------
@pytest.mark.parametrize("hl,s", [(1, 0), (7, 0), (7, 3), (7, 6), (128, 0), (128, 127), (128, 50)])
def test_delta_filter_is_a_shift(hl, s):
    """h = e_{hl-1-s}  =>  y[t] = C[t] * u[t-s]; s = 0 is the identity tap hl-1."""
    bs, L, g, dg = 2, 200, 2, 4
    x, B, C, _, _ = rand(bs, L, g, dg, hl, dtype=torch.float32)
    h = torch.zeros(g, 1, hl)
    h[:, 0, hl - 1 - s] = 1.0
    u = B * x
    want = torch.zeros_like(u)
    want[:, s:] = u[:, : L - s]
    want = C * want
    for f in (oracle.gcg_fwd_oracle, oracle.gcg_fwd_ref_torch):
        torch.testing.assert_close(f(x, B, C, h), want, atol=1e-6, rtol=1e-6)


def test_all_ones_gives_running_filter_sum():
    """x = B = C = 1  =>  y[t] = sum of the last min(t+1, hl) taps."""
    bs, L, g, dg, hl = 1, 50, 3, 2, 9
    h = torch.randn(g, 1, hl, dtype=torch.float64)
    one = torch.ones(bs, L, g, dg, dtype=torch.float64)
    got = oracle.gcg_fwd_oracle(one, one, one, h).double()
    csum = torch.cumsum(h[:, 0].flip(-1), dim=-1)           # csum[j] = h[hl-1] + ... + h[hl-1-j]
    for t in range(L):
        want = csum[:, min(t, hl - 1)]
        torch.testing.assert_close(got[0, t, :, 0], want, atol=1e-6, rtol=1e-6)
        torch.testing.assert_close(got[0, t, :, 1], want, atol=1e-6, rtol=1e-6)


def test_filters_are_blocked_per_group_not_striped():
    """Channel c uses filter c // dg (repeat_interleave, ref_fwd.py:115), not c % g."""
    bs, L, g, dg, hl = 1, 12, 3, 2, 2
    one = torch.ones(bs, L, g, dg)
    h = torch.zeros(g, 1, hl)
    h[:, 0, hl - 1] = torch.tensor([1.0, 2.0, 3.0])
    y = oracle.gcg_fwd_oracle(one, one, one, h)
    assert y[0, 5].flatten().tolist() == [1.0, 1.0, 2.0, 2.0, 3.0, 3.0]


def test_causality_and_support():
    """Perturbing u at t0 changes y only on [t0, t0+hl-1]."""
    bs, L, g, dg, hl, t0 = 1, 64, 1, 2, 9, 20
    x, B, C, h, _ = rand(bs, L, g, dg, hl, dtype=torch.float32)
    y0 = oracle.gcg_fwd_oracle(x, B, C, h)
    x2 = x.clone()
    x2[0, t0] += 1.0
    diff = (oracle.gcg_fwd_oracle(x2, B, C, h) - y0).abs().amax(dim=(0, 2, 3))
    changed = torch.nonzero(diff > 0).flatten().tolist()
    assert changed[0] == t0 and changed[-1] == t0 + hl - 1 and len(changed) == hl


def test_linearity_and_gate_symmetry():
    x, B, C, h, _ = rand(2, 30, 2, 3, 6, dtype=torch.float64)
    h2 = torch.randn_like(h)
    f = oracle.gcg_fwd_ref_torch
    torch.testing.assert_close(f(x, B, C, 2 * h + h2), 2 * f(x, B, C, h) + f(x, B, C, h2))
    torch.testing.assert_close(f(x, B, C, h), f(B, x, C, h))  # pre-gate pair is symmetric
    g = oracle.gcg_fwd_oracle
    torch.testing.assert_close(g(x, B, C, h), g(B, x, C, h))


# ---- Toeplitz known answers ---------------------------------------------------------------
def test_toeplitz_arange_known_answer():
    """h = arange(g*hl) (tests/test_toeplitz.py:39 of the reference): T[i,j] = h[hl-1-(i-j)],
    Tc[i,j] = h[hl-1-(i+cs-j)], written out by hand for hl = 4, chunk 6."""
    g, hl, cs = 2, 4, 6
    h = torch.arange(g * hl, dtype=torch.float64).reshape(g, 1, hl)   # group 0: 0 1 2 3, group 1: 4 5 6 7
    T, Tc = oracle.toeplitz(h, cs), oracle.correction_toeplitz(h, cs)
    want_T0 = torch.tensor([
        [3, 0, 0, 0, 0, 0],
        [2, 3, 0, 0, 0, 0],
        [1, 2, 3, 0, 0, 0],
        [0, 1, 2, 3, 0, 0],
        [0, 0, 1, 2, 3, 0],
        [0, 0, 0, 1, 2, 3]], dtype=torch.float64)
    want_T1 = torch.tensor([
        [7, 0, 0, 0, 0, 0],
        [6, 7, 0, 0, 0, 0],
        [5, 6, 7, 0, 0, 0],
        [4, 5, 6, 7, 0, 0],
        [0, 4, 5, 6, 7, 0],
        [0, 0, 4, 5, 6, 7]], dtype=torch.float64)
    want_Tc1 = torch.tensor([
        [0, 0, 0, 4, 5, 6],
        [0, 0, 0, 0, 4, 5],
        [0, 0, 0, 0, 0, 4],
        [0, 0, 0, 0, 0, 0],
        [0, 0, 0, 0, 0, 0],
        [0, 0, 0, 0, 0, 0]], dtype=torch.float64)
    torch.testing.assert_close(T[0], want_T0)
    torch.testing.assert_close(T[1], want_T1)
    torch.testing.assert_close(Tc[1], want_Tc1)
    # the C builder agrees
    lib = gcg_ref.load_c_oracle()
    hv = np.arange(hl, 2 * hl, dtype=np.float64)
    Tn, Tcn = np.zeros((cs, cs)), np.zeros((cs, cs))
    assert lib.gcg_oracle_toeplitz_f64(hv.ctypes.data, hl, cs, Tn.ctypes.data, Tcn.ctypes.data) == 0
    np.testing.assert_array_equal(Tn, want_T1.numpy())
    np.testing.assert_array_equal(Tcn, want_Tc1.numpy())


def test_toeplitz_product_is_full_convolution_matrix():
    """[Tc | T] stacked over chunks is the banded lower-triangular Toeplitz matrix of the
    whole sequence: compare with scipy's construction."""
    from scipy.linalg import toeplitz as sp_toeplitz

    hl, cs, n = 5, 8, 3
    h = torch.randn(1, 1, hl, dtype=torch.float64)
    T, Tc = oracle.toeplitz(h, cs)[0], oracle.correction_toeplitz(h, cs)[0]
    col = np.zeros(cs * n)
    col[:hl] = h[0, 0].flip(-1).numpy()                      # lag 0 first
    full = sp_toeplitz(col, np.zeros(cs * n))
    for i in range(n):
        np.testing.assert_allclose(full[i * cs:(i + 1) * cs, i * cs:(i + 1) * cs], T.numpy())
        if i:
            np.testing.assert_allclose(full[i * cs:(i + 1) * cs, (i - 1) * cs:i * cs], Tc.numpy())
        if i > 1:
            assert not full[i * cs:(i + 1) * cs, :(i - 1) * cs].any()


# ---- chunk invariance (tests/test_two_pass_ref.py:36-50 of the reference) --------------------------
@pytest.mark.parametrize("hl", [1, 4, 16, 17])
@pytest.mark.parametrize("chunk", [16, 32, 64])
def test_two_pass_matches_direct(hl, chunk):
    bs, L, g, dg = 2, 128, 2, 4
    x, B, C, h, dy = rand(bs, L, g, dg, hl)
    want = oracle.gcg_fwd_ref_torch(x, B, C, h)
    torch.testing.assert_close(oracle.gcg_two_pass_chunked_fwd(x, B, C, h, chunk), want, atol=1e-12, rtol=1e-12)
    got = oracle.gcg_two_pass_chunked_bwd(dy, x, B, C, h, chunk)
    ref = oracle.gcg_bwd_ref_torch(dy, x, B, C, h)
    for a, b, n in zip(got, ref, ("dx", "dB", "dC", "dh")):
        torch.testing.assert_close(a, b, atol=1e-11, rtol=1e-11, msg=n)


# ---- gradients -------------------------------------------------------------------------
@pytest.mark.parametrize("bs,L,g,dg,hl", SHAPES[:4])
def test_c_bwd_matches_autograd(bs, L, g, dg, hl):
    x, B, C, h, dy = rand(bs, L, g, dg, hl, dtype=torch.float32)
    got = oracle.gcg_bwd_oracle(dy, x, B, C, h)
    ref = oracle.gcg_bwd_ref_torch(dy, x, B, C, h)
    for a, b, n in zip(got, ref, ("dx", "dB", "dC", "dh")):
        torch.testing.assert_close(a.double(), b, atol=2e-5, rtol=2e-5, msg=n)


def test_c_bwd_matches_finite_differences():
    """The C backward against central differences of <dy, y>, y from the library-form forward evaluated in fp64
    (plain function values: autograd is not involved)."""
    bs, L, g, dg, hl = 1, 12, 2, 2, 5
    x, B, C, h, dy = rand(bs, L, g, dg, hl, dtype=torch.float64)
    dx, dB, dC, dh = oracle.gcg_bwd_oracle(dy, x, B, C, h)
    f = lambda *a: (dy * oracle.gcg_fwd_ref_torch(*a)).sum().item()
    eps = 1e-6
    args = [x, B, C, h]
    for idx, grad in enumerate((dx, dB, dC, dh)):
        flat = args[idx].reshape(-1)
        for probe in (0, flat.numel() // 2, flat.numel() - 1):
            keep = flat[probe].item()
            flat[probe] = keep + eps
            up = f(*args)
            flat[probe] = keep - eps
            dn = f(*args)
            flat[probe] = keep
            fd = (up - dn) / (2 * eps)
            assert abs(fd - grad.reshape(-1)[probe].item()) < 1e-4 * max(1.0, abs(fd))


def test_gradcheck_library_form():
    x, B, C, h, _ = rand(1, 10, 2, 2, 4)
    for t in (x, B, C, h):
        t.requires_grad_(True)
    assert torch.autograd.gradcheck(oracle.gcg_fwd_ref_torch, (x, B, C, h), atol=1e-6)


def test_dh_equals_conv1d_weight():
    """dh via torch.nn.grad.conv1d_weight, the routine the reference backward calls
    (src/bwd.py:415-418)."""
    from torch.nn.grad import conv1d_weight

    bs, L, g, dg, hl = 2, 50, 3, 4, 6
    x, B, C, h, dy = rand(bs, L, g, dg, hl)
    d = g * dg
    u = (B * x).reshape(bs, L, d).transpose(1, 2)
    g2 = (dy * C).reshape(bs, L, d).transpose(1, 2)
    dw = conv1d_weight(F.pad(u, (hl - 1, 0)), (d, 1, hl), g2, groups=d)
    want = dw.reshape(g, dg, 1, hl).sum(1)
    got = oracle.gcg_bwd_oracle(dy, x, B, C, h)[3]
    torch.testing.assert_close(got.double(), want, atol=1e-4, rtol=1e-5)


def test_bf16_rounding_helper():
    t = torch.tensor([1.0, 1.0 + 2 ** -9, 1.0 + 2 ** -8, 3.14159, -1e-3])
    torch.testing.assert_close(oracle.bf16_round(t), t.to(torch.bfloat16).float())
    x, B, C, h, _ = rand(1, 20, 1, 2, 3, dtype=torch.float32)
    bx, _, _ = oracle.gcg_fwd_oracle(x, B, C, h, round_bx_bf16=True, return_intermediates=True)
    torch.testing.assert_close(bx, oracle.bf16_round(B * x))
    # the rounded product also enters the sums: same y2, y as the plain oracle fed the rounded product as x with B = 1
    _, y2r, yr = oracle.gcg_fwd_oracle(x, B, C, h, round_bx_bf16=True, return_intermediates=True)
    _, y2p, yp = oracle.gcg_fwd_oracle(oracle.bf16_round(B * x), torch.ones_like(B), C, h, return_intermediates=True)
    assert torch.equal(y2r, y2p) and torch.equal(yr, yp)
    assert not torch.equal(y2r, oracle.gcg_fwd_oracle(x, B, C, h, return_intermediates=True)[1])
