"""CPU oracle for y = C * conv(B * x, h)  --  TEST INFRASTRUCTURE, not product code.

Three independent statements of the same operator, so that each can be pinned
against the others and against closed forms (tests/test_oracle.py):

* ``gcg_fwd_oracle`` / ``gcg_bwd_oracle``: nested sums with double accumulators in
  C (oracle/gcg_oracle.c), following
  savanna/kernels/triton_src/cgcg/ref_fwd.py:82-136 and src/bwd.py:442-471.
* ``gcg_fwd_ref_torch`` / ``gcg_bwd_ref_torch``: the library formulation the
  reference itself uses as ground truth -- a depthwise ``F.conv1d`` cross-correlation
  with left padding hl-1 (ref_fwd.py:109-129) and autograd of it
  (tests/test_bwd_refactor.py:95-103).
* ``gcg_two_pass_chunked_fwd`` / ``gcg_two_pass_chunked_bwd``: the chunked Toeplitz
  form  Y_n = T U_n + Tc U_{n-1}  (ref_fwd.py:223-277) and its adjoint with the
  diagonal-sum filter gradient (ref_bwd.py:5-115).

Layout everywhere: x, B, C, y, dy (bs, L, g, dg) channel-fastest; h (g, 1, hl).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def load_c_oracle() -> ctypes.CDLL:
    """Load oracle/libgcg_oracle.so, building it with make when it is absent."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = os.path.join(_HERE, "libgcg_oracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", _HERE, "-s"])
    lib = ctypes.CDLL(path)
    f32p, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32
    lib.gcg_oracle_fwd_f32.argtypes = [f32p] * 7 + [i64, i64, i32, i32, i32, i32]
    lib.gcg_oracle_fwd_f32.restype = ctypes.c_int
    lib.gcg_oracle_bwd_f32.argtypes = [f32p] * 9 + [i64, i64, i32, i32, i32]
    lib.gcg_oracle_bwd_f32.restype = ctypes.c_int
    lib.gcg_oracle_toeplitz_f64.argtypes = [f32p, i32, i32, f32p, f32p]
    lib.gcg_oracle_toeplitz_f64.restype = ctypes.c_int
    _LIB = lib
    return lib


def _f32c(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to(device="cpu", dtype=torch.float32).contiguous()


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    """Round an fp32 tensor to the nearest bfloat16 value, returned as fp32."""
    return t.to(torch.bfloat16).to(torch.float32)


def _dims(x: torch.Tensor, h: torch.Tensor):
    bs, L, g, dg = x.shape
    assert h.dim() == 3 and h.shape[0] == g and h.shape[1] == 1, "h must be (g, 1, hl)"
    return bs, L, g, dg, h.shape[-1]


# ----------------------------------------------------------------------------- C sums
def gcg_fwd_oracle(x, B, C, h, round_bx_bf16: bool = False, return_intermediates: bool = False):
    """Forward by direct summation in double precision; fp32 in, fp32 out.

    Returns y, or (Bx, y2, y) like gcg_fwd_ref_corrected(return_intermediates=True)
    (ref_fwd.py:131-135).
    """
    lib = load_c_oracle()
    bs, L, g, dg, hl = _dims(x, h)
    x_, B_, C_, h_ = _f32c(x), _f32c(B), _f32c(C), _f32c(h)
    y = torch.empty_like(x_)
    y2 = torch.empty_like(x_)
    bx = torch.empty_like(x_)
    rc = lib.gcg_oracle_fwd_f32(
        x_.data_ptr(), B_.data_ptr(), C_.data_ptr(), h_.data_ptr(),
        y.data_ptr(), y2.data_ptr(), bx.data_ptr(), bs, L, g, dg, hl, int(round_bx_bf16),
    )
    assert rc == 0, rc
    return (bx, y2, y) if return_intermediates else y


def gcg_bwd_oracle(dy, x, B, C, h):
    """(dx, dB, dC, dh) by direct summation in double precision; dh is (g, 1, hl)."""
    lib = load_c_oracle()
    bs, L, g, dg, hl = _dims(x, h)
    dy_, x_, B_, C_, h_ = _f32c(dy), _f32c(x), _f32c(B), _f32c(C), _f32c(h)
    dx, dB, dC = torch.empty_like(x_), torch.empty_like(x_), torch.empty_like(x_)
    dh = torch.empty(g, 1, hl, dtype=torch.float32)
    rc = lib.gcg_oracle_bwd_f32(
        dy_.data_ptr(), x_.data_ptr(), B_.data_ptr(), C_.data_ptr(), h_.data_ptr(),
        dx.data_ptr(), dB.data_ptr(), dC.data_ptr(), dh.data_ptr(), bs, L, g, dg, hl,
    )
    assert rc == 0, rc
    return dx, dB, dC, dh


# ------------------------------------------------------------------- library formulation
def gcg_fwd_ref_torch(x, B, C, h, return_intermediates: bool = False):
    """Depthwise cross-correlation statement (ref_fwd.py:109-129), any float dtype.

    Left-pads hl-1 zeros explicitly instead of padding both sides and trimming the
    tail; the two are the same map.
    """
    bs, L, g, dg, hl = _dims(x, h)
    d = g * dg
    u = B * x
    u_cl = u.reshape(bs, L, d).transpose(1, 2)                 # (bs, d, L)
    w = h.repeat_interleave(dg, dim=0)                          # (d, 1, hl), blocked per group
    y2_cl = F.conv1d(F.pad(u_cl, (hl - 1, 0)), w, groups=d)     # no flip: tap hl-1 hits sample t
    y2 = y2_cl.transpose(1, 2).reshape(bs, L, g, dg)
    y = C * y2
    return (u, y2, y) if return_intermediates else y


def gcg_bwd_ref_torch(dy, x, B, C, h, dtype=torch.float64):
    """Gradients by autograd of gcg_fwd_ref_torch, evaluated in ``dtype``."""
    xs = [t.detach().to(dtype).clone().requires_grad_(True) for t in (x, B, C, h)]
    y = gcg_fwd_ref_torch(*xs)
    y.backward(dy.detach().to(dtype))
    return tuple(t.grad for t in xs)  # dx, dB, dC, dh


# ------------------------------------------------------------------------- brute force
def brute_force_fwd(x, B, C, h):
    """Pure-Python quadruple loop over the defining sum; tiny shapes only."""
    bs, L, g, dg, hl = _dims(x, h)
    y = torch.zeros(bs, L, g, dg, dtype=torch.float64)
    xd, Bd, Cd, hd = (t.double() for t in (x, B, C, h))
    for b in range(bs):
        for t in range(L):
            for gi in range(g):
                for c in range(dg):
                    s = 0.0
                    for k in range(hl):
                        src = t - (hl - 1) + k
                        if src >= 0:
                            s += float(hd[gi, 0, k]) * float(Bd[b, src, gi, c]) * float(xd[b, src, gi, c])
                    y[b, t, gi, c] = float(Cd[b, t, gi, c]) * s
    return y


# ------------------------------------------------------------------------ two-pass form
def toeplitz(h: torch.Tensor, chunk: int) -> torch.Tensor:
    """In-chunk factor: T[g,i,j] = h[g,0,hl-1-(i-j)] for 0 <= i-j < hl, else 0.

    Equals utils.toeplitz(h[:, 0].flip(-1), chunk) of the reference (utils.py:5-24,
    called that way at ref_fwd.py:234-242).
    """
    g, _, hl = h.shape
    i = torch.arange(chunk).view(-1, 1)
    j = torch.arange(chunk).view(1, -1)
    lag = i - j
    ok = (lag >= 0) & (lag < hl)
    idx = (hl - 1 - lag).clamp(0, hl - 1)
    return torch.where(ok.unsqueeze(0), h[:, 0, :][:, idx], torch.zeros((), dtype=h.dtype))


def correction_toeplitz(h: torch.Tensor, chunk: int) -> torch.Tensor:
    """Carry factor: Tc[g,i,j] = h[g,0,hl-1-(i+chunk-j)] for 0 <= i+chunk-j < hl, else 0
    (utils.py:38-51 applied to the flipped filter, ref_fwd.py:253)."""
    g, _, hl = h.shape
    i = torch.arange(chunk).view(-1, 1)
    j = torch.arange(chunk).view(1, -1)
    lag = i + chunk - j
    ok = (lag >= 0) & (lag < hl)
    idx = (hl - 1 - lag).clamp(0, hl - 1)
    return torch.where(ok.unsqueeze(0), h[:, 0, :][:, idx], torch.zeros((), dtype=h.dtype))


def _chunked(t: torch.Tensor, chunk: int) -> torch.Tensor:
    bs, L, g, dg = t.shape
    return t.reshape(bs, L // chunk, chunk, g, dg).permute(0, 1, 3, 2, 4)  # b n g i c


def _unchunked(t: torch.Tensor) -> torch.Tensor:
    bs, n, g, chunk, dg = t.shape
    return t.permute(0, 1, 3, 2, 4).reshape(bs, n * chunk, g, dg)


def gcg_two_pass_chunked_fwd(x, B, C, h, chunk: int, return_intermediates: bool = False):
    """Y_n = T U_n + Tc U_{n-1} with U_{-1} = 0 (ref_fwd.py:223-277). Needs hl <= chunk+1."""
    bs, L, g, dg, hl = _dims(x, h)
    assert L % chunk == 0 and hl - 1 <= chunk
    U = _chunked(B * x, chunk)
    T, Tc = toeplitz(h, chunk), correction_toeplitz(h, chunk)
    U_prev = torch.zeros_like(U)
    U_prev[:, 1:] = U[:, :-1]
    y2 = _unchunked(T @ U + Tc @ U_prev)
    y = C * y2
    return (y2, y) if return_intermediates else y


def gcg_two_pass_chunked_bwd(dy, x, B, C, h, chunk: int):
    """Adjoint of the two-pass form (ref_bwd.py:31-115):
    dU_n = T^T G_n + Tc^T G_{n+1};  dT = sum G_n U_n^T;  dTc = sum G_n U_{n-1}^T;
    dh[hl-1-i] = sum diag_{-i}(dT);  dh[i] += sum diag_{chunk-(hl-1)+i}(dTc) (ref_bwd.py:5-28).
    """
    bs, L, g, dg, hl = _dims(x, h)
    y2, _ = gcg_two_pass_chunked_fwd(x, B, C, h, chunk, return_intermediates=True)
    dC = dy * y2
    G = _chunked(dy * C, chunk)
    U = _chunked(B * x, chunk)
    T, Tc = toeplitz(h, chunk), correction_toeplitz(h, chunk)
    G_next = torch.zeros_like(G)
    G_next[:, :-1] = G[:, 1:]
    U_prev = torch.zeros_like(U)
    U_prev[:, 1:] = U[:, :-1]
    dU = _unchunked(T.transpose(1, 2) @ G + Tc.transpose(1, 2) @ G_next)
    dT = (G @ U.transpose(3, 4)).sum(dim=(0, 1))           # g, i, j
    dTc = (G @ U_prev.transpose(3, 4)).sum(dim=(0, 1))
    dh = torch.zeros(g, 1, hl, dtype=dT.dtype)
    for i in range(hl):
        dh[:, 0, hl - 1 - i] += dT.diagonal(offset=-i, dim1=1, dim2=2).sum(-1)
        off = chunk - (hl - 1) + i
        if off < chunk:
            dh[:, 0, i] += dTc.diagonal(offset=off, dim1=1, dim2=2).sum(-1)
    return dU * B, dU * x, dC, dh
