"""The featurizer conv and the two fused mixers on a projection output of 3 * 2^31 elements (B=1, L=2^19, 4096
channels, bf16): byte offsets into the tensor pass 2^32 and element offsets 2^31.  With a featurizer that delays by
one row and an operator filter that delays by a few, every output element is a product of input elements
(block.py:873-888 into hyena.py:517-531 / :825-840 written out for those filters), so an offset that wrapped
anywhere would move data and fail an exact comparison on the whole tensor."""
import pytest
import torch

from savanna_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BS, L, G, DG, KF = 1, 1 << 19, 256, 16, 3
DT = torch.bfloat16


def _raw_and_dy():
    raw = torch.empty(BS, L, G, DG, 3, dtype=DT, device=DEV)
    dy = torch.empty(BS, L, G, DG, dtype=DT, device=DEV)
    gen = torch.Generator(device=DEV)
    for s, t0 in enumerate(range(0, L, 1 << 16)):
        gen.manual_seed(300 + s)
        raw[:, t0:t0 + (1 << 16)].normal_(generator=gen)
        dy[:, t0:t0 + (1 << 16)].normal_(generator=gen)
    return raw, dy


def _delay_featurizer():
    wf = torch.zeros(3 * G * DG, 1, KF, dtype=DT, device=DEV)
    wf[:, 0, KF - 2] = 1.0                              # f[t] = raw[t-1]
    return wf


def _shifted(raw):
    f = torch.zeros_like(raw)
    f[:, 1:] = raw[:, :-1]
    return f


def test_featurizer_64bit_offsets(gcg_lib):
    raw, _ = _raw_and_dy()
    wf = _delay_featurizer()
    flat = raw.view(BS, L, 3 * G * DG, 1)
    f = _lib.dwconv_fwd(flat, wf)
    torch.cuda.synchronize()
    assert torch.equal(f[:, 1:], flat[:, :-1]) and not f[:, 0].any()
    # its backward advances by one row: d raw[t] = d f[t+1]; the filter gradient sums d f[t] * raw[t-2+k]
    draw, dwf = _lib.dwconv_bwd(f, flat, wf)
    torch.cuda.synchronize()
    assert torch.equal(draw[:, :-1], flat[:, :-1]) and not draw[:, -1].any()
    assert torch.isfinite(dwf.float()).all()


@pytest.mark.parametrize("planar", [False, True], ids=["interleaved", "planar"])
@pytest.mark.parametrize("kind", ["mr", "se"])
def test_fused_mixers_64bit_offsets(gcg_lib, kind, planar):
    hl, s = (128, 5) if kind == "mr" else (7, 2)
    raw, dy = _raw_and_dy()
    if planar:
        raw = raw.view(BS, L, 3, G, DG)                 # the same values read as "(p g dg)" rows (block.py:881-884)
    part = (lambda t, p: t[:, :, p]) if planar else (lambda t, p: t[..., p])
    wf = _delay_featurizer()
    h = torch.zeros(G, 1, hl, dtype=DT, device=DEV)
    h[:, 0, hl - 1 - s] = 1.0                           # y[t] = C[t] * (B*x)[t-s] on the featurized rows
    fwd, bwd = (_lib.mixer_mr_fwd, _lib.mixer_mr_bwd) if kind == "mr" else (_lib.mixer_se_fwd, _lib.mixer_se_bwd)
    assert kind == "se" or _lib.mixer_mr_supported(DG, hl, KF, raw)
    y = fwd(raw, wf, h, planar=planar)
    torch.cuda.synchronize()
    f = _shifted(raw)
    # the matrix-core kernels hold u = B*x and dy*C as 16-bit operands, the register-window kernels in fp32
    rnd = (lambda t: t.to(DT).float()) if kind == "mr" else (lambda t: t)
    u = rnd(part(f, 1).float() * part(f, 2).float())
    want = torch.zeros_like(y)
    want[:, s:] = (part(f, 0)[:, s:].float() * u[:, :-s]).to(DT)
    assert torch.equal(y, want), "y"
    del want, y

    draw, dwf, dh = bwd(dy, raw, wf, h, planar=planar)
    torch.cuda.synchronize()
    assert torch.isfinite(dh.float()).all() and torch.isfinite(dwf.float()).all()
    # gradient of the featurized rows, then one row earlier in d raw (the featurizer's delay, transposed)
    want = torch.zeros_like(dy)
    want[:, s:] = (dy[:, s:].float() * u[:, :-s]).to(DT)                            # dC[t] = dy[t] * u[t-s]
    assert torch.equal(part(draw, 0)[:, :-1], want[:, 1:]) and not draw[:, -1].any(), "d raw, C"
    del u
    g2 = rnd(dy.float() * part(f, 0).float())
    want.zero_()
    want[:, :-s] = (g2[:, s:] * part(f, 2)[:, :-s].float()).to(DT)                  # dB[t] = x[t] * (dy*C)[t+s]
    assert torch.equal(part(draw, 1)[:, :-1], want[:, 1:]), "d raw, B"
    want.zero_()
    want[:, :-s] = (g2[:, s:] * part(f, 1)[:, :-s].float()).to(DT)                  # dx[t] = B[t] * (dy*C)[t+s]
    assert torch.equal(part(draw, 2)[:, :-1], want[:, 1:]), "d raw, x"
