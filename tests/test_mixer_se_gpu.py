"""Featurizer conv + short gated convolution in one pass (gcg_mixer_se_fwd / gcg_mixer_se_bwd) through the
C ABI: against the chain of entry points it replaces (gcg_dwconv_* and gcg_*_interleaved) and against
the CPU oracle applied twice, which follows
block.py:867-890 and hyena.py:825-840 of the reference."""
import pytest
import torch

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]

# (bs, L, g, dg, hl, kf)
SHAPES = [
    (2, 64, 4, 16, 7, 3),        # Hyena-SE: 7 taps after a 3-tap featurizer
    (1, 300, 3, 8, 7, 3),        # ragged length, three runs
    (2, 77, 2, 2, 4, 4),
    (1, 1, 8, 2, 7, 3),          # a single row
    (1, 5, 1, 4, 8, 4),
    (1, 513, 2, 16, 3, 2),
    (3, 129, 5, 6, 7, 1),        # featurizer of one tap: a per-channel scale
    (1, 1000, 6, 10, 5, 3),
    (2, 256, 130, 4, 7, 3),      # more lanes than one workgroup
    (1, 40, 2, 6, 1, 3),         # operator of one tap
]


def data(bs, L, g, dg, hl, kf, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    raw = torch.randn(bs, L, g, dg, 3, generator=gen).to(dtype)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    wf = (torch.randn(3 * g * dg, 1, kf, generator=gen) / kf ** 0.5).to(dtype)
    h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype)
    return raw, dy, wf, h


def oracle_chain(raw, dy, wf, h, dtype):
    """fp32 oracle of featurizer -> round to dtype -> gated convolution, and its backward with the
    gradient of the features rounded to dtype in between, as the chain of kernels stores it."""
    bs, L, g, dg, _ = raw.shape
    r4 = raw.float().reshape(bs, L, 3 * g * dg, 1)
    one = torch.ones_like(r4)
    f = oracle.gcg_fwd_oracle(r4, one, one, wf.float()).to(dtype).float().reshape(bs, L, g, dg, 3)
    C, B, x = f[..., 0].contiguous(), f[..., 1].contiguous(), f[..., 2].contiguous()
    y = oracle.gcg_fwd_oracle(x, B, C, h.float())
    dx, dB, dC, dh = oracle.gcg_bwd_oracle(dy.float(), x, B, C, h.float())
    df = torch.stack([dC, dB, dx], dim=-1).to(dtype).float().reshape(bs, L, 3 * g * dg, 1)
    draw, _, _, dwf = oracle.gcg_bwd_oracle(df, r4, one, one, wf.float())
    return y, draw.reshape(raw.shape), dwf, dh


def kernel_chain(raw, dy, wf, h):
    bs, L, g, dg, _ = raw.shape
    r4 = raw.view(bs, L, 3 * g * dg, 1)
    f = _lib.dwconv_fwd(r4, wf).view(bs, L, g, dg, 3)
    y = _lib.fwd_interleaved(f, h)
    df, dh = _lib.bwd_interleaved(dy, f, h)
    draw, dwf = _lib.dwconv_bwd(df.view(bs, L, 3 * g * dg, 1), r4, wf)
    return y, draw.view(raw.shape), dwf, dh


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("bs,L,g,dg,hl,kf", SHAPES)
def test_mixer_se_fwd_bwd(gcg_lib, bs, L, g, dg, hl, kf, dtype):
    raw, dy, wf, h = data(bs, L, g, dg, hl, kf, dtype, seed=L + hl)
    ref = oracle_chain(raw, dy, wf, h, dtype)
    rawd, dyd, wfd, hd = (t.to(DEV) for t in (raw, dy, wf, h))
    y = _lib.mixer_se_fwd(rawd, wfd, hd)
    draw, dwf, dh = _lib.mixer_se_bwd(dyd, rawd, wfd, hd)
    torch.cuda.synchronize()
    assert y.shape == (bs, L, g, dg) and draw.shape == raw.shape and dwf.shape == wf.shape and dh.shape == h.shape
    # two rounded stages back to back: the gradient's tolerance is twice the single-stage one
    assert_close(y, ref[0], TOL[dtype], "y")
    assert_close(draw, ref[1], 2 * TOL[dtype], "d raw")
    if bs * L * dg >= 256 or dtype == torch.float32:      # a tap summed from a handful of rounded terms can cancel
        assert_close(dwf, ref[2], 2 * TOL_DH[dtype], "dwf")
        assert_close(dh, ref[3], TOL_DH[dtype], "dh")
    if (3 * g * dg) % 4 == 0:                              # the stand-alone featurizer takes multiples of 4 channels
        y_c, draw_c, dwf_c, dh_c = kernel_chain(rawd, dyd, wfd, hd)
        torch.cuda.synchronize()
        # same products, other summation orders: equal up to rounding
        assert_close(y, y_c, 1e-5 if dtype == torch.float32 else TOL[dtype], "y vs chain")
        assert_close(draw, draw_c, 1e-5 if dtype == torch.float32 else TOL[dtype], "d raw vs chain")
        if bs * L * dg >= 256 or dtype == torch.float32:
            assert_close(dwf, dwf_c, TOL_DH[dtype], "dwf vs chain")
            assert_close(dh, dh_c, TOL_DH[dtype], "dh vs chain")


@pytest.mark.parametrize("planar", [False, True], ids=["interleaved", "planar"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("bs,L,g,dg,hl,kf", SHAPES)
def test_fp32_filter_on_16_bit_tensors(gcg_lib, bs, L, g, dg, hl, kf, dtype, planar):
    """16-bit raw and wf with an fp32 operator filter (cgcg_dtype float32 on 16-bit activations, hyena.py:812-816):
    the featurizer's output is rounded to the tensors' type, the operator's taps and arithmetic stay in fp32, dh
    comes back in fp32.  Against the oracle of that chain and against the chain of kernels."""
    raw, dy, wf, _ = data(bs, L, g, dg, hl, kf, dtype, seed=L + hl + 1)
    h = torch.randn(g, 1, hl, generator=torch.Generator().manual_seed(L)) / hl ** 0.5          # fp32, not representable in 16 bits
    ref = oracle_chain(raw, dy, wf, h, dtype)
    rawd, dyd, wfd, hd = (t.to(DEV) for t in (raw, dy, wf, h))
    if planar:
        d = g * dg
        raw_in = rawd.permute(0, 1, 4, 2, 3).contiguous()
        wf_in = wfd.view(d, 3, 1, kf).permute(1, 0, 2, 3).reshape(3 * d, 1, kf).contiguous()
    else:
        raw_in, wf_in = rawd, wfd
    y = _lib.mixer_se_fwd(raw_in, wf_in, hd, planar=planar)
    draw, dwf, dh = _lib.mixer_se_bwd(dyd, raw_in, wf_in, hd, planar=planar)
    torch.cuda.synchronize()
    assert y.dtype == dtype and draw.dtype == dtype and dwf.dtype == dtype and dh.dtype == torch.float32
    if planar:
        draw = draw.permute(0, 1, 3, 4, 2)
        dwf = dwf.view(3, g * dg, 1, kf).permute(1, 0, 2, 3).reshape(3 * g * dg, 1, kf)
    assert_close(y, ref[0], TOL[dtype], "y")
    assert_close(draw, ref[1], 2 * TOL[dtype], "d raw")
    if bs * L * dg >= 256:
        assert_close(dwf, ref[2], 2 * TOL_DH[dtype], "dwf")
        assert_close(dh, ref[3], TOL_DH[dtype], "dh")
    if (3 * g * dg) % 4 == 0 and dg % 4 == 0:          # what the stand-alone kernels take
        y_c, draw_c, dwf_c, dh_c = kernel_chain(rawd, dyd, wfd, hd)
        torch.cuda.synchronize()
        assert dh_c.dtype == torch.float32
        assert_close(y, y_c, TOL[dtype], "y vs chain")
        assert (y != y_c).float().mean() < 0.02, "more than rounding separates y from the chain of kernels"
        assert_close(draw, draw_c, TOL[dtype], "d raw vs chain")
        if bs * L * dg >= 256:
            assert_close(dh, dh_c, 1e-4, "dh vs chain")          # both in fp32


def test_mixer_se_is_deterministic_and_rejects_what_it_cannot_run(gcg_lib):
    raw, dy, wf, h = (t.to(DEV) for t in data(2, 512, 8, 16, 7, 3, torch.bfloat16, seed=1))
    a, b = _lib.mixer_se_bwd(dy, raw, wf, h), _lib.mixer_se_bwd(dy, raw, wf, h)
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    raw9, dy9, wf9, h9 = (t.to(DEV) for t in data(1, 64, 8, 2, 9, 3, torch.float32, seed=2))      # 9 taps
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.mixer_se_fwd(raw9, wf9, h9)
    raw5, dy5, wf5, h5 = (t.to(DEV) for t in data(1, 64, 8, 2, 7, 5, torch.float32, seed=2))      # 5 featurizer taps
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.mixer_se_bwd(dy5, raw5, wf5, h5)
    raw3, _, wf3, h3 = (t.to(DEV) for t in data(1, 64, 8, 3, 7, 3, torch.float32, seed=2))        # odd group width
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.mixer_se_fwd(raw3, wf3, h3)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _lib.mixer_se_fwd(raw.cpu(), wf.cpu(), h.cpu())


def test_mixer_se_shape_of_a_40b_layer(gcg_lib):
    """B=1, L=8192, 8192 channels in 256 groups, 7 taps after 3, bf16: against the chain of kernels,
    and a shift featurizer with a one-tap operator must reproduce products of the input bit for bit."""
    bs, L, g, dg, hl, kf, dtype = 1, 8192, 256, 32, 7, 3, torch.bfloat16
    gen = torch.Generator(device=DEV).manual_seed(7)
    raw = torch.randn(bs, L, g, dg, 3, generator=gen, device=DEV).to(dtype)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=DEV)).to(dtype)
    wf = (torch.randn(3 * g * dg, 1, kf, generator=gen, device=DEV) / kf ** 0.5).to(dtype)
    h = (torch.randn(g, 1, hl, generator=gen, device=DEV) / hl ** 0.5).to(dtype)
    y = _lib.mixer_se_fwd(raw, wf, h)
    draw, dwf, dh = _lib.mixer_se_bwd(dy, raw, wf, h)
    y_c, draw_c, dwf_c, dh_c = kernel_chain(raw, dy, wf, h)
    torch.cuda.synchronize()
    # the featurizer's taps are summed two at a time here and one at a time in the chain: the same
    # products, another rounding of their sum
    assert_close(y, y_c, TOL[dtype], "y")
    assert_close(draw, draw_c, TOL[dtype], "d raw")
    assert (y != y_c).float().mean() < 0.02, "more than rounding separates y from the chain of kernels"
    assert_close(dwf, dwf_c, TOL_DH[dtype], "dwf")
    assert_close(dh, dh_c, TOL_DH[dtype], "dh")
    # featurizer = delay by one row, operator = delay by two: y[t] = C[t-1] * (B * x)[t-3]
    wf.zero_(); wf[:, 0, 1] = 1.0
    h.zero_(); h[:, 0, hl - 3] = 1.0
    y = _lib.mixer_se_fwd(raw, wf, h)
    torch.cuda.synchronize()
    C, B, x = raw[..., 0].float(), raw[..., 1].float(), raw[..., 2].float()
    want = (C[:, 2:-1] * (B[:, :-3] * x[:, :-3])).to(dtype)
    assert torch.equal(y[:, 3:], want) and not y[:, :3].any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_hyena_mixer_routes_short_operators_through_the_fused_kernels(gcg_lib, dtype):
    """HyenaMixer with a Hyena-SE operator: the fused path (one kernel each way) against the same
    module with fuse_short=False (featurizer kernel, then interleaved operator), output and all
    gradients; activations in bf16 or fp32 with fp32 parameters, as the block holds them."""
    import copy

    from savanna_amd.operators.hyena import CgcgConfig, HyenaMixer, HyenaSEOperator, _FeaturizedShortGateConvGate

    torch.manual_seed(5)
    bs, L, hidden, groups = 2, 300, 192, 12
    cfg = CgcgConfig(cgcg_dtype="bfloat16" if dtype == torch.bfloat16 else "float32")
    fused = HyenaMixer(HyenaSEOperator(hidden, groups, 7, cfg, device=DEV), 3, device=DEV)
    chain = copy.deepcopy(fused)
    chain.fuse_short = False
    feats = torch.randn(bs, L, 3 * hidden, device=DEV).to(dtype)
    dz = (0.1 * torch.randn(bs, L, hidden, device=DEV)).to(dtype)
    assert fused._fusable(feats, 7) and not chain._fusable(feats, 7)
    out = []
    for m in (fused, chain):
        x = feats.clone().requires_grad_(True)
        z = m(x)
        z.backward(dz)
        out.append((z, x.grad, m.hyena_proj_conv.short_conv_weight.grad, m.mixer.short_conv_weight.grad))
    torch.cuda.synchronize()
    tol = TOL[dtype] if dtype != torch.float32 else 1e-5
    assert_close(out[0][0], out[1][0], tol, "z")
    assert_close(out[0][1], out[1][1], tol, "d features")
    assert_close(out[0][2], out[1][2], TOL_DH[dtype], "d featurizer weight")
    assert_close(out[0][3], out[1][3], TOL_DH[dtype], "d operator weight")
    # the fused path really is the one that ran
    x = feats.clone().requires_grad_(True)
    producer = fused(x).grad_fn.next_functions[0][0]            # below the reshape to (b, l, hidden)
    assert type(producer).__name__.startswith(_FeaturizedShortGateConvGate.__name__)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_fused_kernels_in_a_replayed_graph(gcg_lib, dtype):
    """Forward and backward of the fused kernels captured in one HIP graph and replayed with new
    contents, with eager work between the replays; every replay must equal the eager result bit for
    bit (the library allocates nothing and clears nothing; the workspace comes from the capture's pool)."""
    bs, L, g, dg, hl, kf = 1, 1024, 8, 16, 7, 3
    raw = torch.randn(bs, L, g, dg, 3, device=DEV).to(dtype)
    dy = torch.randn(bs, L, g, dg, device=DEV).to(dtype)
    wf = (torch.randn(3 * g * dg, 1, kf, device=DEV) / kf ** 0.5).to(dtype)
    h = (torch.randn(g, 1, hl, device=DEV) / hl ** 0.5).to(dtype)

    def both(raw_t, dy_t):
        return (_lib.mixer_se_fwd(raw_t, wf, h),) + _lib.mixer_se_bwd(dy_t, raw_t, wf, h)

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):                      # warm-up on the capture stream
        both(raw, dy)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = both(raw, dy)
    for it in range(3):
        raw_new = torch.randn(bs, L, g, dg, 3, device=DEV).to(dtype)
        dy_new = torch.randn(bs, L, g, dg, device=DEV).to(dtype)
        raw.copy_(raw_new)
        dy.copy_(dy_new)
        graph.replay()
        torch.cuda.synchronize()
        out_e = both(raw_new, dy_new)               # eager work between replays
        torch.cuda.synchronize()
        for a, b, n in zip(out_g, out_e, ("y", "d raw", "dwf", "dh")):
            assert torch.equal(a, b), f"replay {it}: {n}"


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("bs,L,g,dg,hl,kf", SHAPES + [(2, 4096, 64, 16, 7, 3)])
def test_planar_features_match_interleaved(gcg_lib, bs, L, g, dg, hl, kf, dtype):
    """gcg_mixer_se_fwd_planar / _bwd_planar -- raw (bs, L, 3, g, dg), the split without interleaving of
    block.py:881-884, with the featurizer's filters in that channel order -- give the interleaved entry points'
    results on the same values, bit for bit (the same arithmetic on pieces loaded plane by plane)."""
    raw, dy, wf, h = (t.to(DEV) for t in data(bs, L, g, dg, hl, kf, dtype, seed=17))
    d = g * dg
    raw_pl = raw.permute(0, 1, 4, 2, 3).contiguous()                                  # (bs, L, 3, g, dg)
    wf_pl = wf.view(d, 3, 1, kf).permute(1, 0, 2, 3).reshape(3 * d, 1, kf).contiguous()    # row p * d + c <- row 3 c + p
    y = _lib.mixer_se_fwd(raw, wf, h)
    draw, dwf, dh = _lib.mixer_se_bwd(dy, raw, wf, h)
    y_pl = _lib.mixer_se_fwd(raw_pl, wf_pl, h, planar=True)
    draw_pl, dwf_pl, dh_pl = _lib.mixer_se_bwd(dy, raw_pl, wf_pl, h, planar=True)
    torch.cuda.synchronize()
    assert y_pl.shape == y.shape and draw_pl.shape == raw_pl.shape and dwf_pl.shape == wf.shape
    assert torch.equal(y_pl, y)
    assert torch.equal(draw_pl, draw.permute(0, 1, 4, 2, 3))
    assert torch.equal(dwf_pl.view(3, d, 1, kf), dwf.view(d, 3, 1, kf).permute(1, 0, 2, 3))
    assert torch.equal(dh_pl, dh)


def test_hyena_mixer_planar_fused(gcg_lib):
    """HyenaMixer(interleave_projections=False) with a Hyena-SE operator: one kernel each way, same output and
    gradients as the two-kernel chain on the same layout up to the rounding of fp32 sums."""
    from savanna_amd.operators.hyena import CgcgConfig, HyenaMixer, HyenaSEOperator

    torch.manual_seed(2)
    bs, L, hidden, groups = 2, 512, 128, 8
    cfg = CgcgConfig(cgcg_dtype="bfloat16")
    mixer = HyenaMixer(HyenaSEOperator(hidden, groups, 7, cfg, device=DEV), 3, dtype=torch.bfloat16, device=DEV,
                       interleave_projections=False)
    feats = torch.randn(bs, L, 3 * hidden, device=DEV).to(torch.bfloat16).requires_grad_(True)
    dz = (0.1 * torch.randn(bs, L, hidden, device=DEV)).to(torch.bfloat16)
    params = list(mixer.parameters())

    def run(fuse):
        mixer.fuse_short = fuse
        feats.grad = None
        for p in params:
            p.grad = None
        z = mixer(feats)
        z.backward(dz)
        return [z.detach(), feats.grad.clone()] + [p.grad.clone() for p in params]

    want = run(False)
    from torch.profiler import ProfilerActivity, profile
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        got = run(True)
        torch.cuda.synchronize()
    for a, b, n in zip(got, want, ("z", "d features", "p0", "p1")):
        assert_close(a, b, 2e-2, n)
    big = [e.key for e in prof.key_averages() if "mixer_se" in e.key or "dwconv" in e.key or "window" in e.key]
    assert len(big) == 2 and all("mixer_se" in k for k in big), big


@pytest.mark.parametrize("planar", [False, True], ids=["interleaved", "planar"])
def test_hyena_mixer_16_bit_features_fp32_arithmetic(gcg_lib, planar):
    """bf16 activations with cgcg_dtype float32 (the default, global_config.py:404): the featurizer's output is
    rounded to bf16 before the operator's casts (block.py:873, hyena.py:812-816).  The one-kernel path does the
    same on the 16-bit features with an fp32 filter and fp32 arithmetic -- no fp32 copy of the features -- and
    gives the values of the reference's chain written with torch ops."""
    import torch.nn.functional as F

    from savanna_amd.operators.hyena import CgcgConfig, HyenaMixer, HyenaSEOperator

    torch.manual_seed(8)
    bs, L, hidden, groups, hl, kf = 2, 500, 128, 8, 7, 3
    dg = hidden // groups
    mixer = HyenaMixer(HyenaSEOperator(hidden, groups, hl, CgcgConfig(cgcg_dtype="float32"), device=DEV), kf,
                       dtype=torch.bfloat16, device=DEV, interleave_projections=not planar)
    feats = torch.randn(bs, L, 3 * hidden, device=DEV).to(torch.bfloat16)
    dz = (0.1 * torch.randn(bs, L, hidden, device=DEV)).to(torch.bfloat16)
    assert mixer._fusable(feats, hl)
    x = feats.clone().requires_grad_(True)
    z = mixer(x)
    assert type(z.grad_fn.next_functions[0][0]).__name__.startswith("_FeaturizedShortGateConvGate")    # below the reshape
    z.backward(dz)
    assert z.dtype == torch.bfloat16 and x.grad.dtype == torch.bfloat16
    got = (z, x.grad, mixer.hyena_proj_conv.short_conv_weight.grad.clone(), mixer.mixer.short_conv_weight.grad.clone())

    # the reference's chain: conv on (B, 3D, L) in bf16, split, casts to fp32, gated conv, cast back
    xr = feats.clone().requires_grad_(True)
    wf = mixer.hyena_proj_conv.short_conv_weight.detach().clone().requires_grad_(True)
    h = mixer.mixer.short_conv_weight.detach().clone().requires_grad_(True)
    f = F.conv1d(F.pad(xr.transpose(1, 2), (kf - 1, 0)), wf.to(torch.bfloat16), groups=3 * hidden).transpose(1, 2)
    if planar:
        x1, x2, v = f.reshape(bs, L, 3, groups, dg).unbind(2)
    else:
        x1, x2, v = f.reshape(bs, L, groups, dg, 3).unbind(4)
    u = (v.float() * x2.float()).reshape(bs, L, hidden).transpose(1, 2)
    y = F.conv1d(F.pad(u, (hl - 1, 0)), h.float().repeat_interleave(dg, 0), groups=hidden).transpose(1, 2)
    zr = (x1.float().reshape(bs, L, hidden) * y).to(torch.bfloat16)
    zr.backward(dz)
    torch.cuda.synchronize()
    assert_close(got[0], zr, TOL[torch.bfloat16], "z")
    assert_close(got[1], xr.grad, 2 * TOL[torch.bfloat16], "d features")
    assert_close(got[2], wf.grad, TOL_DH[torch.bfloat16], "d featurizer weight")
    assert_close(got[3], h.grad, TOL_DH[torch.bfloat16], "d operator weight")
