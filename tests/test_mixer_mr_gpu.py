"""Featurizer conv and Hyena-MR operator without the featurized tensor in memory (gcg_mixer_mr_fwd /
gcg_mixer_mr_bwd): the chain of savanna/model/block.py:867-890 (featurizer conv on the projected features,
interleaved split) into ParallelHyenaOperator's cgcg branch (hyena.py:517-531), with the rows of the features made
inside the operator's kernels.  Checked against the oracle applied twice (featurizer with both gates at one and
the intermediate rounded to the tensors' type, then the operator) and against the two-call chain of entry points."""
import pytest
import torch

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# (bs, L, g, dg, hl, kf)
SHAPES = [
    (2, 300, 3, 16, 128, 3),
    (1, 1000, 5, 16, 100, 3),     # partial channel tile
    (3, 2500, 10, 16, 128, 2),    # several runs per column; two taps
    (1, 2049, 20, 16, 98, 3),
    (2, 40, 2, 32, 128, 1),       # one tap: the featurizer scales its channels
    (1, 700, 17, 16, 128, 3),     # d = 272
    (1, 3000, 3, 64, 128, 3),     # a filter group as wide as a workgroup's channel block
    (2, 4100, 8, 16, 128, 3),     # runs of more than a hundred steps
    (2, 900, 6, 16, 64, 3),       # shorter filters (hyena_mr_len 64 in some configurations): the far slices are zero
    (1, 1300, 4, 32, 33, 2),
    (2, 500, 5, 16, 9, 3),
    (1, 200, 3, 16, 97, 3),
    (1, 20, 2, 16, 20, 3),        # sequences shorter than a step of 32 rows (the operator cuts hl to the length)
    (2, 31, 3, 16, 9, 3),
    (1, 33, 2, 16, 33, 1),
    (3, 9, 1, 16, 9, 2),
]
TYPES = [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16), (torch.float32, torch.float32),
         (torch.bfloat16, torch.float32)]


def make(bs, L, g, dg, hl, kf, dtype, filt, seed=0):
    gen = torch.Generator().manual_seed(seed)
    raw = torch.randn(bs, L, g, dg, 3, generator=gen).to(dtype)
    wf = (torch.randn(3 * g * dg, 1, kf, generator=gen) / kf ** 0.5).to(dtype)
    h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(filt)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    return raw, wf, h, dy


def chain(raw, wf, h, dy):
    bs, L, g, dg, _ = raw.shape
    flat = raw.reshape(bs, L, 3 * g * dg, 1)
    f = _lib.dwconv_fwd(flat, wf)
    y = _lib.fwd_interleaved(f.reshape(bs, L, g, dg, 3), h)
    dfeat, dh = _lib.bwd_interleaved(dy, f.reshape(bs, L, g, dg, 3), h)
    draw, dwf = _lib.dwconv_bwd(dfeat.reshape(bs, L, 3 * g * dg, 1), flat, wf)
    return y, draw.reshape(raw.shape), dwf, dh


def _cases():
    for shape in SHAPES:
        for dtype, filt in TYPES:
            yield pytest.param(*shape, dtype, filt, id="x".join(map(str, shape)) + f"-{str(dtype)[6:]}-{str(filt)[6:]}")


@pytest.mark.parametrize("bs,L,g,dg,hl,kf,dtype,filt", list(_cases()))
def test_against_oracle_and_chain(gcg_lib, bs, L, g, dg, hl, kf, dtype, filt):
    raw, wf, h, dy = make(bs, L, g, dg, hl, kf, dtype, filt)
    rd, wd, hd, dyd = (t.to(DEV) for t in (raw, wf, h, dy))
    y = _lib.mixer_mr_fwd(rd, wd, hd)
    draw, dwf, dh = _lib.mixer_mr_bwd(dyd, rd, wd, hd)
    torch.cuda.synchronize()
    assert y.shape == (bs, L, g, dg) and draw.shape == raw.shape and dwf.shape == wf.shape and dh.shape == h.shape
    assert y.dtype == dtype and draw.dtype == dtype and dwf.dtype == dtype and dh.dtype == filt
    # oracle twice: the featurizer is the gated oracle with both gates at one and one filter per feature channel
    flat = raw.float().reshape(bs, L, 3 * g * dg, 1)
    one = torch.ones_like(flat)
    f = oracle.gcg_fwd_oracle(flat, one, one, wf.float()).to(dtype).float().reshape(bs, L, g, dg, 3)
    C, B, x = f[..., 0], f[..., 1], f[..., 2]
    tol = TOL[dtype] if filt == dtype else 1.1 * 2.0 ** -8
    assert_close(y, oracle.gcg_fwd_oracle(x, B, C, h.float()), tol, "y")
    dx, dB, dC, dh_ref = oracle.gcg_bwd_oracle(dy.float(), x, B, C, h.float())
    assert_close(dh, dh_ref, TOL_DH[filt], "dh")
    dfeat = torch.stack([dC, dB, dx], dim=-1).to(dtype).float().reshape(bs, L, 3 * g * dg, 1)
    draw_ref, _, _, dwf_ref = oracle.gcg_bwd_oracle(dfeat, flat, one, one, wf.float())
    assert_close(draw.reshape(flat.shape), draw_ref, TOL[dtype], "draw")
    assert_close(dwf, dwf_ref, TOL_DH[dtype], "dwf")
    # the two-call chain: same arithmetic on the same values
    exact = dtype != torch.float16       # (f16: the featurizer's taps are summed in another grouping in the two kernels)
    one_kernel = filt == dtype and dtype != torch.float32      # the backward that never stores the gradient of the features
    for a, b, n in zip((y, draw, dwf, dh), chain(rd, wd, hd, dyd), ("y", "draw", "dwf", "dh")):
        if n == "dwf" and one_kernel:
            assert_close(a, b, TOL_DH[dtype], n)                # its partial sums are taken over other pieces of the rows
        elif exact and n != "dh":
            assert torch.equal(a, b), n
        elif n == "dh":
            assert_close(a, b, 1e-6 if filt == torch.float32 else TOL_DH[filt], n)     # other run lengths, other order of partial sums
        else:
            assert (a == b).float().mean().item() > 0.99 and torch.allclose(a.float(), b.float(), rtol=2e-3, atol=1e-3), n


def test_full_size_against_chain(gcg_lib):
    """The 7B layer shape (B=2, L=8192, D=4096, bf16): the one-kernel forward and backward against the chain of four
    kernels on the same values -- y, d raw and dh bit for bit, d wf up to the order of its partial sums."""
    gen = torch.Generator(device=DEV).manual_seed(3)
    bs, L, g, dg, hl, kf = 2, 8192, 256, 16, 128, 3
    raw = torch.randn(bs, L, g, dg, 3, generator=gen, device=DEV).to(torch.bfloat16)
    wf = (torch.randn(3 * g * dg, 1, kf, generator=gen, device=DEV) / kf ** 0.5).to(torch.bfloat16)
    h = (torch.randn(g, 1, hl, generator=gen, device=DEV) / hl ** 0.5).to(torch.bfloat16)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=DEV)).to(torch.bfloat16)
    y = _lib.mixer_mr_fwd(raw, wf, h)
    draw, dwf, dh = _lib.mixer_mr_bwd(dy, raw, wf, h)
    y_c, draw_c, dwf_c, dh_c = chain(raw, wf, h, dy)
    torch.cuda.synchronize()
    assert torch.equal(y, y_c), "y"
    assert torch.equal(draw, draw_c), "draw"
    assert_close(dh, dh_c, TOL_DH[torch.bfloat16], "dh")
    assert (dh == dh_c).float().mean().item() > 0.99, "dh"
    assert_close(dwf, dwf_c, TOL_DH[torch.bfloat16], "dwf")
    # every row of d raw was written: rows at run ends and at the sequence end take the other code paths
    assert torch.isfinite(draw.float()).all() and draw[:, -2:].float().abs().sum() > 0 and draw[:, 4094:4098].float().abs().sum() > 0


@pytest.mark.parametrize("dtype,filt", TYPES)
@pytest.mark.parametrize("bs,L,g,dg,hl,kf,lc", [(2, 700, 6, 16, 128, 3, 160), (1, 3000, 3, 64, 128, 3, 128),
                                                (2, 1100, 5, 32, 100, 2, 128)])
def test_filter_formed_in_the_kernels(gcg_lib, bs, L, g, dg, hl, kf, lc, dtype, filt):
    """gcg_mixer_mr_fwd_decay / _bwd_decay against the explicit-filter entry points given h = F(w * decay)[:, :hl]
    from gcg_filter_decay_fwd, and dw against gcg_filter_decay_bwd of their dh: bit for bit."""
    raw, wf, _, dy = (t.to(DEV) for t in make(bs, L, g, dg, hl, kf, dtype, filt, seed=5))
    gen = torch.Generator().manual_seed(6)
    w = (torch.randn(g, lc, generator=gen) / lc ** 0.5).to(DEV)
    decay = torch.exp(-torch.logspace(0, 2, g)[:, None] * torch.linspace(0, 1, lc)[None]).to(DEV)
    y = _lib.mixer_mr_fwd_decay(raw, wf, w, decay, hl, filt)
    draw, dwf, dw = _lib.mixer_mr_bwd_decay(dy, raw, wf, w, decay, hl, filt)
    h = _lib.filter_decay_fwd(w, decay, hl, filt)
    assert torch.equal(y, _lib.mixer_mr_fwd(raw, wf, h))
    draw2, dwf2, dh2 = _lib.mixer_mr_bwd(dy, raw, wf, h)
    torch.cuda.synchronize()
    assert torch.equal(draw, draw2) and torch.equal(dwf, dwf2)
    assert dw.shape == w.shape and torch.equal(dw, _lib.filter_decay_bwd(dh2, decay))
    if dtype == filt and dtype != torch.float32:
        # and on planar features (one-kernel path: 16-bit arithmetic)
        d = g * dg
        raw_pl = raw.permute(0, 1, 4, 2, 3).contiguous()
        wf_pl = wf.view(d, 3, 1, kf).permute(1, 0, 2, 3).reshape(3 * d, 1, kf).contiguous()
        y_pl = _lib.mixer_mr_fwd_decay(raw_pl, wf_pl, w, decay, hl, filt, planar=True)
        draw_pl, dwf_pl, dw_pl = _lib.mixer_mr_bwd_decay(dy, raw_pl, wf_pl, w, decay, hl, filt, planar=True)
        torch.cuda.synchronize()
        assert torch.equal(y_pl, y) and torch.equal(draw_pl, draw.permute(0, 1, 4, 2, 3)) and torch.equal(dw_pl, dw)
        assert torch.equal(dwf_pl.view(3, d, 1, kf), dwf.view(d, 3, 1, kf).permute(1, 0, 2, 3))


def test_refused_shapes(gcg_lib):
    raw, wf, h, dy = (t.to(DEV) for t in make(1, 64, 2, 8, 64, 3, torch.bfloat16, torch.bfloat16))
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.mixer_mr_fwd(raw, wf, h)                      # groups of 8 channels: less than a matrix tile
    raw, wf, h, dy = (t.to(DEV) for t in make(1, 64, 2, 16, 128, 4, torch.bfloat16, torch.bfloat16))
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.mixer_mr_bwd(dy, raw, wf, h)                  # four featurizer taps
    assert not _lib.mixer_mr_supported(8, 64, 3) and not _lib.mixer_mr_supported(16, 128, 4) and _lib.mixer_mr_supported(16, 128, 3)
    assert _lib.mixer_mr_supported(16, 64, 3) and not _lib.mixer_mr_supported(16, 7, 3)      # (Hyena-SE filters: gcg_mixer_se_*)


@pytest.mark.parametrize("act,cgcg", [(torch.bfloat16, "bfloat16"), (torch.float32, "float32"), (torch.bfloat16, "float32")])
def test_hyena_mixer_keeps_no_featurized_tensor(gcg_lib, act, cgcg):
    """HyenaMixer with a Hyena-MR operator: same output and gradients with and without the featurized tensor,
    and the fused path runs two large kernels (16-bit arithmetic; three with fp32 arithmetic, where the featurizer's
    backward is a kernel of its own) plus its small reductions."""
    from savanna_amd.operators.hyena import CgcgConfig, HyenaMROperator, HyenaMixer

    torch.manual_seed(0)
    bs, L, g, dg = 2, 384, 4, 16
    op = HyenaMROperator(g * dg, g, 128, CgcgConfig(cgcg_dtype=cgcg), small_init=False, device=DEV)
    mixer = HyenaMixer(op, 3, dtype=act, device=DEV)
    feats = torch.randn(bs, L, 3 * g * dg, device=DEV).to(act).requires_grad_(True)
    dz = (0.1 * torch.randn(bs, L, g * dg, device=DEV)).to(act)
    params = [op.filter.h, mixer.hyena_proj_conv.short_conv_weight]

    def run(fuse):
        mixer.fuse_medium = fuse
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
    for a, b, n in zip(got, want, ("z", "dfeatures", "dw", "dwf")):
        assert a.dtype == b.dtype, n
        if n == "dw":
            assert_close(a, b, 2e-5, n)
        elif n == "dwf" and cgcg == "bfloat16":
            assert_close(a, b, TOL_DH[act], n)
        else:
            assert torch.equal(a, b), n
    big = [e.key for e in prof.key_averages() if "mfma_il" in e.key or "dwconv" in e.key or "mixer_mr" in e.key]
    assert len(big) == (2 if cgcg == "bfloat16" else 3), big
    if cgcg == "bfloat16":       # filter, featurizer and operator: nothing else of the library's is launched
        ours = [e.key for e in prof.key_averages() if "gcg::" in e.key and e.device_time_total > 0]
        assert len(ours) == 2 and all("mixer_mr" in k for k in ours), ours


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("bs,L,g,dg,hl,kf", SHAPES)
def test_planar_features_match_interleaved(gcg_lib, bs, L, g, dg, hl, kf, dtype):
    """gcg_mixer_mr_fwd_planar / _bwd_planar -- raw (bs, L, 3, g, dg), the split without interleaving of
    block.py:881-884, with the featurizer's filters in that channel order -- give the interleaved entry points'
    results on the same values, bit for bit (the same arithmetic on pieces loaded plane by plane)."""
    raw, wf, h, dy = (t.to(DEV) for t in make(bs, L, g, dg, hl, kf, dtype, dtype, seed=23))
    d = g * dg
    raw_pl = raw.permute(0, 1, 4, 2, 3).contiguous()                                          # (bs, L, 3, g, dg)
    wf_pl = wf.view(d, 3, 1, kf).permute(1, 0, 2, 3).reshape(3 * d, 1, kf).contiguous()       # row p * d + c <- row 3 c + p
    y = _lib.mixer_mr_fwd(raw, wf, h)
    draw, dwf, dh = _lib.mixer_mr_bwd(dy, raw, wf, h)
    y_pl = _lib.mixer_mr_fwd(raw_pl, wf_pl, h, planar=True)
    draw_pl, dwf_pl, dh_pl = _lib.mixer_mr_bwd(dy, raw_pl, wf_pl, h, planar=True)
    torch.cuda.synchronize()
    assert y_pl.shape == y.shape and draw_pl.shape == raw_pl.shape and dwf_pl.shape == wf.shape
    assert torch.equal(y_pl, y)
    assert torch.equal(draw_pl, draw.permute(0, 1, 4, 2, 3))
    assert torch.equal(dwf_pl.view(3, d, 1, kf), dwf.view(d, 3, 1, kf).permute(1, 0, 2, 3))
    assert torch.equal(dh_pl, dh)


def test_planar_full_size(gcg_lib):
    """The same at the 7B layer shape."""
    bs, L, g, dg, hl, kf = 2, 8192, 256, 16, 128, 3
    gen = torch.Generator(device=DEV).manual_seed(3)
    raw = torch.randn(bs, L, g, dg, 3, generator=gen, device=DEV).to(torch.bfloat16)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=DEV)).to(torch.bfloat16)
    wf = (torch.randn(3 * g * dg, 1, kf, generator=gen, device=DEV) / kf ** 0.5).to(torch.bfloat16)
    h = (torch.randn(g, 1, hl, generator=gen, device=DEV) / hl ** 0.5).to(torch.bfloat16)
    d = g * dg
    raw_pl = raw.permute(0, 1, 4, 2, 3).contiguous()
    wf_pl = wf.view(d, 3, 1, kf).permute(1, 0, 2, 3).reshape(3 * d, 1, kf).contiguous()
    y = _lib.mixer_mr_fwd(raw, wf, h)
    draw, dwf, dh = _lib.mixer_mr_bwd(dy, raw, wf, h)
    y_pl = _lib.mixer_mr_fwd(raw_pl, wf_pl, h, planar=True)
    draw_pl, dwf_pl, dh_pl = _lib.mixer_mr_bwd(dy, raw_pl, wf_pl, h, planar=True)
    torch.cuda.synchronize()
    assert torch.equal(y_pl, y) and torch.equal(draw_pl, draw.permute(0, 1, 4, 2, 3)) and torch.equal(dh_pl, dh)
    assert torch.equal(dwf_pl.view(3, d, 1, kf), dwf.view(d, 3, 1, kf).permute(1, 0, 2, 3))


def test_planar_refused_for_fp32_arithmetic(gcg_lib):
    raw, wf, h, dy = (t.to(DEV) for t in make(1, 64, 2, 16, 128, 3, torch.float32, torch.float32))
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.mixer_mr_fwd(raw.permute(0, 1, 4, 2, 3).contiguous(), wf, h, planar=True)


def test_hyena_mixer_planar_fused(gcg_lib):
    """HyenaMixer(interleave_projections=False) with a Hyena-MR operator: one kernel each way, same output and
    gradients as the two-kernel chain on the same layout."""
    from savanna_amd.operators.hyena import CgcgConfig, HyenaMROperator, HyenaMixer

    torch.manual_seed(0)
    bs, L, g, dg = 2, 384, 4, 16
    op = HyenaMROperator(g * dg, g, 128, CgcgConfig(cgcg_dtype="bfloat16"), small_init=False, device=DEV)
    mixer = HyenaMixer(op, 3, dtype=torch.bfloat16, device=DEV, interleave_projections=False)
    feats = torch.randn(bs, L, 3 * g * dg, device=DEV).to(torch.bfloat16).requires_grad_(True)
    dz = (0.1 * torch.randn(bs, L, g * dg, device=DEV)).to(torch.bfloat16)
    params = [op.filter.h, mixer.hyena_proj_conv.short_conv_weight]

    def run(fuse):
        mixer.fuse_medium = fuse
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
    for a, b, n in zip(got, want, ("z", "dfeatures", "dw", "dwf")):
        if n == "dw":
            assert_close(a, b, 2e-5, n)
        elif n == "dwf":
            assert_close(a, b, TOL_DH[torch.bfloat16], n)
        else:
            assert torch.equal(a, b), n
    big = [e.key for e in prof.key_averages() if "mfma" in e.key or "dwconv" in e.key or "mixer_mr" in e.key]
    assert len(big) == 2 and all("mixer_mr" in k for k in big), big
    ours = [e.key for e in prof.key_averages() if "gcg::" in e.key and e.device_time_total > 0]
    assert len(ours) == 2, ours               # the filter is formed in the kernels on this layout too


@pytest.mark.parametrize("planar", [False, True], ids=["interleaved", "planar"])
def test_graph_replays_match_eager(gcg_lib, planar):
    """The fused forward and backward (explicit filter and filter formed in the kernels) recorded in a HIP graph: three
    replays on fresh data, with eager launches of the same kernels between them (the backward's arrival counters
    and partial sums are shared by every launch), each replay equal to eager bit for bit."""
    bs, L, g, dg, hl, kf, lc = 2, 2100, 6, 16, 128, 3, 128
    raw, wf, h, dy = (t.to(DEV) for t in make(bs, L, g, dg, hl, kf, torch.bfloat16, torch.bfloat16, seed=11))
    if planar:
        raw = raw.permute(0, 1, 4, 2, 3).contiguous()
    gen = torch.Generator().manual_seed(12)
    w = (torch.randn(g, lc, generator=gen) / lc ** 0.5).to(DEV)
    decay = torch.exp(-torch.logspace(0, 2, g)[:, None] * torch.linspace(0, 1, lc)[None]).to(DEV)

    def step(raw_, dy_):
        y = _lib.mixer_mr_fwd(raw_, wf, h, planar=planar)
        draw, dwf, dh = _lib.mixer_mr_bwd(dy_, raw_, wf, h, planar=planar)
        y2 = _lib.mixer_mr_fwd_decay(raw_, wf, w, decay, hl, torch.bfloat16, planar=planar)
        draw2, dwf2, dw = _lib.mixer_mr_bwd_decay(dy_, raw_, wf, w, decay, hl, torch.bfloat16, planar=planar)
        return y, draw, dwf, dh, y2, draw2, dwf2, dw

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):                      # warm-up on the capture stream
        step(raw, dy)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs_g = step(raw, dy)
    names = ("y", "d raw", "dw featurizer", "dh", "y decay", "d raw decay", "dw featurizer decay", "dw")
    for it in range(3):
        fresh_raw, fresh_dy = torch.randn_like(raw), 0.1 * torch.randn_like(dy)
        raw.copy_(fresh_raw)
        dy.copy_(fresh_dy)
        graph.replay()
        torch.cuda.synchronize()
        outs_e = step(fresh_raw, fresh_dy)
        torch.cuda.synchronize()
        for a, b, n in zip(outs_g, outs_e, names):
            assert torch.equal(a, b), f"replay {it}: {n}"
