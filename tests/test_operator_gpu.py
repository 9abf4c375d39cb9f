"""The drop-in path end to end on the GPU: operator module -> autograd function -> C ABI.
Mirrors tests/test_bwd_refactor.py:270-369 of the reference (the full
two_pass_chunked_gate_conv_gate autograd path against autograd of the F.conv1d form)."""
import pytest
import torch

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib, two_pass_chunked_gate_conv_gate
from savanna_amd.kernels.cgcg.src.kernel_utils import BwdKernelConfigRefactor, FwdKernelConfigRefactor
from savanna_amd.operators import hyena

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hl", [4, 7, 128])
@pytest.mark.parametrize("fused", [True, False])
def test_autograd_path(gcg_lib, hl, dtype, fused):
    bs, L, g, dg = 2, 1024, 8, 16
    gen = torch.Generator().manual_seed(hl)
    x, B, C = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(3))
    h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    dev = [t.to(DEV).requires_grad_(True) for t in (x, B, C, h)]
    cfg = FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row", num_warps=4, num_stages=3)
    y = two_pass_chunked_gate_conv_gate(*dev, bs, L, g, dg, fwd_autotune=False, bwd_autotune=not fused,
                                        fused_bwd=fused, fwd_kernel_cfg=cfg,
                                        bwd_kernel_cfg=BwdKernelConfigRefactor() if fused else None)
    assert y.shape == (bs, L, g, dg) and y.dtype == dtype
    y.backward(dy.to(DEV))
    y_ref = oracle.gcg_fwd_ref_torch(x.double(), B.double(), C.double(), h.double())
    grads_ref = oracle.gcg_bwd_ref_torch(dy, x, B, C, h)
    assert_close(y, y_ref, TOL[dtype], "y")
    for t, r, n in zip(dev, grads_ref, ("dx", "dB", "dC", "dh")):
        assert t.grad.shape == t.shape and t.grad.dtype == dtype
        assert_close(t.grad, r, TOL_DH[dtype] if n == "dh" else TOL[dtype], n)


def test_non_contiguous_inputs_are_accepted(gcg_lib):
    """The block hands the operator stride-3 views of the projected features
    (savanna/model/block.py:886-888); the boundary copies them (interface.py:51-54)."""
    torch.manual_seed(41)
    bs, L, g, dg = 1, 256, 4, 16
    feats = torch.randn(bs, L, g, 3, dg, device=DEV, dtype=torch.bfloat16)
    x1, x2, v = feats.unbind(3)
    assert not x1.is_contiguous()
    h = torch.randn(g, 1, 7, device=DEV, dtype=torch.bfloat16) * 0.3
    cfg = FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row")
    y = two_pass_chunked_gate_conv_gate(v, x2, x1, h, bs, L, g, dg, fwd_kernel_cfg=cfg)
    ref = oracle.gcg_fwd_oracle(v.float().cpu(), x2.float().cpu(), x1.float().cpu(), h.float().cpu())
    assert_close(y, ref, 1e-2, "y")


@pytest.mark.parametrize("kind", ["mr", "se"])
def test_operator_modules(gcg_lib, kind):
    b, l, g, dg = 2, 512, 8, 16
    gen = torch.Generator().manual_seed(1)
    x1, x2, v = (torch.randn(b, l, g, dg, generator=gen).to(torch.bfloat16).to(DEV) for _ in range(3))
    cfg = hyena.CgcgConfig(cgcg_dtype="bfloat16")
    if kind == "mr":
        op = hyena.HyenaMROperator(g * dg, g, hyena_mr_len=128, cfg=cfg, small_init=False)
    else:
        op = hyena.HyenaSEOperator(g * dg, g, hyena_se_len=7, cfg=cfg)
    op = op.to(DEV).to(torch.bfloat16)
    z = op(x1, x2, v)
    assert z.shape == (b, l, g * dg) and z.dtype == torch.bfloat16
    h = op._filter(l).detach()
    ref = oracle.gcg_fwd_oracle(v.float().cpu(), x2.float().cpu(), x1.float().cpu(), h.float().cpu())
    assert_close(z.reshape(b, l, g, dg), ref, 1e-2, "z")
    # the pre-gate pair is symmetric: swapping x2 and v changes nothing
    assert_close(op(x1, v, x2), z.float(), 2e-3, "swap")
    # gradients reach the filter parameters
    z.float().square().mean().backward()
    p = op.filter.h if kind == "mr" else op.short_conv_weight
    assert p.grad is not None and torch.isfinite(p.grad).all() and p.grad.abs().max() > 0
    # fp32 kernel dtype under bf16 activations: cast in, cast out (hyena.py:499-503, 533-534)
    op32 = hyena.HyenaSEOperator(g * dg, g, hyena_se_len=7, cfg=hyena.CgcgConfig(cgcg_dtype="float32")).to(DEV)
    z32 = op32(x1, x2, v)
    assert z32.dtype == torch.bfloat16


def test_preallocated_output(gcg_lib):
    from savanna_amd.kernels.cgcg.src.fwd import two_pass_fwd_grouped

    torch.manual_seed(83)
    bs, L, g, dg = 1, 128, 2, 16
    x, B, C = (torch.randn(bs, L, g, dg, device=DEV) for _ in range(3))
    h = torch.randn(g, 1, 7, device=DEV)
    buf = torch.full((bs, L, g * dg), float("nan"), device=DEV)
    bx, y2, y = two_pass_fwd_grouped(x, B, C, h, y=buf, autotune=False, CHUNK_SIZE=128, BLOCK_D=16)
    assert y.data_ptr() == buf.data_ptr() and torch.isfinite(buf).all()
    ref = oracle.gcg_fwd_oracle(x.cpu(), B.cpu(), C.cpu(), h.cpu(), return_intermediates=True)
    for got, want, n in zip((bx, y2, y), ref, ("bx", "y2", "y")):
        assert_close(got, want, 1e-5, n)


def test_runs_on_the_callers_stream(gcg_lib):
    """Kernels are enqueued on torch's current stream, not on the null stream."""
    from savanna_amd import _lib

    bs, L, g, dg, hl = 2, 2048, 16, 16, 128
    x, B, C, dy = (torch.randn(bs, L, g, dg, device=DEV, dtype=torch.bfloat16) for _ in range(4))
    h = (torch.randn(g, 1, hl, device=DEV) / hl ** 0.5).to(torch.bfloat16)
    _, _, y_ref = _lib.fwd(x, B, C, h)
    grads_ref = _lib.bwd(dy, x, B, C, h)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        # work queued on the side stream first: the convolution must wait for it, which it only
        # does when it is launched on the same stream
        x2 = x.clone()
        for _ in range(20):
            x2 = x2 * 1.0
        _, _, y = _lib.fwd(x2, B, C, h)
        grads = _lib.bwd(dy, x2, B, C, h)
    side.synchronize()
    assert torch.equal(y, y_ref)
    for a, b in zip(grads, grads_ref):
        assert torch.equal(a, b)


def test_backward_launches_overlap_on_streams(gcg_lib):
    """Backward launches in flight on four streams at once (each with its own inputs, outputs and workspace): every
    launch counts its workgroups' arrivals on a set of counters of its own, so each result equals the one computed
    alone, bit for bit -- the operator's kernel and the one-kernel Hyena-MR mixer."""
    bs, L, g, dg, hl, kf = 2, 4096, 16, 16, 128, 3
    dt = torch.bfloat16
    n = 4
    gen = torch.Generator(device=DEV).manual_seed(21)
    rnd = lambda *shape: torch.randn(*shape, device=DEV, generator=gen).to(dt)
    sets = [[rnd(bs, L, g, dg) for _ in range(4)] for _ in range(n)]                 # x, B, C, dy
    raws = [rnd(bs, L, g, dg, 3) for _ in range(n)]
    h = (torch.randn(g, 1, hl, device=DEV, generator=gen) / hl ** 0.5).to(dt)
    wf = (torch.randn(3 * g * dg, 1, kf, device=DEV, generator=gen) / kf ** 0.5).to(dt)
    alone = [(_lib.bwd(s[3], s[0], s[1], s[2], h), _lib.mixer_mr_bwd(s[3], r, wf, h)) for s, r in zip(sets, raws)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(n)]
    for rep in range(5):
        got = []
        for st, s, r in zip(streams, sets, raws):
            with torch.cuda.stream(st):
                got.append((_lib.bwd(s[3], s[0], s[1], s[2], h), _lib.mixer_mr_bwd(s[3], r, wf, h)))
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, alone)):
            for fam in range(2):
                for t, (u, v) in enumerate(zip(a[fam], b[fam])):
                    assert torch.equal(u, v), f"repeat {rep}, stream {i}, family {fam}, output {t}"


@pytest.mark.parametrize("hl,dtype", [(7, torch.float32), (128, torch.bfloat16)])
def test_graph_capture_and_replay(gcg_lib, hl, dtype):
    """The launch-bound small shapes are what a HIP graph is for: forward and backward are
    captured once and replayed with new input contents; every replay must equal the eager result.
    (The library itself allocates nothing and issues no memset; the tensors come from the
    capture's private pool.)"""
    from savanna_amd import _lib

    bs, L, g, dg = 1, 2048, 16, 16
    static = [torch.randn(bs, L, g, dg, device=DEV).to(dtype) for _ in range(4)]       # x, B, C, dy
    h = (torch.randn(g, 1, hl, device=DEV) / hl ** 0.5).to(dtype)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):                      # warm-up on the capture stream
        _lib.fwd(static[0], static[1], static[2], h)
        _lib.bwd(static[3], static[0], static[1], static[2], h)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _, _, y_g = _lib.fwd(static[0], static[1], static[2], h)
        grads_g = _lib.bwd(static[3], static[0], static[1], static[2], h)
    for it in range(3):
        fresh = [torch.randn(bs, L, g, dg, device=DEV).to(dtype) for _ in range(4)]
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        _, _, y_e = _lib.fwd(fresh[0], fresh[1], fresh[2], h)       # eager work between replays
        grads_e = _lib.bwd(fresh[3], fresh[0], fresh[1], fresh[2], h)
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_e), f"replay {it}: y"
        for a, b, n in zip(grads_g, grads_e, ("dx", "dB", "dC", "dh")):
            assert torch.equal(a, b), f"replay {it}: {n}"


@pytest.mark.parametrize("kind", ["mr", "se"])
def test_mixer_on_projected_features(gcg_lib, kind):
    """HyenaMixer (featurizer conv -> interleaved split -> operator) against the reference's chain
    written with torch ops: permute, F.pad + F.conv1d on (B, 3D, L), permute, the interleaved
    rearrange / unbind of block.py:886-888, and the operator on the three views."""
    import torch.nn.functional as F
    from einops import rearrange

    from savanna_amd.operators.hyena import CgcgConfig, HyenaMixer, HyenaMROperator, HyenaSEOperator

    torch.manual_seed(21)
    bs, L, hidden, groups = 2, 320, 128, 8
    cfg = CgcgConfig(cgcg_dtype="bfloat16")
    op = (HyenaMROperator(hidden, groups, 128, cfg, small_init=False, device=DEV) if kind == "mr"
          else HyenaSEOperator(hidden, groups, 7, cfg, device=DEV))
    mixer = HyenaMixer(op, 3, dtype=torch.bfloat16, device=DEV)
    feats = torch.randn(bs, L, 3 * hidden, device=DEV).to(torch.bfloat16)
    z = mixer(feats)
    assert z.shape == (bs, L, hidden)

    w = mixer.hyena_proj_conv.short_conv_weight.detach()
    f = F.conv1d(F.pad(feats.permute(0, 2, 1).float(), (2, 0)), w.float(), groups=3 * hidden)[..., :L]
    f = f.to(torch.bfloat16).permute(0, 2, 1)
    x1, x2, v = rearrange(f, "b l (g dg p) -> b l g p dg", p=3, g=groups).unbind(dim=3)
    z_ref = op(x1, x2, v)                       # the operator on the split views (checked against the oracle above)
    torch.cuda.synchronize()
    assert_close(z, z_ref, 1e-2, "z")


@pytest.mark.parametrize("repeat_interleave", [True, False])
def test_run_short_hyena_layout(gcg_lib, repeat_interleave):
    """run_short_hyena on (seqlen, bs, g, dg) inputs against the reference's own statement of that
    operator (short_hyena/utils.py:36-66: rearrange to (bs, d, seqlen), F.conv1d with padding K-1 on
    both sides trimmed to seqlen, times q, rearranged to (bs, g, seqlen, dg)), with gradients."""
    import torch.nn.functional as F
    from einops import rearrange

    from savanna_amd.kernels.short_hyena import run_short_hyena

    seqlen, bs, g, dg, hl = 96, 2, 4, 16, 3
    gen = torch.Generator().manual_seed(31)
    q, k, v = (torch.randn(seqlen, bs, g, dg, generator=gen) for _ in range(3))
    w = torch.randn(g if repeat_interleave else g * dg, 1, hl, generator=gen) / hl ** 0.5
    dy = 0.1 * torch.randn(bs, g, seqlen, dg, generator=gen)

    dev = [t.to(DEV).requires_grad_(True) for t in (q, k, v, w)]
    out = run_short_hyena(*dev, repeat_interleave=repeat_interleave, autotune=True)
    assert out.shape == (bs, g, seqlen, dg)
    out.backward(dy.to(DEV))

    ref_in = [t.double().requires_grad_(True) for t in (q, k, v, w)]
    rq, rk, rv, rw = ref_in
    wd = rw.repeat_interleave(dg, dim=0) if repeat_interleave else rw
    kv = rearrange(rk * rv, "s b g d -> b (g d) s")
    conv = F.conv1d(kv, wd, bias=None, stride=1, padding=hl - 1, groups=g * dg)[..., :seqlen]
    ref = rearrange(conv * rearrange(rq, "s b g d -> b (g d) s"), "b (g d) s -> b g s d", g=g)
    ref.backward(dy.double())
    torch.cuda.synchronize()
    assert_close(out, ref, TOL[torch.float32], "out")
    for a, r, n in zip(dev, ref_in, ("dq", "dk", "dv", "dw")):
        assert_close(a.grad, r.grad, TOL_DH[torch.float32] if n == "dw" else TOL[torch.float32], n)
    with pytest.raises(AssertionError, match="Must specify"):
        run_short_hyena(*dev)


@pytest.mark.parametrize("seqlen,bs,g,dg,hl,dtype", [
    (8192, 16, 48, 16, 7, torch.bfloat16),     # the reference's own case: d_model 768, group size 16, kernel 7
    (1000, 3, 5, 20, 4, torch.float32),        # ragged length, odd batch, dg not a power of two
    (513, 2, 6, 16, 8, torch.float16),
    (300, 4, 3, 32, 5, "bf16-fp32"),           # bf16 tensors with an fp32 filter
], ids=["ref-shape-bf16", "ragged-f32", "f16", "bf16-fp32-filter"])
def test_run_short_hyena_in_place(gcg_lib, seqlen, bs, g, dg, hl, dtype):
    """run_short_hyena reads (seqlen, bs, g, dg) operands where they lie: the reference's test shape
    (tests/model/test_kernels.py:133-137, seqlen 8192, bs 16, d_model 768 in groups of 16, 7 taps, bf16), against
    the oracle on whole filter groups, and a kernel trace without any copy or permute kernel."""
    from savanna_amd.kernels.short_hyena import run_short_hyena

    mixed = dtype == "bf16-fp32"
    tdt = torch.bfloat16 if mixed else dtype
    gen = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(seqlen, bs, g, dg, generator=gen).to(tdt) for _ in range(3))
    w = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(torch.float32 if mixed else tdt)
    dy = (0.1 * torch.randn(bs, seqlen, g, dg, generator=gen)).to(tdt)
    dev = [t.to(DEV).requires_grad_(True) for t in (q, k, v, w)]
    dyd = dy.to(DEV)
    from torch.profiler import ProfilerActivity, profile
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        out = run_short_hyena(*dev, autotune=True)
        out.backward(dyd.permute(0, 2, 1, 3))          # a gradient laid out like the kernel's own result
        torch.cuda.synchronize()
    assert out.shape == (bs, g, seqlen, dg)
    names = [e.key for e in prof.key_averages() if e.device_time_total > 0 and "Memcpy" not in e.key and "Memset" not in e.key]
    assert all("gcg::" in n for n in names) and len(names) == 3, names     # forward, backward, filter-gradient reduction
    # oracle on a few whole filter groups of every batch entry (the operator is independent across groups)
    gs = sorted({0, g // 2, g - 1})
    to_blgd = lambda t: t[:, :, gs].permute(1, 0, 2, 3).float()
    ref_y = oracle.gcg_fwd_oracle(to_blgd(v), to_blgd(k), to_blgd(q), w[gs].float())
    ref = oracle.gcg_bwd_oracle(dy[:, :, gs].float(), to_blgd(v), to_blgd(k), to_blgd(q), w[gs].float())
    tol = 1.1 * 2.0 ** -8 if mixed else TOL[tdt]
    assert_close(out.permute(0, 2, 1, 3)[:, :, gs], ref_y, tol, "out")
    for a, r, n in zip((dev[2], dev[1], dev[0]), ref[:3], ("dv", "dk", "dq")):
        assert a.grad.shape == (seqlen, bs, g, dg) and a.grad.is_contiguous()
        assert_close(a.grad[:, :, gs].permute(1, 0, 2, 3), r, tol, n)
    assert dev[3].grad.dtype == w.dtype
    assert_close(dev[3].grad[gs], ref[3], TOL_DH[w.dtype], "dw")
    # and bit for bit what the batch-major kernels give on permuted copies
    x_, B_, C_ = (t.detach().permute(1, 0, 2, 3).contiguous() for t in (dev[2], dev[1], dev[0]))
    _, _, y2 = _lib.fwd(x_, B_, C_, dev[3].detach(), algo="window")
    assert torch.equal(out.permute(0, 2, 1, 3), y2)
    dx2, dB2, dC2, dh2 = _lib.bwd(dyd, x_, B_, C_, dev[3].detach(), algo="window")
    assert torch.equal(dev[2].grad.permute(1, 0, 2, 3), dx2) and torch.equal(dev[0].grad.permute(1, 0, 2, 3), dC2)
    assert torch.equal(dev[3].grad, dh2)


def test_time_major_64bit_offsets(gcg_lib):
    """(seqlen, bs, g, dg) operands of 2^31 elements each (seqlen 2^18, bs 2, 4096 channels, bf16): a filter that
    delays by two rows makes every output a product of input elements, so a wrapped offset fails an exact comparison."""
    seqlen, bs, g, dg, hl, s_ = 1 << 18, 2, 256, 16, 7, 2
    dt = torch.bfloat16
    gen = torch.Generator(device=DEV)
    tensors = []
    for i in range(4):                                  # x, B, C (seqlen, bs, g, dg); dy (bs, seqlen, g, dg)
        t = torch.empty((seqlen, bs, g, dg) if i < 3 else (bs, seqlen, g, dg), dtype=dt, device=DEV)
        flat = t.view(-1)
        for k, o in enumerate(range(0, flat.numel(), 1 << 28)):
            gen.manual_seed(500 + 10 * i + k)
            flat[o:o + (1 << 28)].normal_(generator=gen)
        tensors.append(t)
    x, B, C, dy = tensors
    h = torch.zeros(g, 1, hl, dtype=dt, device=DEV)
    h[:, 0, hl - 1 - s_] = 1.0
    y = _lib.fwd_time_major(x, B, C, h)           # (bs, seqlen, g, dg)
    torch.cuda.synchronize()
    u = x.float() * B.float()                           # exact in fp32; these kernels keep it there
    want = torch.zeros_like(x)
    want[s_:] = (C[s_:].float() * u[:-s_]).to(dt)
    assert torch.equal(y, want.permute(1, 0, 2, 3)), "y"
    del y
    dx, dB, dC, dh = _lib.bwd_time_major(dy, x, B, C, h)
    torch.cuda.synchronize()
    assert torch.isfinite(dh.float()).all()
    dyt = dy.permute(1, 0, 2, 3)
    want.zero_()
    want[s_:] = (dyt[s_:].float() * u[:-s_]).to(dt)
    assert torch.equal(dC, want), "dC"
    del u
    g2 = dyt.float() * C.float()
    want.zero_()
    want[:-s_] = (g2[s_:] * x[:-s_].float()).to(dt)
    assert torch.equal(dB, want), "dB"
    want.zero_()
    want[:-s_] = (g2[s_:] * B[:-s_].float()).to(dt)
    assert torch.equal(dx, want), "dx"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "f16"])
def test_decayed_filter_in_one_launch(gcg_lib, dtype):
    """gcg_filter_decay_fwd / _bwd against the expression of explicit.py:68-75 followed by the
    [:, None] and cast of hyena.py:440-441, :499-503, with autograd for the backward."""
    from savanna_amd.operators.hyena import ExplicitSingleDecayFilter

    g, l_cache, hl = 24, 160, 128
    torch.manual_seed(41)
    f = ExplicitSingleDecayFilter(g, l_cache, small_init=False, device=DEV)
    h = f.fused(hl, dtype)
    assert h.shape == (g, 1, hl) and h.dtype == dtype
    dh = torch.randn(g, 1, hl, device=DEV).to(dtype)
    h.backward(dh)
    got_dw = f.h.grad.clone()
    f.h.grad = None
    h_ref = (f.h[:, :hl] * f.decay[:, :hl])[:, None].to(dtype)
    h_ref.backward(dh)
    assert torch.equal(h, h_ref)
    assert_close(got_dw, f.h.grad, 1e-6, "dw")
    assert not got_dw[:, hl:].any()


@pytest.mark.parametrize("hl,dtype", [(7, torch.float32), (128, torch.bfloat16)])
def test_graph_capture_of_the_feature_chain(gcg_lib, hl, dtype):
    """Featurizer conv, interleaved operator and their backwards captured in one HIP graph and
    replayed with new contents; every replay must equal the eager result."""
    from savanna_amd import _lib

    bs, L, g, dg = 1, 1024, 8, 16
    raw = torch.randn(bs, L, 3 * g * dg, 1, device=DEV).to(dtype)
    dy = torch.randn(bs, L, g, dg, device=DEV).to(dtype)
    wf = (torch.randn(3 * g * dg, 1, 3, device=DEV) / 3 ** 0.5).to(dtype)
    h = (torch.randn(g, 1, hl, device=DEV) / hl ** 0.5).to(dtype)

    def chain(raw_t, dy_t):
        f = _lib.dwconv_fwd(raw_t, wf)
        feat = f.view(bs, L, g, dg, 3)
        y = _lib.fwd_interleaved(feat, h)
        dfeat, dh = _lib.bwd_interleaved(dy_t, feat, h)
        draw, dwf = _lib.dwconv_bwd(dfeat.view(bs, L, 3 * g * dg, 1), raw_t, wf)
        return y, dh, draw, dwf

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        chain(raw, dy)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs_g = chain(raw, dy)
    for it in range(3):
        fresh_raw, fresh_dy = torch.randn_like(raw), torch.randn_like(dy)
        raw.copy_(fresh_raw)
        dy.copy_(fresh_dy)
        graph.replay()
        torch.cuda.synchronize()
        outs_e = chain(fresh_raw, fresh_dy)
        torch.cuda.synchronize()
        for a, b, n in zip(outs_g, outs_e, ("y", "dh", "d raw", "dw featurizer")):
            assert torch.equal(a, b), f"replay {it}: {n}"
