"""The operator on planar operands: x1, x2, v as the thirds of the rows of one projected-features tensor, the split
without interleaving of savanna/model/block.py:881-884 (``interleave_projections = false``), read without the three
gathers of cgcg/interface.py:51-54.  Checked against the CPU oracle, against the entry points on separate tensors
(same kernels, so bit for bit), and through the reference's own split expression.
"""
import pytest
import torch
from einops import rearrange

import oracle
from helpers import TOL, TOL_DH, assert_close, inputs, oracle_bwd, oracle_fwd
from savanna_amd import _lib
from savanna_amd.kernels.cgcg import interface
from savanna_amd.kernels.cgcg.interface import (
    two_pass_chunked_gate_conv_gate,
    two_pass_chunked_gate_conv_gate_planar,
)
from savanna_amd.kernels.cgcg.src.kernel_utils import BwdKernelConfigRefactor, FwdKernelConfigRefactor
from test_parity_gpu import DTYPES, SMALL, algos_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def pack(x, B, C):
    """(bs, L, 3, g, dg) with [:, :, 0] = C, [:, :, 1] = B, [:, :, 2] = x."""
    return torch.stack([C, B, x], dim=2).contiguous()


def _cases():
    for shape in SMALL:
        bs, L, g, dg, hl = shape
        for dtype in DTYPES:
            for algo in algos_for(hl, dg, dtype):
                yield pytest.param(*shape, dtype, algo, id=f"{bs}x{L}x{g}x{dg}-hl{hl}-{str(dtype)[6:]}-{algo}")


def same_kernel_family(hl, algo):
    """The planar matrix-core kernels always walk five slices of the banded matrix; the separate-tensor entry point
    picks fewer for a short filter, and the zero slices then group the fp32 sums of dh differently."""
    return algo != "mfma" or hl >= 98


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype,algo", list(_cases()))
def test_fwd_planar_small(gcg_lib, bs, L, g, dg, hl, dtype, algo):
    x, B, C, h, _ = inputs(bs, L, g, dg, hl, dtype, seed=4)
    _, _, y_ref = oracle_fwd(x, B, C, h)
    xd, Bd, Cd, hd = (t.to(DEV) for t in (x, B, C, h))
    y = _lib.fwd_planar(pack(xd, Bd, Cd), hd, algo=algo)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == (bs, L, g, dg)
    assert_close(y, y_ref, TOL[dtype], "y")
    _, _, y_plain = _lib.fwd(xd, Bd, Cd, hd, algo=algo)
    assert torch.equal(y, y_plain), "y: planar and separate-tensor results differ"


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype,algo", list(_cases()))
def test_bwd_planar_small(gcg_lib, bs, L, g, dg, hl, dtype, algo):
    x, B, C, h, dy = inputs(bs, L, g, dg, hl, dtype, seed=5, dy_scale=0.1)
    ref = oracle_bwd(dy, x, B, C, h)
    xd, Bd, Cd, hd, dyd = (t.to(DEV) for t in (x, B, C, h, dy))
    dfeat, dh = _lib.bwd_planar(dyd, pack(xd, Bd, Cd), hd, algo=algo)
    torch.cuda.synchronize()
    assert dfeat.shape == (bs, L, 3, g, dg) and dfeat.dtype == dtype and dh.shape == h.shape
    plain = _lib.bwd(dyd, xd, Bd, Cd, hd, algo=algo)
    got = (dfeat[:, :, 2], dfeat[:, :, 1], dfeat[:, :, 0], dh)
    few_terms = algo == "mfma" and bs * L * dg < 256     # see test_parity_gpu.test_bwd_small
    for o, p, r, n in zip(got, plain, ref, ("dx", "dB", "dC", "dh")):
        if n == "dh" and not same_kernel_family(hl, algo):
            assert_close(o, p, TOL_DH[dtype], "dh (planar vs separate tensors)")
        else:
            assert torch.equal(o, p), f"{n}: planar and separate-tensor results differ"
        if not (n == "dh" and few_terms):
            assert_close(o, r, TOL_DH[dtype] if n == "dh" else TOL[dtype], n)


def _cfgs():
    return (FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row"),
            BwdKernelConfigRefactor(pre_conv_BLOCK_X=128, pre_conv_BLOCK_Y=128, pre_conv_num_warps=4,
                                    post_conv_BLOCK_X=32, post_conv_BLOCK_Y=128, post_conv_num_warps=4))


@pytest.mark.parametrize("hl,dtype", [(7, torch.float32), (128, torch.bfloat16), (7, torch.bfloat16)],
                         ids=["se-f32", "mr-bf16", "se-bf16"])
def test_reference_split_views_take_the_planar_path(gcg_lib, monkeypatch, hl, dtype):
    """features -> rearrange("b l (p g dg) -> b l p g dg").unbind(2) exactly as block.py:881-884 -> the operator with
    the argument mapping of hyena.py:517-531 (x=v, B=x2, C=x1).  The three views must reach the planar entry points
    (no gathers), and forward and feature gradient must match the library formulation on gathered copies."""
    bs, L, g, dg = 2, 384, 4, 16
    gen = torch.Generator().manual_seed(11)
    feat_cpu = torch.randn(bs, L, 3 * g * dg, generator=gen).to(dtype)
    h_cpu = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype)
    dy_cpu = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)

    calls = {"fwd": 0, "bwd": 0, "plain": 0}
    real_f, real_b, real_p = _lib.fwd_planar, _lib.bwd_planar, _lib.fwd
    monkeypatch.setattr(interface._lib, "fwd_planar",
                        lambda *a, **k: (calls.__setitem__("fwd", calls["fwd"] + 1), real_f(*a, **k))[1])
    monkeypatch.setattr(interface._lib, "bwd_planar",
                        lambda *a, **k: (calls.__setitem__("bwd", calls["bwd"] + 1), real_b(*a, **k))[1])
    monkeypatch.setattr(interface._lib, "fwd",
                        lambda *a, **k: (calls.__setitem__("plain", calls["plain"] + 1), real_p(*a, **k))[1])

    features = feat_cpu.to(DEV).requires_grad_(True)
    hd = h_cpu.to(DEV).requires_grad_(True)
    x1, x2, v = rearrange(features, "b l (p g dg) -> b l p g dg", p=3, g=g).unbind(dim=2)
    fwd_cfg, bwd_cfg = _cfgs()
    z = two_pass_chunked_gate_conv_gate(x=v, B=x2, C=x1, h=hd, bs=bs, seqlen=L, g=g, dg=dg,
                                        fwd_autotune=False, bwd_autotune=False, fused_bwd=True,
                                        fwd_kernel_cfg=fwd_cfg, bwd_kernel_cfg=bwd_cfg)
    z.backward(dy_cpu.to(DEV))
    torch.cuda.synchronize()
    assert calls == {"fwd": 1, "bwd": 1, "plain": 0}

    f32 = feat_cpu.float().requires_grad_(True)
    h32 = h_cpu.float().requires_grad_(True)
    a1, a2, av = rearrange(f32, "b l (p g dg) -> b l p g dg", p=3, g=g).unbind(dim=2)
    z_ref = oracle.gcg_fwd_ref_torch(av.contiguous(), a2.contiguous(), a1.contiguous(), h32)
    z_ref.backward(dy_cpu.float())
    assert_close(z, z_ref, TOL[dtype], "z")
    assert_close(features.grad, f32.grad, TOL[dtype], "d features")
    assert_close(hd.grad, h32.grad, TOL_DH[dtype], "dh")


def test_features_entry_point(gcg_lib):
    """two_pass_chunked_gate_conv_gate_planar(features, h): same result and gradients as the operator on gathered
    copies of the split views."""
    bs, L, g, dg, hl, dtype = 1, 512, 8, 16, 128, torch.bfloat16
    gen = torch.Generator().manual_seed(12)
    feat = torch.randn(bs, L, 3 * g * dg, generator=gen).to(dtype).to(DEV)
    h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype).to(DEV)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype).to(DEV)

    fa, ha = feat.clone().requires_grad_(True), h.clone().requires_grad_(True)
    za = two_pass_chunked_gate_conv_gate_planar(fa, ha, bs, L, g, dg)
    za.backward(dy)

    fb, hb = feat.clone().requires_grad_(True), h.clone().requires_grad_(True)
    x1, x2, v = rearrange(fb, "b l (p g dg) -> b l p g dg", p=3, g=g).unbind(dim=2)
    fwd_cfg, bwd_cfg = _cfgs()
    zb = two_pass_chunked_gate_conv_gate(v.contiguous(), x2.contiguous(), x1.contiguous(), hb, bs, L, g, dg,
                                         fwd_kernel_cfg=fwd_cfg, bwd_kernel_cfg=bwd_cfg, bwd_autotune=False)
    zb.backward(dy)
    torch.cuda.synchronize()
    assert torch.equal(za, zb)
    assert torch.equal(fa.grad, fb.grad)
    assert torch.equal(ha.grad, hb.grad)


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype", [
    (2, 8192, 256, 16, 128, torch.bfloat16),     # Hyena-MR, 7B layer shape
    (1, 32768, 512, 16, 7, torch.bfloat16),      # Hyena-SE, 40B layer shape
    (1, 8192, 256, 16, 128, torch.float32),
    (1, 4096, 512, 16, 7, torch.float32),
], ids=["mr-7b-bf16", "se-40b-bf16", "mr-f32", "se-f32"])
def test_benchmark_shapes_match_separate_tensors(gcg_lib, bs, L, g, dg, hl, dtype):
    """Every element of y, d features and dh equals what the separate-tensor entry points give (those are checked
    against the oracle at these shapes in test_fullsize_gpu.py)."""
    gen = torch.Generator(device=DEV).manual_seed(13)
    feat = torch.randn(bs, L, 3, g, dg, generator=gen, device=DEV).to(dtype)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=DEV)).to(dtype)
    h = (torch.randn(g, 1, hl, generator=gen, device=DEV) / hl ** 0.5).to(dtype)
    y = _lib.fwd_planar(feat, h)
    dfeat, dh = _lib.bwd_planar(dy, feat, h)
    C, B, x = (feat[:, :, i].contiguous() for i in range(3))
    _, _, y_p = _lib.fwd(x, B, C, h)
    dx, dB, dC, dh_p = _lib.bwd(dy, x, B, C, h)
    torch.cuda.synchronize()
    assert torch.equal(y, y_p)
    assert torch.equal(dfeat[:, :, 0], dC) and torch.equal(dfeat[:, :, 1], dB) and torch.equal(dfeat[:, :, 2], dx)
    assert torch.equal(dh, dh_p)


def test_planar_64bit_offsets(gcg_lib):
    """3 * 2^31 feature elements: flat offsets into the planar tensor pass 2^32."""
    bs, L, g, dg, hl, dtype = 1, 1 << 19, 256, 16, 128, torch.bfloat16
    feat = torch.empty(bs, L, 3, g, dg, dtype=dtype, device=DEV)
    gen = torch.Generator(device=DEV)
    for s, t0 in enumerate(range(0, L, 1 << 16)):
        gen.manual_seed(100 + s)
        feat[:, t0:t0 + (1 << 16)].normal_(generator=gen)
    h = torch.zeros(g, 1, hl, dtype=dtype, device=DEV)
    h[:, 0, hl - 1 - 5] = 1.0                          # y[t] = C[t] * (B*x)[t-5], exactly
    y = _lib.fwd_planar(feat, h)
    torch.cuda.synchronize()
    u = (feat[:, :, 1].float() * feat[:, :, 2].float()).to(dtype)
    want = torch.zeros_like(y)
    want[:, 5:] = (feat[:, 5:, 0].float() * u[:, :-5].float()).to(dtype)
    assert torch.equal(y, want)
    del u, want, y


@pytest.mark.parametrize("kind", ["mr", "se"])
def test_mixer_without_interleaving(gcg_lib, kind):
    """HyenaMixer(interleave_projections=False) against the reference's chain written with torch ops: permute,
    F.pad + F.conv1d on (B, 3D, L), permute, the split of block.py:881-884, and the operator on the three views."""
    import torch.nn.functional as F

    from savanna_amd.operators.hyena import CgcgConfig, HyenaMixer, HyenaMROperator, HyenaSEOperator

    torch.manual_seed(21)
    bs, L, hidden, groups = 2, 320, 128, 8
    cfg = CgcgConfig(cgcg_dtype="bfloat16")
    op = (HyenaMROperator(hidden, groups, 128, cfg, small_init=False, device=DEV) if kind == "mr"
          else HyenaSEOperator(hidden, groups, 7, cfg, device=DEV))
    mixer = HyenaMixer(op, 3, dtype=torch.bfloat16, device=DEV, interleave_projections=False)
    feats = torch.randn(bs, L, 3 * hidden, device=DEV).to(torch.bfloat16).requires_grad_(True)
    dz = (0.1 * torch.randn(bs, L, hidden, device=DEV)).to(torch.bfloat16)
    z = mixer(feats)
    assert z.shape == (bs, L, hidden)
    z.backward(dz)
    got = [z.detach(), feats.grad.clone()] + [p.grad.clone() for p in mixer.parameters()]

    feats.grad = None
    for p in mixer.parameters():
        p.grad = None
    w = mixer.hyena_proj_conv.short_conv_weight
    f = F.conv1d(F.pad(feats.permute(0, 2, 1).float(), (2, 0)), w.float(), groups=3 * hidden)[..., :L]
    f = f.to(torch.bfloat16).permute(0, 2, 1)
    x1, x2, v = rearrange(f, "b l (p g dg) -> b l p g dg", p=3, g=groups).unbind(dim=2)
    z_ref = op(x1, x2, v)
    z_ref.backward(dz)
    torch.cuda.synchronize()
    want = [z_ref.detach(), feats.grad.clone()] + [p.grad.clone() for p in mixer.parameters()]
    for a, b, n in zip(got, want, ["z", "d features"] + [n for n, _ in mixer.named_parameters()]):
        assert_close(a, b, 2e-2 if n != "z" else 1e-2, n)


@pytest.mark.parametrize("kind", ["mr", "se"])
def test_operator_modules_read_planar_views_in_place(gcg_lib, monkeypatch, kind):
    """HyenaMROperator / HyenaSEOperator called as ParallelSequenceMixer does, on the three views of the split
    without interleaving: the planar kernels run (no gathers), for Hyena-MR with its filter from one small launch."""
    from savanna_amd.operators.hyena import CgcgConfig, HyenaMROperator, HyenaSEOperator

    calls = {"planar": 0, "plain": 0, "decay": 0}
    real_pl, real_p, real_d = _lib.fwd_planar, _lib.fwd, _lib.fwd_decay
    monkeypatch.setattr(interface._lib, "fwd_planar",
                        lambda *a, **k: (calls.__setitem__("planar", calls["planar"] + 1), real_pl(*a, **k))[1])
    monkeypatch.setattr(interface._lib, "fwd",
                        lambda *a, **k: (calls.__setitem__("plain", calls["plain"] + 1), real_p(*a, **k))[1])
    monkeypatch.setattr(interface._lib, "fwd_decay",
                        lambda *a, **k: (calls.__setitem__("decay", calls["decay"] + 1), real_d(*a, **k))[1])
    torch.manual_seed(5)
    bs, L, hidden, groups = 2, 256, 128, 8
    cfg = CgcgConfig(cgcg_dtype="bfloat16")
    op = (HyenaMROperator(hidden, groups, 128, cfg, small_init=False, device=DEV) if kind == "mr"
          else HyenaSEOperator(hidden, groups, 7, cfg, device=DEV))
    feats = torch.randn(bs, L, 3 * hidden, device=DEV).to(torch.bfloat16)
    x1, x2, v = rearrange(feats, "b l (p g dg) -> b l p g dg", p=3, g=groups).unbind(dim=2)
    z = op(x1, x2, v)
    z_ref = op(x1.contiguous(), x2.contiguous(), v.contiguous())
    torch.cuda.synchronize()
    assert calls["planar"] == 1 and calls["plain"] + calls["decay"] == 1, calls
    assert torch.equal(z, z_ref)


@pytest.mark.parametrize("act", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("hl,algo", [(128, "mfma"), (64, "mfma"), (7, "window"), (7, "direct")])
def test_planar_with_fp32_arithmetic(gcg_lib, act, hl, algo):
    """16-bit planar features with an fp32 filter (fp32 arithmetic inside, cgcg_dtype float32 on 16-bit activations):
    the same results as on gathered copies."""
    bs, L, g, dg = 2, 700, 5, 16
    x, B, C, h, dy = inputs(bs, L, g, dg, hl, act, seed=8, dy_scale=0.1)
    h = h.float()
    xd, Bd, Cd, hd, dyd = (t.to(DEV) for t in (x, B, C, h, dy))
    feat = pack(xd, Bd, Cd)
    y = _lib.fwd_planar(feat, hd, algo=algo)
    dfeat, dh = _lib.bwd_planar(dyd, feat, hd, algo=algo)
    _, _, y_p = _lib.fwd(xd, Bd, Cd, hd, algo=algo)
    dx, dB, dC, dh_p = _lib.bwd(dyd, xd, Bd, Cd, hd, algo=algo)
    torch.cuda.synchronize()
    assert y.dtype == act and dh.dtype == torch.float32
    assert torch.equal(y, y_p)
    assert torch.equal(dfeat[:, :, 0], dC) and torch.equal(dfeat[:, :, 1], dB) and torch.equal(dfeat[:, :, 2], dx)
    if same_kernel_family(hl, algo):
        assert torch.equal(dh, dh_p)
    else:
        assert_close(dh, dh_p, 2e-5, "dh")


@pytest.mark.parametrize("bs,L,g,dg,hl,dtype", [(3, 2106, 25, 4, 3, torch.bfloat16), (2, 31, 15, 4, 5, torch.float16),
                                                (2, 1000, 23, 4, 7, torch.float16), (1, 300, 31, 4, 6, torch.float32)])
def test_planes_eight_bytes_apart(gcg_lib, bs, L, g, dg, hl, dtype):
    """d * element size not a multiple of 16: the planes are only 8-byte aligned, which the register-window kernels
    take (their rows are no better aligned on separate tensors of that width): same kernels, same results."""
    x, B, C, h, dy = (t.to(DEV) for t in inputs(bs, L, g, dg, hl, dtype, seed=3, dy_scale=0.1))
    feat = pack(x, B, C)
    y = _lib.fwd_planar(feat, h, algo="window")
    dfeat, dh = _lib.bwd_planar(dy, feat, h, algo="window")
    _, _, y_p = _lib.fwd(x, B, C, h, algo="window")
    dx, dB, dC, dh_p = _lib.bwd(dy, x, B, C, h, algo="window")
    torch.cuda.synchronize()
    assert torch.equal(y, y_p) and torch.equal(dh, dh_p)
    assert torch.equal(dfeat[:, :, 0], dC) and torch.equal(dfeat[:, :, 1], dB) and torch.equal(dfeat[:, :, 2], dx)
