"""The ungated short causal depthwise convolution (featurizer): gcg_dwconv_fwd / gcg_dwconv_bwd
through the C ABI against the CPU oracle (the gated operator with both gates at one), against
F.conv1d phrased exactly as ParallelCausalDepthwiseConv1d.forward does it
(savanna/model/operators/hyena/hyena.py:136-176), and composed with the interleaved operator."""
import pytest
import torch
import torch.nn.functional as F
from einops import rearrange

import oracle
from helpers import TOL, TOL_DH, assert_close
from savanna_amd import _lib
from savanna_amd.kernels.cgcg.interface import two_pass_chunked_gate_conv_gate_interleaved
from savanna_amd.operators.hyena import CausalDepthwiseConv1d

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]

# (bs, L, g, dg, hl): per-channel filters (dg = 1) and shared ones, ragged lengths, single rows
SHAPES = [
    (2, 64, 48, 1, 3),        # the featurizer: one 3-tap filter per channel
    (1, 300, 12, 1, 3),
    (2, 77, 8, 1, 4),
    (1, 1, 16, 1, 3),
    (1, 5, 4, 1, 7),
    (2, 130, 3, 4, 3),        # filters shared by 4 channels
    (1, 513, 2, 16, 7),
    (1, 200, 6, 8, 8),
    (1, 1000, 100, 1, 5),
    (3, 129, 1, 64, 1),       # single tap
]


def data(bs, L, g, dg, hl, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(bs, L, g, dg, generator=gen).to(dtype)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    w = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype)
    return x, dy, w


def conv_as_reference(x_bdl, weight_d1k):
    """hyena.py:139,159,168-175: left pad K-1, F.conv1d with one group per channel, keep L samples."""
    K = weight_d1k.shape[-1]
    L = x_bdl.shape[-1]
    xp = F.pad(x_bdl, (K - 1, 0))
    return F.conv1d(xp, weight_d1k, bias=None, stride=1, padding=0, groups=x_bdl.shape[1])[..., :L]


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("bs,L,g,dg,hl", SHAPES)
def test_dwconv_fwd_bwd(gcg_lib, bs, L, g, dg, hl, dtype):
    x, dy, w = data(bs, L, g, dg, hl, dtype, seed=hl + L)
    one = torch.ones(bs, L, g, dg)
    y_ref = oracle.gcg_fwd_oracle(x.float(), one, one, w.float())
    dx_ref, _, _, dw_ref = oracle.gcg_bwd_oracle(dy.float(), x.float(), one, one, w.float())
    y = _lib.dwconv_fwd(x.to(DEV), w.to(DEV))
    dx, dw = _lib.dwconv_bwd(dy.to(DEV), x.to(DEV), w.to(DEV))
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == x.shape and dw.shape == w.shape
    assert_close(y, y_ref, TOL[dtype], "y")
    assert_close(dx, dx_ref, TOL[dtype], "dx")
    if bs * L * dg >= 64:       # a tap summed from a handful of rounded terms can cancel
        assert_close(dw, dw_ref, TOL_DH[dtype], "dw")
    # the same, phrased as the reference module does it on (B, D, L)
    wd = w.float().repeat_interleave(dg, dim=0)
    y_mod = conv_as_reference(x.float().reshape(bs, L, g * dg).permute(0, 2, 1), wd).permute(0, 2, 1)
    assert_close(y.reshape(bs, L, g * dg), y_mod, TOL[dtype], "y vs F.conv1d")


def test_dwconv_is_deterministic_and_rejects_what_it_cannot_run(gcg_lib):
    x, dy, w = (t.to(DEV) for t in data(2, 512, 64, 1, 3, torch.float32, seed=1))
    a, b = _lib.dwconv_bwd(dy, x, w), _lib.dwconv_bwd(dy, x, w)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    x2, _, w2 = (t.to(DEV) for t in data(1, 64, 8, 2, 3, torch.float32, seed=2))     # dg = 2
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.dwconv_fwd(x2, w2)
    x3, _, w3 = (t.to(DEV) for t in data(1, 64, 8, 1, 9, torch.float32, seed=2))     # 9 taps
    with pytest.raises(RuntimeError, match="not supported"):
        _lib.dwconv_fwd(x3, w3)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _lib.dwconv_fwd(x.cpu(), w.cpu())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_module_matches_the_reference_formulation(gcg_lib, dtype):
    """CausalDepthwiseConv1d on (B, D, L) against pad + F.conv1d with the module's own weight, with
    gradients for input and weight."""
    B, D, L, K = 2, 96, 200, 3
    torch.manual_seed(3)
    m = CausalDepthwiseConv1d(D, K, dtype=dtype, device=DEV)
    x = torch.randn(B, D, L).to(dtype)
    dy = (0.1 * torch.randn(B, D, L)).to(dtype)
    xd = x.to(DEV).requires_grad_(True)
    y = m(xd)
    assert y.shape == (B, D, L)
    y.backward(dy.to(DEV))
    x32 = x.float().requires_grad_(True)
    w32 = m.short_conv_weight.detach().float().cpu().requires_grad_(True)
    y_ref = conv_as_reference(x32, w32)
    y_ref.backward(dy.float())
    assert_close(y, y_ref, TOL[dtype], "y")
    assert_close(xd.grad, x32.grad, TOL[dtype], "dx")
    assert_close(m.short_conv_weight.grad, w32.grad, TOL_DH[dtype], "dw")


def test_featurizer_then_interleaved_operator(gcg_lib):
    """block.py:867-890 end to end on (B, L, 3D): featurizer conv, interleaved split, gated
    convolution -- against the same chain written with F.conv1d and the library formulation."""
    bs, L, g, dg, hl, dtype = 2, 256, 4, 16, 128, torch.bfloat16
    d3 = 3 * g * dg
    gen = torch.Generator().manual_seed(9)
    u = torch.randn(bs, L, d3, generator=gen).to(dtype)
    h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype)
    dz = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype)
    torch.manual_seed(4)
    feat = CausalDepthwiseConv1d(d3, 3, dtype=dtype, device=DEV)

    ud, hd = u.to(DEV).requires_grad_(True), h.to(DEV).requires_grad_(True)
    z = two_pass_chunked_gate_conv_gate_interleaved(feat.forward_bld(ud), hd, bs, L, g, dg)
    z.backward(dz.to(DEV))
    torch.cuda.synchronize()

    u32 = u.float().requires_grad_(True)
    h32 = h.float().requires_grad_(True)
    w32 = feat.short_conv_weight.detach().float().cpu().requires_grad_(True)
    f = conv_as_reference(u32.permute(0, 2, 1), w32).permute(0, 2, 1)
    f = f + (f.to(dtype).float() - f).detach()          # the featurizer's output is stored in bf16
    x1, x2, v = rearrange(f, "b l (g dg p) -> b l g p dg", p=3, g=g).unbind(dim=3)
    z_ref = oracle.gcg_fwd_ref_torch(v.contiguous(), x2.contiguous(), x1.contiguous(), h32)
    z_ref.backward(dz.float())
    assert_close(z, z_ref, TOL[dtype], "z")
    assert_close(ud.grad, u32.grad, 2e-2, "d input")     # two bf16 stages back to back
    assert_close(hd.grad, h32.grad, TOL_DH[dtype], "dh")
    assert_close(feat.short_conv_weight.grad, w32.grad, 2e-2, "dw featurizer")


def test_featurizer_shape_of_a_7b_layer(gcg_lib):
    """B=2, L=8192, 12288 channels, 3 taps: a shift filter must reproduce the input bit for bit,
    and sampled channels must match the oracle with random filters."""
    bs, L, D, K, dtype = 2, 8192, 12288, 3, torch.bfloat16
    gen = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(bs, L, D, 1, generator=gen, device=DEV).to(dtype)
    dy = (0.1 * torch.randn(bs, L, D, 1, generator=gen, device=DEV)).to(dtype)
    w = torch.zeros(D, 1, K, dtype=dtype, device=DEV)
    w[:, 0, 0] = 1.0                                   # tap 0 multiplies the sample K-1 rows back
    y = _lib.dwconv_fwd(x, w)
    dx, dw = _lib.dwconv_bwd(dy, x, w)
    torch.cuda.synchronize()
    assert torch.equal(y[:, K - 1:], x[:, :L - K + 1]) and not y[:, :K - 1].any()
    assert torch.equal(dx[:, :L - K + 1], dy[:, K - 1:]) and not dx[:, L - K + 1:].any()
    w = (torch.randn(D, 1, K, generator=gen, device=DEV) / K ** 0.5).to(dtype)
    y = _lib.dwconv_fwd(x, w)
    dx, dw = _lib.dwconv_bwd(dy, x, w)
    idx = torch.tensor([0, 1, 2, 3, 4095, 8191, 12287], device=DEV)
    xs, dys, ws = (t.index_select(2 if t.dim() == 4 else 0, idx).float().cpu() for t in (x, dy, w))
    one = torch.ones_like(xs)
    y_ref = oracle.gcg_fwd_oracle(xs, one, one, ws)
    dx_ref, _, _, dw_ref = oracle.gcg_bwd_oracle(dys, xs, one, one, ws)
    assert_close(y.index_select(2, idx), y_ref, TOL[dtype], "y")
    assert_close(dx.index_select(2, idx), dx_ref, TOL[dtype], "dx")
    assert_close(dw.index_select(0, idx), dw_ref, TOL_DH[dtype], "dw")


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
def test_keep_output_changes_the_cache_policy_not_the_values(gcg_lib, dtype):
    """GCG_KEEP_OUTPUT on the two entry points that write a chain's intermediates: the featurized
    tensor (gcg_dwconv_fwd) and the gradient of the features (gcg_bwd_interleaved, matrix-core and
    register-window families); an unknown flag is refused."""
    x, _, w = (t.to(DEV) for t in data(2, 300, 48, 1, 3, dtype, seed=4))
    assert torch.equal(_lib.dwconv_fwd(x, w), _lib.dwconv_fwd(x, w, keep_output=True))
    for (bs, L, g, dg, hl) in [(1, 300, 3, 16, 128), (2, 200, 4, 8, 7)]:
        gen = torch.Generator().manual_seed(hl)
        feat = torch.randn(bs, L, g, dg, 3, generator=gen).to(dtype).to(DEV)
        dy = torch.randn(bs, L, g, dg, generator=gen).to(dtype).to(DEV)
        h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype).to(DEV)
        a, b = _lib.bwd_interleaved(dy, feat, h), _lib.bwd_interleaved(dy, feat, h, keep_output=True)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    lib = _lib.load()
    p = x.data_ptr()
    assert lib.gcg_dwconv_fwd(p, p, p, 1, 64, 16, 1, 3, 0, 2, None) == -1        # unknown flag
