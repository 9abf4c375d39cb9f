"""HyenaMixer over the grid of its routes -- operator kind and filter length, feature layout, activation and
cgcg dtype, featurizer length, group width -- against the reference's chain written with torch ops on the same
values: featurizer conv on (B, 3D, L) (block.py:867-876), the split with or without interleaving (:881-888), the
casts to cgcg_dtype and back around the gated convolution (hyena.py:499-503, :533-534, :812-816, :842-843), and
the decayed filter (explicit.py:68-75).  Output and the gradients of the features, the featurizer's weight and
the operator's filter parameter; whichever kernels a combination selects, the values must be the chain's."""
import itertools

import pytest
import torch
import torch.nn.functional as F

from helpers import TOL, TOL_DH, assert_close
from savanna_amd.operators.hyena import CgcgConfig, HyenaMixer, HyenaMROperator, HyenaSEOperator

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

KINDS = {"se7": ("se", 7), "se4": ("se", 4), "se9": ("se", 9), "mr128": ("mr", 128), "mr64": ("mr", 64)}
# (activations, cgcg_dtype)
TYPES = {"bf16": (torch.bfloat16, "bfloat16"), "f32": (torch.float32, "float32"), "bf16-f32": (torch.bfloat16, "float32"),
         "f16": (torch.float16, "float16")}
GRID = [(k, pl, t, kf, dg)
        for k, pl, t, (kf, dg) in itertools.product(KINDS, (False, True), TYPES, ((3, 16), (4, 16), (3, 2), (2, 32)))
        if not (kf == 4 and k.startswith("mr") and t != "bf16")      # one type is enough for the unfused featurizer
        and not (dg == 2 and k.startswith("mr"))]                    # Hyena-MR groups are 16 wide or more (fwd.py:80)


def _reference(feats, wf, filt_param, decay, kind, hl, planar, act, cgcg, g, dg, kf):
    bs, L, d3 = feats.shape
    d = d3 // 3
    # featurizer: fp32 sums of the products, stored in the activations' type
    f = F.conv1d(F.pad(feats.float().transpose(1, 2), (kf - 1, 0)), wf.to(act).float(), groups=d3).transpose(1, 2).to(act)
    if planar:
        x1, x2, v = f.reshape(bs, L, 3, g, dg).unbind(2)
    else:
        x1, x2, v = f.reshape(bs, L, g, dg, 3).unbind(4)
    if kind == "mr":
        h = (filt_param[:, :hl] * decay[:, :hl]).to(cgcg)[:, None]
    else:
        h = filt_param.to(cgcg)
    x1, x2, v = (t.to(cgcg) for t in (x1, x2, v))
    u = (v * x2).float().reshape(bs, L, d).transpose(1, 2)                  # B*x in cgcg_dtype (fwd_kernels.py:700)
    y = F.conv1d(F.pad(u, (hl - 1, 0)), h.float().repeat_interleave(dg, 0), groups=d).transpose(1, 2)
    z = (x1.float().reshape(bs, L, d) * y).to(cgcg)                         # fp32 until after the post-gate
    return z.to(act)


@pytest.mark.parametrize("kind,planar,types,kf,dg", GRID,
                         ids=[f"{k}-{'planar' if pl else 'interleaved'}-{t}-kf{kf}-dg{dg}" for k, pl, t, kf, dg in GRID])
def test_every_route_gives_the_chains_values(gcg_lib, kind, planar, types, kf, dg):
    op_kind, hl = KINDS[kind]
    act, cgcg_name = TYPES[types]
    cgcg = getattr(torch, cgcg_name)
    torch.manual_seed(GRID.index((kind, planar, types, kf, dg)))       # the same values in every run
    bs, L, g = 2, 333, 6
    hidden = g * dg
    cfg = CgcgConfig(cgcg_dtype=cgcg_name)
    op = (HyenaMROperator(hidden, g, hl, cfg, small_init=False, device=DEV) if op_kind == "mr"
          else HyenaSEOperator(hidden, g, hl, cfg, device=DEV))
    mixer = HyenaMixer(op, kf, dtype=act, device=DEV, interleave_projections=not planar)
    feats = torch.randn(bs, L, 3 * hidden, device=DEV).to(act)
    dz = (0.1 * torch.randn(bs, L, hidden, device=DEV)).to(act)

    x = feats.clone().requires_grad_(True)
    z = mixer(x)
    z.backward(dz)
    filt_param = op.filter.h if op_kind == "mr" else op.short_conv_weight
    got = (z.detach(), x.grad, mixer.hyena_proj_conv.short_conv_weight.grad, filt_param.grad)
    assert z.dtype == act and z.shape == (bs, L, hidden) and x.grad.dtype == act

    xr = feats.clone().requires_grad_(True)
    wf = mixer.hyena_proj_conv.short_conv_weight.detach().clone().requires_grad_(True)
    fp = filt_param.detach().clone().requires_grad_(True)
    decay = op.filter.decay if op_kind == "mr" else None
    zr = _reference(xr, wf, fp, decay, op_kind, hl, planar, act, cgcg, g, dg, kf)
    zr.backward(dz)
    torch.cuda.synchronize()
    low = torch.float32 if (act == torch.float32 and cgcg == torch.float32) else (torch.float16 if act == torch.float16 else torch.bfloat16)
    tol, tol_w = TOL[low], TOL_DH[low]
    assert_close(got[0], zr, tol, "z")
    assert_close(got[1], xr.grad, 2 * tol, "d features")
    assert_close(got[2], wf.grad, 2 * tol_w, "d featurizer weight")
    assert_close(got[3], fp.grad, 2 * tol_w, "d filter parameter")


@pytest.mark.parametrize("planar", [False, True], ids=["interleaved", "planar"])
@pytest.mark.parametrize("kind", ["mr", "se"])
def test_ways_a_training_loop_calls_the_module(gcg_lib, kind, planar):
    """Views with a larger row stride as features and as output gradient, a second backward through a retained graph,
    no_grad, frozen features, autocast around the call, and parameters converted to bf16: the same values each time."""
    torch.manual_seed(0)
    bs, L, g, dg = 2, 500, 4, 16
    hidden = g * dg
    cfg = CgcgConfig(cgcg_dtype="bfloat16")
    op = (HyenaMROperator(hidden, g, 128, cfg, small_init=False, device=DEV) if kind == "mr"
          else HyenaSEOperator(hidden, g, 7, cfg, device=DEV))
    m = HyenaMixer(op, 3, dtype=torch.bfloat16, device=DEV, interleave_projections=not planar)
    feats = torch.randn(bs, L, 3 * hidden + 64, device=DEV).to(torch.bfloat16)[..., :3 * hidden]
    dz = (0.1 * torch.randn(bs, L, hidden * 2, device=DEV)).to(torch.bfloat16)[..., ::2]
    assert not feats.is_contiguous() and not dz.is_contiguous()
    ref_in = feats.contiguous().requires_grad_(True)
    z_ref = m(ref_in)
    z_ref.backward(dz, retain_graph=True)
    g1 = ref_in.grad.clone()
    ref_in.grad = None
    z_ref.backward(dz)
    assert torch.equal(ref_in.grad, g1), "second backward"
    x = feats.detach().requires_grad_(True)
    z = m(x)
    assert torch.equal(z, z_ref), "features with a larger row stride"
    z.backward(dz)
    assert torch.equal(x.grad, g1), "their gradient"
    with torch.no_grad():
        assert torch.equal(m(feats), z_ref), "no_grad"
    for p in m.parameters():
        p.grad = None
    m(feats.contiguous()).backward(dz)
    assert all(p.grad is not None for p in m.parameters()), "frozen features"
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert torch.equal(m(feats.contiguous()), z_ref), "autocast"
    import copy
    m16 = copy.deepcopy(m).bfloat16()                   # every parameter in bf16: the filter is then formed by torch ops
    z16 = m16(feats.contiguous())
    assert_close(z16, z_ref, 3 * TOL[torch.bfloat16], "bf16 parameters")      # w and decay rounded before their product
    z16.sum().backward()
    assert all(p.grad is not None and p.grad.dtype == torch.bfloat16 for p in m16.parameters())
