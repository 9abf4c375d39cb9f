"""The torch.ops.gcg operators on the GPU: results against the oracle, agreement of the two bindings of the library
(torch operators and ctypes), torch.library's own operator checks, and torch.compile(fullgraph=True) of the
reference-compatible entry point against eager (the reference compiles its filter, explicit.py:71, so callers of
this path are traced)."""
import os

import pytest
import torch

from helpers import TOL, TOL_DH, assert_close, inputs, oracle_bwd, oracle_fwd
from savanna_amd import _lib, _ops, two_pass_chunked_gate_conv_gate
from savanna_amd.kernels.cgcg.interface import two_pass_chunked_gate_conv_gate_interleaved
from savanna_amd.kernels.cgcg.src.kernel_utils import FwdKernelConfigRefactor

# with GCG_BINDING=ctypes the operators are deliberately not registered: there is nothing here to test then
pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("GCG_BINDING") == "ctypes", reason="GCG_BINDING=ctypes: no torch operators")]

DEV = "cuda:0"
CFG = FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row")


@pytest.mark.parametrize("shape,dtype", [((2, 300, 3, 16, 128), torch.bfloat16), ((1, 200, 4, 16, 7), torch.float32),
                                         ((1, 700, 2, 16, 200), torch.float16)])
def test_ops_against_oracle(gcg_lib, shape, dtype):
    assert _ops.AVAILABLE, _ops.LOAD_ERROR
    x, B, C, h, dy = inputs(*shape, dtype)
    xd, Bd, Cd, hd, dyd = (t.to(DEV) for t in (x, B, C, h, dy))
    bx, y2, y = torch.ops.gcg.fwd_full(xd, Bd, Cd, hd, True, True)
    rbx, ry2, ry = oracle_fwd(x, B, C, h)
    for name, got, ref in (("bx", bx, rbx), ("y2", y2, ry2), ("y", y, ry)):
        assert_close(got, ref, TOL[dtype], name)
    assert torch.equal(torch.ops.gcg.fwd(xd, Bd, Cd, hd), y)
    out = torch.full_like(xd, float("nan"))
    torch.ops.gcg.fwd_out(xd, Bd, Cd, hd, out)
    assert torch.equal(out, y)
    got = torch.ops.gcg.bwd(dyd, xd, Bd, Cd, hd)
    for name, g_, r_ in zip(("dx", "dB", "dC", "dh"), got, oracle_bwd(dy, x, B, C, h)):
        assert_close(g_, r_, TOL_DH[dtype] if name == "dh" else TOL[dtype], name)


def test_both_bindings_give_the_same_bits(gcg_lib, monkeypatch):
    x, B, C, h, dy = (t.to(DEV) for t in inputs(2, 1000, 5, 16, 100, torch.bfloat16, seed=3))
    feat = torch.stack([C, B, x], dim=-1).contiguous()
    via_ops = (_lib.fwd(x, B, C, h)[2], *_lib.bwd(dy, x, B, C, h), _lib.fwd_interleaved(feat, h),
               *_lib.bwd_interleaved(dy, feat, h))
    monkeypatch.setattr(_lib, "TORCH_OPS", False)
    via_ctypes = (_lib.fwd(x, B, C, h)[2], *_lib.bwd(dy, x, B, C, h), _lib.fwd_interleaved(feat, h),
                  *_lib.bwd_interleaved(dy, feat, h))
    for a, b in zip(via_ops, via_ctypes):
        assert torch.equal(a, b)


def test_ops_run_on_the_current_stream_and_device(gcg_lib):
    """Enqueued on torch's current stream: a side stream's result is complete once that stream is waited on."""
    x, B, C, h, _ = (t.to(DEV) for t in inputs(1, 4096, 16, 16, 128, torch.bfloat16, seed=5))
    ref = torch.ops.gcg.fwd(x, B, C, h)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            y = torch.ops.gcg.fwd(x, B, C, h)
    torch.cuda.current_stream().wait_stream(side)
    assert torch.equal(y, ref)


def test_library_opcheck(gcg_lib):
    """torch.library.opcheck: schema (no undeclared mutation or aliasing) and meta implementation vs device result."""
    x, B, C, h, dy = (t.to(DEV) for t in inputs(1, 130, 2, 16, 33, torch.bfloat16))
    feat = torch.stack([C, B, x], dim=-1).contiguous()
    checks = ("test_schema", "test_faketensor")
    torch.library.opcheck(torch.ops.gcg.fwd, (x, B, C, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.fwd_full, (x, B, C, h, True, True), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.bwd, (dy, x, B, C, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.fwd_interleaved, (feat, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.bwd_interleaved, (dy, feat, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.fwd_out, (x, B, C, h, torch.empty_like(x)), test_utils=checks)
    planar = torch.stack([C, B, x], dim=2).contiguous()
    torch.library.opcheck(torch.ops.gcg.fwd_planar, (planar, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.bwd_planar, (dy, planar, h), test_utils=checks)
    # the Hyena-MR mixer operators, with the filter given and formed in the kernels
    x, B, C, h, dy = (t.to(DEV) for t in inputs(1, 130, 2, 16, 128, torch.bfloat16))
    feat = torch.stack([C, B, x], dim=-1).contiguous()
    wf = (torch.randn(3 * 2 * 16, 1, 3, device=DEV) / 3 ** 0.5).to(torch.bfloat16)
    w = torch.randn(2, 128, device=DEV) / 128 ** 0.5
    decay = torch.rand(2, 128, device=DEV)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_fwd, (feat, wf, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_bwd, (dy, feat, wf, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_fwd_decay, (feat, wf, w, decay, 128, torch.bfloat16), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_bwd_decay, (dy, feat, wf, w, decay, 128, torch.bfloat16),
                          test_utils=checks)
    pl, wf_pl = feat.permute(0, 1, 4, 2, 3).contiguous(), wf        # planar flag (the filters' order is immaterial here)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_fwd, (pl, wf_pl, h, True), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_bwd, (dy, pl, wf_pl, h, True), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_fwd_decay, (pl, wf_pl, w, decay, 128, torch.bfloat16, True), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_mr_bwd_decay, (dy, pl, wf_pl, w, decay, 128, torch.bfloat16, True),
                          test_utils=checks)
    # the filter alone and inside the operator's kernels
    torch.library.opcheck(torch.ops.gcg.filter_decay_fwd, (w, decay, 128, torch.bfloat16), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.filter_decay_bwd, (torch.randn(2, 1, 128, device=DEV), decay), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.fwd_decay, (x, B, C, w, decay, 128, torch.bfloat16), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.bwd_decay, (dy, x, B, C, w, decay, 128, torch.bfloat16), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.fwd_interleaved_decay, (feat, w, decay, 128, torch.bfloat16), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.bwd_interleaved_decay, (dy, feat, w, decay, 128, torch.bfloat16), test_utils=checks)
    # the featurizer, the Hyena-SE mixer (both layouts) and time-major operands
    x, B, C, h, dy = (t.to(DEV) for t in inputs(1, 130, 2, 16, 7, torch.bfloat16))
    feat = torch.stack([C, B, x], dim=-1).contiguous()
    flat = feat.view(1, 130, 3 * 2 * 16, 1)
    torch.library.opcheck(torch.ops.gcg.dwconv_fwd, (flat, wf), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.dwconv_bwd, (flat, flat, wf), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_se_fwd, (feat, wf, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_se_bwd, (dy, feat, wf, h), test_utils=checks)
    pl = feat.permute(0, 1, 4, 2, 3).contiguous()
    torch.library.opcheck(torch.ops.gcg.mixer_se_fwd, (pl, wf, h, True), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.mixer_se_bwd, (dy, pl, wf, h, True), test_utils=checks)
    xt, Bt, Ct = (t.permute(1, 0, 2, 3).contiguous() for t in (x, B, C))
    torch.library.opcheck(torch.ops.gcg.fwd_time_major, (xt, Bt, Ct, h), test_utils=checks)
    torch.library.opcheck(torch.ops.gcg.bwd_time_major, (dy, xt, Bt, Ct, h), test_utils=checks)
    checked = {"fwd", "fwd_full", "bwd", "fwd_interleaved", "bwd_interleaved", "fwd_out", "fwd_planar", "bwd_planar",
               "mixer_mr_fwd", "mixer_mr_bwd", "mixer_mr_fwd_decay", "mixer_mr_bwd_decay", "filter_decay_fwd",
               "filter_decay_bwd", "fwd_decay", "bwd_decay", "fwd_interleaved_decay", "bwd_interleaved_decay", "dwconv_fwd",
               "dwconv_bwd", "mixer_se_fwd", "mixer_se_bwd", "fwd_time_major", "bwd_time_major"}
    assert checked == set(_ops.OP_NAMES)                # a new operator gets its check here


def _grads(fn, tensors, dy):
    leaves = [t.detach().clone().requires_grad_(True) for t in tensors]
    y = fn(*leaves)
    y.backward(dy)
    return [y.detach()] + [t.grad for t in leaves]


@pytest.mark.parametrize("shape,dtype", [((2, 512, 4, 16, 128), torch.bfloat16), ((1, 256, 8, 16, 7), torch.float32)])
def test_compile_fullgraph_matches_eager(gcg_lib, shape, dtype):
    bs, L, g, dg, hl = shape
    x, B, C, h, dy = (t.to(DEV) for t in inputs(*shape, dtype, seed=7))

    def op(x, B, C, h):
        return two_pass_chunked_gate_conv_gate(x, B, C, h, bs, L, g, dg, fwd_kernel_cfg=CFG)

    eager = _grads(op, (x, B, C, h), dy)
    torch._dynamo.reset()
    compiled = _grads(torch.compile(op, fullgraph=True, backend="aot_eager"), (x, B, C, h), dy)
    for name, a, b in zip(("y", "dx", "dB", "dC", "dh"), eager, compiled):
        assert torch.equal(a, b), name


def test_compile_fullgraph_interleaved(gcg_lib):
    bs, L, g, dg, hl = 1, 384, 4, 16, 128
    x, B, C, h, dy = (t.to(DEV) for t in inputs(bs, L, g, dg, hl, torch.bfloat16, seed=9))
    feat = torch.stack([C, B, x], dim=-1).reshape(bs, L, 3 * g * dg).contiguous()

    def op(feat, h):
        return two_pass_chunked_gate_conv_gate_interleaved(feat, h, bs, L, g, dg)

    eager = _grads(op, (feat, h), dy)
    torch._dynamo.reset()
    compiled = _grads(torch.compile(op, fullgraph=True, backend="aot_eager"), (feat, h), dy)
    for name, a, b in zip(("y", "dfeat", "dh"), eager, compiled):
        assert torch.equal(a, b), name


@pytest.mark.parametrize("planar", [False, True], ids=["interleaved", "planar"])
@pytest.mark.parametrize("kind", ["mr", "se", "se-grouped"])
def test_compile_fullgraph_hyena_mixer(gcg_lib, kind, planar):
    """HyenaMixer (featurizer conv, split, operator; for Hyena-MR with the filter formed in the kernel) traced by
    torch.compile without a graph break: output and every gradient equal to eager."""
    from savanna_amd.operators.hyena import CgcgConfig, HyenaMixer, HyenaMROperator, HyenaSEOperator

    torch.manual_seed(3)
    bs, L, g, dg = 2, 384, 4, 16
    cfg = CgcgConfig(cgcg_dtype="bfloat16")
    op = (HyenaMROperator(g * dg, g, 128, cfg, small_init=False, device=DEV) if kind == "mr"
          else HyenaSEOperator(g * dg, g * dg if kind == "se" else g, 7, cfg, device=DEV))
    mixer = HyenaMixer(op, 3, dtype=torch.bfloat16, device=DEV, interleave_projections=not planar)
    feats = torch.randn(bs, L, 3 * g * dg, device=DEV).to(torch.bfloat16).requires_grad_(True)
    dz = (0.1 * torch.randn(bs, L, g * dg, device=DEV)).to(torch.bfloat16)
    params = list(mixer.parameters())

    def run(fn):
        feats.grad = None
        for p in params:
            p.grad = None
        z = fn(feats)
        z.backward(dz)
        return [z.detach(), feats.grad.clone()] + [p.grad.clone() for p in params]

    eager = run(mixer)
    torch._dynamo.reset()
    compiled = run(torch.compile(mixer, fullgraph=True, backend="aot_eager"))
    assert len(eager) == len(compiled) == 2 + len(params)
    for i, (a, b) in enumerate(zip(eager, compiled)):
        assert torch.equal(a, b), i


def _leaves(*ts):
    return [t.detach().clone().requires_grad_(True) for t in ts]


def test_forward_operators_are_differentiable(gcg_lib):
    """A call of torch.ops.gcg.* on tensors that require grad is part of the autograd graph: the gradients are the
    backward operator's outputs, bit for bit, and opcheck finds the registration in order."""
    ops = torch.ops.gcg
    x, B, C, h, dy = (t.to(DEV) for t in inputs(2, 300, 3, 16, 128, torch.bfloat16, seed=9, dy_scale=0.1))
    feat = torch.stack([C, B, x], dim=-1).contiguous()
    planar = torch.stack([C, B, x], dim=2).contiguous()
    wf = (torch.randn(3 * 3 * 16, 1, 3, device=DEV) / 3 ** 0.5).to(torch.bfloat16)
    w = torch.randn(3, 128, device=DEV) / 128 ** 0.5
    decay = torch.rand(3, 128, device=DEV)
    hs = h[..., :7].contiguous()
    cases = [
        (ops.fwd, (x, B, C, h), lambda a: ops.bwd(dy, *a)),
        (ops.fwd_interleaved, (feat, h), lambda a: ops.bwd_interleaved(dy, *a)),
        (ops.fwd_planar, (planar, h), lambda a: ops.bwd_planar(dy, *a)),
        (ops.mixer_mr_fwd, (feat, wf, h), lambda a: ops.mixer_mr_bwd(dy, *a)),
        (ops.mixer_se_fwd, (feat, wf, hs), lambda a: ops.mixer_se_bwd(dy, *a)),
        (ops.fwd_time_major, (x.transpose(0, 1).contiguous(), B.transpose(0, 1).contiguous(),
                              C.transpose(0, 1).contiguous(), hs), lambda a: ops.bwd_time_major(dy, *a)),
    ]
    for op, args, backward in cases:
        leaves = _leaves(*args)
        y = op(*leaves)
        assert y.requires_grad, op
        y.backward(dy)
        want = backward(args)
        for leaf, g in zip(leaves, want):
            assert torch.equal(leaf.grad, g), op
    # the featurizer conv (its own gradient shape) and the operators that form the filter inside the kernels
    xs = feat.reshape(2, 300, 144, 1)
    lx, lw = _leaves(xs, wf)
    ops.dwconv_fwd(lx, lw).backward(xs)
    for got, g in zip((lx.grad, lw.grad), ops.dwconv_bwd(xs, xs, wf)):
        assert torch.equal(got, g)
    lv = _leaves(x, B, C, w)
    ops.fwd_decay(*lv, decay, 128, torch.bfloat16).backward(dy)
    for leaf, g in zip(lv, ops.bwd_decay(dy, x, B, C, w, decay, 128, torch.bfloat16)):
        assert torch.equal(leaf.grad, g)
    lf, lw2 = _leaves(feat, w)
    ops.fwd_interleaved_decay(lf, lw2, decay, 128, torch.bfloat16).backward(dy)
    for got, g in zip((lf.grad, lw2.grad), ops.bwd_interleaved_decay(dy, feat, w, decay, 128, torch.bfloat16)):
        assert torch.equal(got, g)
    lr, lwf, lw3 = _leaves(feat, wf, w)
    ops.mixer_mr_fwd_decay(lr, lwf, lw3, decay, 128, torch.bfloat16).backward(dy)
    for got, g in zip((lr.grad, lwf.grad, lw3.grad), ops.mixer_mr_bwd_decay(dy, feat, wf, w, decay, 128, torch.bfloat16)):
        assert torch.equal(got, g)
    (lw4,) = _leaves(w)
    dh = torch.randn(3, 1, 128, device=DEV).to(torch.bfloat16)
    ops.filter_decay_fwd(lw4, decay, 128, torch.bfloat16).backward(dh)
    assert torch.equal(lw4.grad, ops.filter_decay_bwd(dh, decay))
    # the forward with optional extra outputs is not differentiable and says so
    with pytest.raises(RuntimeError, match="not differentiable"):
        ops.fwd_full(*_leaves(x, B, C, h), False, False)[2].backward(dy)
    checks = ("test_schema", "test_autograd_registration", "test_faketensor")
    torch.library.opcheck(ops.fwd, tuple(_leaves(x, B, C, h)), test_utils=checks)
    torch.library.opcheck(ops.fwd_interleaved, tuple(_leaves(feat, h)), test_utils=checks)
    torch.library.opcheck(ops.mixer_mr_fwd, tuple(_leaves(feat, wf, h)), test_utils=checks)
    torch.library.opcheck(ops.dwconv_fwd, tuple(_leaves(xs, wf)), test_utils=checks)
