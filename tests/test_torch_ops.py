"""The PyTorch extension (csrc/gcg_torch.cpp): torch.ops.gcg.* exist with the schemas the Python layers use, and
their meta implementations give the shapes and dtypes of the device ones -- checked here without a GPU on fake
tensors, which is also what torch.compile traces with."""
import pytest
import torch

from savanna_amd import _lib, _ops


def test_extension_loads_and_registers_every_operator(gcg_lib):
    assert _ops.AVAILABLE, _ops.LOAD_ERROR
    assert _lib.TORCH_OPS
    for name in _ops.OP_NAMES:
        assert hasattr(torch.ops.gcg, name), name


def test_meta_shapes_on_fake_gpu_tensors(gcg_lib):
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        bs, L, g, dg, hl = 2, 96, 4, 16, 128
        x = torch.empty(bs, L, g, dg, dtype=torch.bfloat16, device="cuda")
        h = torch.empty(g, 1, hl, dtype=torch.bfloat16, device="cuda")
        y = torch.ops.gcg.fwd(x, x, x, h)
        assert y.shape == x.shape and y.dtype == x.dtype and y.device == x.device
        bx, y2, y = torch.ops.gcg.fwd_full(x, x, x, h, True, False)
        assert bx.shape == x.shape and y2.numel() == 0 and y.shape == x.shape
        dx, dB, dC, dh = torch.ops.gcg.bwd(x, x, x, x, h)
        assert dx.shape == dB.shape == dC.shape == x.shape and dh.shape == h.shape
        feat = torch.empty(bs, L, g, dg, 3, dtype=torch.bfloat16, device="cuda")
        assert torch.ops.gcg.fwd_interleaved(feat, h).shape == x.shape
        dfeat, dh = torch.ops.gcg.bwd_interleaved(x, feat, h)
        assert dfeat.shape == feat.shape and dh.shape == h.shape
        wf = torch.empty(3 * g * dg, 1, 3, dtype=torch.bfloat16, device="cuda")
        h7 = torch.empty(g, 1, 7, dtype=torch.bfloat16, device="cuda")
        assert torch.ops.gcg.mixer_se_fwd(feat, wf, h7).shape == x.shape
        draw, dwf, dh7 = torch.ops.gcg.mixer_se_bwd(x, feat, wf, h7)
        assert draw.shape == feat.shape and dwf.shape == wf.shape and dh7.shape == h7.shape
        w = torch.empty(g, 1, 3, dtype=torch.bfloat16, device="cuda")
        assert torch.ops.gcg.dwconv_fwd(x, w).shape == x.shape
        dxx, dw = torch.ops.gcg.dwconv_bwd(x, x, w)
        assert dxx.shape == x.shape and dw.shape == w.shape
        p = torch.empty(g, 128, device="cuda")
        hh = torch.ops.gcg.filter_decay_fwd(p, p, 64, torch.float16)
        assert hh.shape == (g, 1, 64) and hh.dtype == torch.float16
        assert torch.ops.gcg.filter_decay_bwd(hh, p).shape == p.shape
        planar = torch.empty(bs, L, 3, g, dg, dtype=torch.bfloat16, device="cuda")
        assert torch.ops.gcg.mixer_mr_fwd(planar, wf, h, True).shape == x.shape
        assert torch.ops.gcg.mixer_se_fwd(planar, wf, h7, True).shape == x.shape
        dpl, dwf_pl, dh_pl = torch.ops.gcg.mixer_mr_bwd(x, planar, wf, h, True)
        assert dpl.shape == planar.shape and dwf_pl.shape == wf.shape and dh_pl.shape == h.shape
        dpl, dwf_pl, dh_pl = torch.ops.gcg.mixer_se_bwd(x, planar, wf, h7, True)
        assert dpl.shape == planar.shape and dwf_pl.shape == wf.shape and dh_pl.shape == h7.shape
        assert torch.ops.gcg.mixer_mr_fwd_decay(planar, wf, p, p, 128, torch.bfloat16, True).shape == x.shape
        dpl, dwf_pl, dw_pl = torch.ops.gcg.mixer_mr_bwd_decay(x, planar, wf, p, p, 128, torch.bfloat16, True)
        assert dpl.shape == planar.shape and dwf_pl.shape == wf.shape and dw_pl.shape == p.shape
        assert torch.ops.gcg.fwd_planar(planar, h).shape == x.shape
        dplanar, dh = torch.ops.gcg.bwd_planar(x, planar, h)
        assert dplanar.shape == planar.shape and dh.shape == h.shape
        # Hyena-MR mixer (featurizer + operator), with the filter given and with the filter formed in the kernels
        assert torch.ops.gcg.mixer_mr_fwd(feat, wf, h).shape == x.shape
        draw, dwf, dh = torch.ops.gcg.mixer_mr_bwd(x, feat, wf, h)
        assert draw.shape == feat.shape and dwf.shape == wf.shape and dh.shape == h.shape
        y = torch.ops.gcg.mixer_mr_fwd_decay(feat, wf, p, p, 128, torch.bfloat16)
        assert y.shape == x.shape and y.dtype == x.dtype
        draw, dwf, dw = torch.ops.gcg.mixer_mr_bwd_decay(x, feat, wf, p, p, 128, torch.bfloat16)
        assert draw.shape == feat.shape and dwf.shape == wf.shape and dw.shape == p.shape and dw.dtype == torch.float32
        y = torch.ops.gcg.fwd_interleaved_decay(feat, p, p, 128, torch.bfloat16)
        assert y.shape == x.shape
        dfeat, dw = torch.ops.gcg.bwd_interleaved_decay(x, feat, p, p, 128, torch.bfloat16)
        assert dfeat.shape == feat.shape and dw.shape == p.shape


def test_meta_implementations_check_arguments(gcg_lib):
    x = torch.empty(2, 32, 4, 16, device="meta")
    h = torch.empty(4, 1, 7, device="meta")
    with pytest.raises(RuntimeError, match="one shape"):
        torch.ops.gcg.fwd(x, x[:, :16], x, h)
    with pytest.raises(RuntimeError, match=r"\(g, 1, hl\)"):
        torch.ops.gcg.fwd(x, x, x, h[:2])
    with pytest.raises(RuntimeError, match="one dtype"):
        torch.ops.gcg.fwd(x, x.to(torch.bfloat16), x, h)
    with pytest.raises(RuntimeError, match="filter must have the tensors' dtype"):
        torch.ops.gcg.fwd(x, x, x, h.to(torch.bfloat16))
    # 16-bit tensors with a float32 filter: fp32 arithmetic inside, 16-bit result, float32 filter gradient
    xb = x.to(torch.bfloat16)
    assert torch.ops.gcg.fwd(xb, xb, xb, h).dtype == torch.bfloat16
    assert [t.dtype for t in torch.ops.gcg.bwd(xb, xb, xb, xb, h)] == [torch.bfloat16] * 3 + [torch.float32]
    with pytest.raises(RuntimeError, match="contiguous"):
        torch.ops.gcg.fwd(x, x, x, torch.empty(4, 1, 14, device="meta")[:, :, ::2])


def test_cpu_tensors_are_refused(gcg_lib):
    x = torch.zeros(1, 8, 1, 16)
    h = torch.zeros(1, 1, 3)
    with pytest.raises(RuntimeError):          # the dispatcher has no CPU kernel for the operator
        torch.ops.gcg.fwd(x, x, x, h)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _lib.fwd(x, x, x, h)
