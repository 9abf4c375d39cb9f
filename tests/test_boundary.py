"""Host-side checks that need no GPU: the C-ABI library loads and exports exactly what
include/gcg.h declares, argument errors are reported before anything touches a device, and
the Python mirrors keep the reference's preconditions (interface.py:148-159, :48-49;
kernel_utils.py:289-294)."""
import ctypes
import os
import re
import subprocess

import pytest
import torch

from savanna_amd import _lib, two_pass_chunked_gate_conv_gate
from savanna_amd.kernels.cgcg.src.kernel_utils import BwdKernelConfigRefactor, FwdKernelConfigRefactor
from savanna_amd.operators import hyena

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "gcg.h")).read()
    return sorted(set(re.findall(r"GCG_API[^;(]*?\b(gcg_\w+)\s*\(", text)))


def test_header_and_library_agree(gcg_lib):
    want = declared_symbols()
    assert want == sorted(_lib.EXPORTS), "binding list and header differ"
    for name in want:
        assert hasattr(gcg_lib, name), f"{name} not exported"
    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    exported = sorted(re.findall(r" T (gcg_\w+)", out))
    assert exported == want, "library exports symbols the header does not declare (or misses some)"


def test_version_and_error_text(gcg_lib):
    assert gcg_lib.gcg_version() >= 100
    assert gcg_lib.gcg_strerror(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert len(gcg_lib.gcg_strerror(code)) > 5
    assert gcg_lib.gcg_strerror(-99) == b"unknown error"


def test_argument_errors_need_no_device(gcg_lib):
    p = ctypes.c_void_p(4096)   # never dereferenced: the calls fail on the checks before any launch
    # null pointer
    assert gcg_lib.gcg_fwd(None, p, p, p, p, None, None, 1, 64, 2, 16, 7, 0, 0, None) == -1
    # non-positive size, unknown dtype, unknown algo
    assert gcg_lib.gcg_fwd(p, p, p, p, p, None, None, 1, 0, 2, 16, 7, 0, 0, None) == -1
    assert gcg_lib.gcg_fwd(p, p, p, p, p, None, None, 1, 64, 2, 16, 7, 9, 0, None) == -1
    assert gcg_lib.gcg_fwd(p, p, p, p, p, None, None, 1, 64, 2, 16, 7, 0, 9, None) == -1
    # forced family that cannot take the shape
    assert gcg_lib.gcg_fwd(p, p, p, p, p, None, None, 1, 64, 2, 16, 200, 1, 3, None) == -2   # mfma, hl > 128
    assert gcg_lib.gcg_fwd(p, p, p, p, p, None, None, 1, 64, 2, 16, 9, 0, 2, None) == -2     # window, hl > 8
    assert gcg_lib.gcg_fwd(p, p, p, p, p, None, None, 1, 64, 2, 8, 64, 1, 3, None) == -2     # mfma, dg % 16
    # backward without workspace
    assert gcg_lib.gcg_bwd(p, p, p, p, p, p, p, p, p, None, 0, 1, 64, 2, 16, 7, 0, 0, None) == -3
    assert gcg_lib.gcg_bwd_workspace_bytes(1, 64, 2, 16, 7, 0, 0) > 0
    assert gcg_lib.gcg_bwd_workspace_bytes(1, 64, 2, 16, 7, 0, 0) % 256 == 0
    assert gcg_lib.gcg_bwd_workspace_bytes(0, 64, 2, 16, 7, 0, 0) == 0


def test_algo_selection(gcg_lib):
    bf, f32 = torch.bfloat16, torch.float32
    assert _lib.select_algo(2, 8192, 256, 16, 128, bf) == "mfma"          # Hyena-MR, bf16
    assert _lib.select_algo(2, 8192, 256, 16, 128, bf, backward=True) == "mfma"
    assert _lib.select_algo(1, 32768, 512, 16, 7, bf) == "window"         # Hyena-SE
    assert _lib.select_algo(1, 2048, 16, 16, 7, f32) == "window"          # fp32 SE config
    assert _lib.select_algo(2, 8192, 256, 16, 128, f32) == "mfma"         # fp32 MFMA keeps fp32 accuracy
    assert _lib.select_algo(2, 8192, 256, 4, 128, f32) == "direct"        # narrow groups stay on the vector ALUs
    assert _lib.select_algo(1, 512, 4, 16, 300, bf) == "direct"           # filter longer than a chunk
    assert _lib.select_algo(1, 512, 64, 1, 64, bf) == "direct"            # one channel per filter


def test_no_cpu_path():
    x = torch.randn(1, 8, 1, 16)
    h = torch.randn(1, 1, 3)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _lib.fwd(x, x, x, h)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _lib.bwd(x, x, x, x, h)
    with pytest.raises(TypeError):
        _lib.dtype_code(torch.float64)


def test_interface_preconditions():
    x = torch.randn(1, 8, 1, 16)
    h = torch.randn(1, 1, 3)
    cfg = FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row")
    with pytest.raises(AssertionError, match="fwd_kernel_cfg"):
        two_pass_chunked_gate_conv_gate(x, x, x, h, 1, 8, 1, 16)
    with pytest.raises(AssertionError, match="bwd_kernel_cfg"):
        two_pass_chunked_gate_conv_gate(x, x, x, h, 1, 8, 1, 16, fwd_kernel_cfg=cfg, bwd_autotune=False)
    with pytest.raises(AssertionError):   # declared shape must match the tensors
        two_pass_chunked_gate_conv_gate(x, x, x, h, 1, 9, 1, 16, fwd_kernel_cfg=cfg)
    with pytest.raises(AssertionError):   # B of another shape
        two_pass_chunked_gate_conv_gate(x, x[:, :4], x, h, 1, 8, 1, 16, fwd_kernel_cfg=cfg)
    with pytest.warns(UserWarning, match="Both autotune and fwd_kernel_cfg"):
        with pytest.raises(RuntimeError, match="no CPU path"):
            two_pass_chunked_gate_conv_gate(x, x, x, h, 1, 8, 1, 16, fwd_autotune=True, fwd_kernel_cfg=cfg)


def test_kernel_config_records():
    cfg = FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row")
    assert cfg.schedule == "default" and cfg.RETURN_BX and cfg.RETURN_Y2 and cfg.version == "refactor"
    assert cfg == FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row")
    assert hash(cfg) == hash(FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row"))
    assert "CHUNK_SIZE=128" in str(cfg)
    with pytest.raises(AssertionError):
        FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="diag")
    with pytest.raises(AssertionError):
        FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row", schedule="streamk")
    with pytest.raises(AssertionError):
        FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row", NUM_PIPELINE_STAGES=2)
    b = BwdKernelConfigRefactor()
    assert (b.pre_conv_BLOCK_X, b.post_conv_BLOCK_Y, b.name) == (128, 128, "bwd-refactor")


class _Spy:
    """Stands in for the kernel entry point to record how the operator calls it."""

    def __init__(self):
        self.kw = None

    def __call__(self, **kw):
        self.kw = kw
        return torch.zeros_like(kw["x"])


def test_operator_argument_mapping():
    """x1 -> C (post-gate), x2 -> B, v -> x; tensors and filter go through cgcg_dtype and the
    result comes back in the activation dtype as (b, l, g*dg) (hyena.py:494-534, :807-843)."""
    b, l, g, dg = 2, 16, 4, 16
    x1, x2, v = (torch.randn(b, l, g, dg, dtype=torch.bfloat16) for _ in range(3))
    for op in (hyena.HyenaMROperator(g * dg, g, hyena_mr_len=8, cfg=hyena.CgcgConfig(cgcg_dtype="float32")),
               hyena.HyenaSEOperator(g * dg, g, hyena_se_len=7, cfg=hyena.CgcgConfig(cgcg_dtype="float32"))):
        spy = _Spy()
        op.cgcg_fn = spy
        z = op(x1, x2, v)
        kw = spy.kw
        assert torch.equal(kw["x"], v.float()) and torch.equal(kw["B"], x2.float()) and torch.equal(kw["C"], x1.float())
        assert kw["h"].dtype == torch.float32 and kw["h"].shape[:2] == (g, 1)
        assert (kw["bs"], kw["seqlen"], kw["g"], kw["dg"]) == (b, l, g, dg)
        assert kw["fwd_autotune"] is False and kw["fwd_kernel_cfg"].BLOCK_D == dg
        assert kw["bwd_kernel_cfg"] is None and kw["bwd_autotune"] is True and kw["fused_bwd"] is True
        assert z.shape == (b, l, g * dg) and z.dtype == torch.bfloat16
    # no cast when the activation dtype already is cgcg_dtype
    op = hyena.HyenaSEOperator(g * dg, g, cfg=hyena.CgcgConfig(cgcg_dtype="bfloat16", cgcg_bwd_autotune=False))
    op = op.to(torch.bfloat16)
    spy = _Spy()
    op.cgcg_fn = spy
    op(x1, x2, v)
    assert spy.kw["x"] is v and spy.kw["C"] is x1 and spy.kw["bwd_kernel_cfg"] is not None


def test_explicit_filter_recipe():
    f = hyena.ExplicitSingleDecayFilter(8, 128, decay_preset="strong", small_init=False)
    h = f(128)
    assert h.shape == (8, 128)
    # decay = exp(-r_g * t), t in [0, 1], r_g = logspace(0, 2): first column undamped,
    # last column damped by exp(-r_g)
    torch.testing.assert_close(h[:, 0], f.h[:, 0])
    rates = torch.logspace(0, 2, 8)
    torch.testing.assert_close(h[:, -1], f.h[:, -1] * torch.exp(-rates))
    assert f(64).shape == (8, 64)
    assert hyena.get_groups_and_group_sizes(4096, 256) == (4096, 256, 16)
    assert hyena.get_groups_and_group_sizes(8192, 512, world_size=8) == (1024, 64, 16)


def test_interleaved_views_are_recognised_on_the_host():
    """The split of block.py:886-888 gives three stride-3 views of one buffer; the autograd boundary
    must find that buffer (and only then) so that it can skip the gathers."""
    import torch
    from einops import rearrange

    from savanna_amd.kernels.cgcg.interface import interleaved_source

    g, dg = 4, 16
    feats = torch.randn(2, 5, 3 * g * dg)
    x1, x2, v = rearrange(feats, "b l (g dg p) -> b l g p dg", p=3, g=g).unbind(dim=3)
    src = interleaved_source(x=v, B=x2, C=x1)
    assert src is not None and src.shape == (2, 5, g, dg, 3) and src.data_ptr() == feats.data_ptr()
    assert torch.equal(src[..., 0], x1) and torch.equal(src[..., 1], x2) and torch.equal(src[..., 2], v)
    # wrong order, gathered copies, a padded row stride, the non-interleaved split: not recognised
    assert interleaved_source(x=x1, B=x2, C=v) is None
    assert interleaved_source(x=v.contiguous(), B=x2, C=x1) is None
    padded = torch.randn(2, 5, 3 * g * dg + 3)[:, :, 3:]
    p1, p2, pv = rearrange(padded, "b l (g dg p) -> b l g p dg", p=3, g=g).unbind(dim=3)
    assert interleaved_source(x=pv, B=p2, C=p1) is None
    q1, q2, qv = rearrange(feats, "b l (p g dg) -> b l p g dg", p=3, g=g).unbind(dim=2)
    assert interleaved_source(x=qv, B=q2, C=q1) is None
    # an offset into a larger buffer is fine
    big = torch.randn(3, 5, 3 * g * dg)
    b1, b2, bv = rearrange(big[1:], "b l (g dg p) -> b l g p dg", p=3, g=g).unbind(dim=3)
    src = interleaved_source(x=bv, B=b2, C=b1)
    assert src is not None and src.data_ptr() == big[1:].data_ptr()


def test_planar_views_are_recognised_on_the_host():
    """The split without interleaving (block.py:881-884) gives three views whose rows lie 3 d elements apart;
    the autograd boundary must find their buffer, and only then."""
    import torch
    from einops import rearrange

    from savanna_amd.kernels.cgcg.interface import planar_source

    g, dg = 4, 16
    d = g * dg
    feats = torch.randn(2, 5, 3 * d)
    x1, x2, v = rearrange(feats, "b l (p g dg) -> b l p g dg", p=3, g=g).unbind(dim=2)
    src = planar_source(x=v, B=x2, C=x1)
    assert src is not None and src.shape == (2, 5, 3, g, dg) and src.data_ptr() == feats.data_ptr()
    assert torch.equal(src[:, :, 0], x1) and torch.equal(src[:, :, 1], x2) and torch.equal(src[:, :, 2], v)
    # wrong order, gathered copies, a padded row, the interleaved split, separate tensors: not recognised
    assert planar_source(x=x1, B=x2, C=v) is None
    assert planar_source(x=v.contiguous(), B=x2, C=x1) is None
    padded = torch.randn(2, 5, 3 * d + 8)[:, :, 8:]
    p1, p2, pv = rearrange(padded, "b l (p g dg) -> b l p g dg", p=3, g=g).unbind(dim=2)
    assert planar_source(x=pv, B=p2, C=p1) is None
    q1, q2, qv = rearrange(feats, "b l (g dg p) -> b l g p dg", p=3, g=g).unbind(dim=3)
    assert planar_source(x=qv, B=q2, C=q1) is None
    assert planar_source(x=torch.randn(2, 5, g, dg), B=torch.randn(2, 5, g, dg), C=torch.randn(2, 5, g, dg)) is None
    # an offset into a larger buffer is fine
    big = torch.randn(3, 5, 3 * d)
    b1, b2, bv = rearrange(big[1:], "b l (p g dg) -> b l p g dg", p=3, g=g).unbind(dim=2)
    src = planar_source(x=bv, B=b2, C=b1)
    assert src is not None and src.data_ptr() == big[1:].data_ptr()


def test_workspace_sizing_runs_on_the_host_for_any_shape(gcg_lib):
    """The *_workspace_bytes entry points are host arithmetic (launch plans): every shape, also a
    tensor narrower than a lane's vector, must give a 256-byte multiple or 0 -- never trap."""
    import itertools

    for bs, L, g, dg, hl, dt in itertools.product((1, 3), (1, 7, 4096), (1, 2, 4, 12288), (1, 2, 4, 16), (1, 3, 7, 128, 200),
                                                 (0, 1, 2)):
        for algo in (0, 1, 2, 3):
            n = gcg_lib.gcg_bwd_workspace_bytes(bs, L, g, dg, hl, dt, algo)
            assert n % 256 == 0
            if algo in (0, 1):
                assert n > 0, (bs, L, g, dg, hl, dt, algo)      # the direct family takes everything
        n = gcg_lib.gcg_dwconv_bwd_workspace_bytes(bs, L, g, dg, hl, dt)
        supported = hl <= 8 and (g * dg) % 4 == 0 and (dg == 1 or dg % 4 == 0)
        assert n % 256 == 0 and (n > 0) == supported, (bs, L, g, dg, hl, dt)
        assert gcg_lib.gcg_select_algo(bs, L, g, dg, hl, dt, 1) in (1, 2, 3)
        for kf in (1, 3, 4, 5):
            n = gcg_lib.gcg_mixer_se_bwd_workspace_bytes(bs, L, g, dg, hl, kf, dt)
            assert n % 256 == 0 and (n > 0) == (hl <= 8 and kf <= 4 and dg % 2 == 0), (bs, L, g, dg, hl, kf, dt)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU: asking for more ends with a message, before any device is touched."""
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode != 0
    assert "--gpus must be 1" in r.stderr + r.stdout
    assert "{" not in r.stdout                       # no result line


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the behaviour on a machine without a GPU")
def test_bench_has_no_cpu_path():
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "no GPU" in r.stderr + r.stdout
    assert "{" not in r.stdout


def test_route_predicates_follow_the_library_at_its_limits(gcg_lib):
    """gcg_route_supported answers on the host for every fused route, and the Python predicates that choose between
    a fused entry point and the general ones return what it returns -- also where the refusal comes from how far a
    tensor window reaches (very wide rows, a large batch of time-major rows), which the shape rules alone miss."""
    bf16, f32, mixed = _lib.dtype_code(torch.bfloat16), _lib.dtype_code(torch.float32), _lib.GCG_BF16_F32
    q = gcg_lib.gcg_route_supported
    # shape rules
    assert q(_lib.ROUTE_DECAY, 2, 8192, 256, 16, 128, 0, bf16) == 1
    assert q(_lib.ROUTE_DECAY, 2, 8192, 256, 16, 129, 0, bf16) == 0          # longer than the matrix-core band
    assert q(_lib.ROUTE_DECAY, 2, 8192, 256, 8, 128, 0, bf16) == 0           # groups narrower than a tile
    assert q(_lib.ROUTE_TIME_MAJOR, 16, 8192, 48, 16, 7, 0, bf16) == 1       # the reference's run_short_hyena test shape
    assert q(_lib.ROUTE_TIME_MAJOR, 16, 8192, 48, 16, 9, 0, bf16) == 0
    assert q(_lib.ROUTE_MIXER_SE, 1, 32768, 512, 16, 7, 3, bf16) == 1
    assert q(_lib.ROUTE_MIXER_SE, 1, 32768, 512, 16, 7, 5, bf16) == 0        # featurizer longer than the kernels take
    assert q(_lib.ROUTE_MIXER_MR, 2, 8192, 256, 16, 128, 3, bf16) == 1
    assert q(_lib.ROUTE_MIXER_MR, 2, 8192, 256, 16, 128, 3, mixed) == 1      # fp32 arithmetic: the two-kernel form
    assert q(_lib.ROUTE_MIXER_MR_PLANAR, 2, 8192, 256, 16, 128, 3, bf16) == 1
    assert q(_lib.ROUTE_MIXER_MR_PLANAR, 2, 8192, 256, 16, 128, 3, mixed) == 0   # planar features: one-kernel form only
    assert q(_lib.ROUTE_MIXER_MR_PLANAR, 2, 8192, 256, 16, 128, 3, f32) == 0
    assert q(_lib.ROUTE_MIXER_MR, 2, 8192, 256, 16, 128, 0, bf16) == -1      # a mixer route needs the featurizer's length
    assert q(99, 2, 8192, 256, 16, 128, 3, bf16) == -1 and q(_lib.ROUTE_DECAY, 0, 8192, 256, 16, 128, 0, bf16) == -1
    # window limits: rows too wide for the shortest run with its lead-in to fit one tensor window
    wide_g = 1 << 17                                                        # d = 2 M channels
    assert q(_lib.ROUTE_DECAY, 1, 4096, wide_g, 16, 128, 0, bf16) == 0
    assert q(_lib.ROUTE_MIXER_MR, 1, 4096, wide_g, 16, 128, 3, bf16) == 0
    assert q(_lib.ROUTE_TIME_MAJOR, 4096, 64, 4096, 16, 7, 0, bf16) == 0     # bs * d elements per time row
    assert q(_lib.ROUTE_TIME_MAJOR, 4, 64, 4096, 16, 7, 0, bf16) == 1
    # the predicates: same answers (meta tensors carry the shapes; alignment is not in question here)
    def meta(*shape):
        return torch.empty(*shape, dtype=torch.bfloat16, device="meta")
    import unittest.mock as mock
    with mock.patch.object(_lib, "_all_aligned16", lambda *a, **k: True):
        assert _lib.time_major_supported(16, 7, meta(64, 4, 4096, 16))
        assert not _lib.time_major_supported(16, 7, meta(64, 4096, 4096, 16))
        assert _lib.decay_supported(256, 16, 128, meta(2, 8192, 256, 16))
        assert not _lib.decay_supported(wide_g, 16, 128, meta(1, 4096, wide_g, 16))
        assert _lib.mixer_mr_supported(16, 128, 3, sizes=(2, 8192, 256, bf16))
        assert not _lib.mixer_mr_supported(16, 128, 3, sizes=(1, 4096, wide_g, bf16))
        assert not _lib.mixer_mr_supported(16, 128, 3, planar=True, sizes=(2, 8192, 256, mixed))
        assert _lib.mixer_mr_supported(16, 128, 3)                           # shape rules only, as before
