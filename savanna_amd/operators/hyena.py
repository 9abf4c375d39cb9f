"""Operator dispatch for the gated convolution: the callers of the kernel boundary.

Counterparts of the ``use_cgcg`` branches of savanna's hyena operators, calling the HIP
kernels directly:

* ``HyenaMROperator``  <- ParallelHyenaOperator.forward, medium-cgcg branch
  (savanna/model/operators/hyena/hyena.py:483-535; config built at :270-293)
* ``HyenaSEOperator``  <- ParallelShortHyenaOperator.forward, cgcg short / mlp branch
  (hyena.py:795-844; config built at :657-697)

What is reproduced: the argument mapping (x1 -> C post-gate, x2 -> B, v -> x), the round trip
through ``cgcg_dtype``, the filter shapes ((g, L_cache) explicit decayed filter cut to
``hyena_mr_len``; (g, 1, hl) short filter), the kernel-config records, and the output reshape
to (b, l, g*dg).  As in the reference's cgcg branch the convolution is a cross-correlation
without the ``conv_bias`` skip term (the non-cgcg branches differ, hyena.py:477-478, 544-555).
Everything model-parallel, context-parallel or FFT-based in those classes is outside this
path and absent here.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn

from .. import _lib
from ..kernels.cgcg.interface import (DecayedGateConvGate, InterleavedDecayedGateConvGate,
                                       planar_source, two_pass_chunked_gate_conv_gate,
                                       two_pass_chunked_gate_conv_gate_interleaved,
                                       two_pass_chunked_gate_conv_gate_planar)
from ..kernels.cgcg.src.kernel_utils import BwdKernelConfigRefactor, FwdKernelConfigRefactor

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def get_groups_and_group_sizes(hidden_size: int, num_groups: int, world_size: int = 1, expand_factor: float = 1):
    """(width per rank, groups per rank, channels per group) as hyena.py:184-188; world_size is
    1 on this single-GPU path."""
    assert hidden_size % world_size == 0 and num_groups % world_size == 0
    width = hidden_size // world_size
    groups = int(num_groups // world_size * expand_factor)
    return width, groups, width // groups


@dataclass
class CgcgConfig:
    """The flags of savanna/arguments/global_config.py that reach this path (:389-523),
    with the reference's defaults."""
    cgcg_dtype: str = "float32"                 # global_config.py:404; the 7B configs set "bfloat16"
    cgcg_fwd_chunk_size: int = 128              # :417-440 (medium) / :445-468 (short): Triton tile knobs
    cgcg_fwd_block_d: int = 128
    cgcg_fwd_chunk_tiles_per_program: int = 1
    cgcg_fwd_threadblock_swizzle: str = "row"
    cgcg_fwd_num_warps: int = 4
    cgcg_fwd_num_stages: int = 3
    cgcg_bwd_autotune: bool = True              # :473
    cgcg_fused_bwd: bool = True                 # :478
    cgcg_bwd_pre_conv_block_x: int = 128        # :485-520
    cgcg_bwd_pre_conv_block_y: int = 128
    cgcg_bwd_pre_conv_num_warps: int = 8
    cgcg_bwd_post_conv_block_x: int = 32
    cgcg_bwd_post_conv_block_y: int = 128
    cgcg_bwd_post_conv_num_warps: int = 4

    def torch_dtype(self) -> torch.dtype:
        return _DTYPES[self.cgcg_dtype]

    def fwd_kernel_cfg(self, group_dim: int) -> FwdKernelConfigRefactor:
        # BLOCK_D = min(group_dim, configured) as hyena.py:279, :664
        return FwdKernelConfigRefactor(
            CHUNK_SIZE=self.cgcg_fwd_chunk_size,
            BLOCK_D=min(group_dim, self.cgcg_fwd_block_d),
            CHUNK_TILES_PER_PROGRAM=self.cgcg_fwd_chunk_tiles_per_program,
            THREADBLOCK_SWIZZLE=self.cgcg_fwd_threadblock_swizzle,
            num_warps=self.cgcg_fwd_num_warps,
            num_stages=self.cgcg_fwd_num_stages,
        )

    def bwd_kernel_cfg(self) -> BwdKernelConfigRefactor:
        return BwdKernelConfigRefactor(
            pre_conv_BLOCK_X=self.cgcg_bwd_pre_conv_block_x,
            pre_conv_BLOCK_Y=self.cgcg_bwd_pre_conv_block_y,
            pre_conv_num_warps=self.cgcg_bwd_pre_conv_num_warps,
            post_conv_BLOCK_X=self.cgcg_bwd_post_conv_block_x,
            post_conv_BLOCK_Y=self.cgcg_bwd_post_conv_block_y,
            post_conv_num_warps=self.cgcg_bwd_post_conv_num_warps,
        )


class ExplicitSingleDecayFilter(nn.Module):
    """h[g, t] = w[g, t] * exp(-r_g * t / (L_cache - 1)), r_g log-spaced over the groups
    (savanna/model/operators/hyena/parametrization/explicit.py:15-75, single rank)."""

    PRESETS = {"strong": (0, 2), "normal": (-1, 2), "weak": (-2, 2)}

    def __init__(self, d_model: int, L_cache: int, decay_preset: str = "strong", small_init: bool = True,
                 unit_passthrough: bool = False, device=None):
        super().__init__()
        assert decay_preset in self.PRESETS
        log_r_min, log_r_max = self.PRESETS[decay_preset]
        w = torch.randn(d_model, L_cache, device=device) / math.sqrt(L_cache)
        if small_init:
            w = w * 1e-5
        if unit_passthrough:
            w[:, :1] = 1.0
        self.h = nn.Parameter(w)
        t = torch.linspace(0, 1, L_cache, device=device)[None]
        rates = torch.logspace(log_r_min, log_r_max, d_model, device=device)[:, None]
        self.register_buffer("decay", torch.exp(-rates * t))

    def forward(self, L: int) -> torch.Tensor:
        return self.h[:, :L] * self.decay[:, :L]

    def fused(self, L: int, dtype: torch.dtype) -> torch.Tensor:
        """(g, 1, L) filter in ``dtype`` for the convolution kernels: slice, product and cast in one
        launch, and one launch for their backward (fp32 parameters on the GPU)."""
        return _DecayedFilter.apply(self.h, self.decay, L, dtype)


class _DecayedFilter(torch.autograd.Function):
    @staticmethod
    def forward(ctx, w, decay, hl, dtype):
        ctx.save_for_backward(decay)
        return _lib.filter_decay_fwd(w.contiguous(), decay.contiguous(), hl, dtype)

    @staticmethod
    def backward(ctx, dh):
        (decay,) = ctx.saved_tensors
        return _lib.filter_decay_bwd(dh.contiguous(), decay.contiguous()), None, None, None


class _CgcgOperatorBase(nn.Module):
    def __init__(self, hidden_size: int, num_groups: int, cfg: Optional[CgcgConfig]):
        super().__init__()
        self.cfg = cfg or CgcgConfig()
        self.hidden_size, self.num_groups, self.group_dim = get_groups_and_group_sizes(hidden_size, num_groups)
        self.cgcg_dtype = self.cfg.torch_dtype()
        self.cgcg_fn = two_pass_chunked_gate_conv_gate
        self.cgcg_fwd_config = self.cfg.fwd_kernel_cfg(self.group_dim)
        self.cgcg_bwd_config = self.cfg.bwd_kernel_cfg()

    def _filter(self, L: int) -> torch.Tensor:          # (g, 1, hl)
        raise NotImplementedError

    def forward(self, x1: torch.Tensor, x2: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """x1 (post-gate), x2, v (pre-gate pair): (b, l, g, dg) -> z: (b, l, g*dg)."""
        dtype = x1.dtype
        fused = self._filter_in_kernel(x1.shape[1], x1.shape[2], x1.shape[3], dtype, x1, x2, v)
        if fused is not None:
            hl, filt = fused
            z = DecayedGateConvGate.apply(v, x2, x1, self.filter.h, self.filter.decay, hl, filt)
            return z.reshape(z.shape[0], z.shape[1], -1)
        h = self._filter(x1.shape[1])
        x, B, C = v, x2, x1
        cast = self.cgcg_dtype != dtype
        if cast and self._fp32_inside(dtype, x1):
            # hyena.py:499-503, :533-534 cast the three tensors up and the result down around the call; here the
            # kernels read the 16-bit tensors, keep the filter and all arithmetic in fp32, and round the result once
            h, cast = h.to(torch.float32), False
        elif cast:
            x, B, C, h = (t.to(self.cgcg_dtype) for t in (v, x2, x1, h))
        else:
            h = h.to(dtype)             # parameters kept in another precision than the activations
        bs, seqlen, g, dg = x.shape
        z = self.cgcg_fn(
            x=x, B=B, C=C, h=h, bs=bs, seqlen=seqlen, g=g, dg=dg,
            fwd_autotune=False,
            bwd_autotune=self.cfg.cgcg_bwd_autotune,
            fused_bwd=self.cfg.cgcg_fused_bwd,
            fwd_kernel_cfg=self.cgcg_fwd_config,
            bwd_kernel_cfg=None if self.cfg.cgcg_bwd_autotune else self.cgcg_bwd_config,
        )
        z = z.reshape(bs, seqlen, g * dg)
        return z.to(dtype) if cast else z

    def _filter_in_kernel(self, L, g, dg, dtype, *tensors):
        """(hl, filter dtype) when the convolution kernels can form the decayed filter themselves, else None."""
        return None

    def _fp32_inside(self, dtype: torch.dtype, t: torch.Tensor) -> bool:
        """16-bit activations with ``cgcg_dtype`` float32 on the GPU: one kernel instead of casts around it."""
        return self.cgcg_dtype == torch.float32 and dtype in (torch.bfloat16, torch.float16) and t.is_cuda

    def forward_features(self, features: torch.Tensor, from_featurizer: bool = False,
                         interleaved: bool = True) -> torch.Tensor:
        """The same on the projected features before their split: (b, l, 3*g*dg) laid out
        "(g dg p)" with p = (x1, x2, v) fastest (block.py:886-888) -> z: (b, l, g*dg).  The kernels
        read the tensor as it is and the backward writes its gradient in the same layout.
        ``from_featurizer``: the gradient goes straight into the featurizer's backward (cache hint).
        ``interleaved=False``: the layout is "(p g dg)", the split of block.py:881-884 for checkpoints trained
        without interleaving; the kernels then read the thirds of each row in place."""
        dtype = features.dtype
        bs, seqlen, d3 = features.shape
        g, dg = self.num_groups, self.group_dim
        assert d3 == 3 * g * dg
        if not interleaved:
            h = self._filter(seqlen)
            cast = self.cgcg_dtype != dtype and not self._fp32_inside(dtype, features)
            if cast:
                features = features.to(self.cgcg_dtype)
            z = two_pass_chunked_gate_conv_gate_planar(features, h.to(self.cgcg_dtype), bs, seqlen, g, dg)
            z = z.reshape(bs, seqlen, g * dg)
            return z.to(dtype) if cast else z
        fused = self._filter_in_kernel(seqlen, g, dg, dtype, features)
        if fused is not None:
            hl, filt = fused
            z = InterleavedDecayedGateConvGate.apply(features.reshape(bs, seqlen, g, dg, 3), self.filter.h,
                                                     self.filter.decay, hl, filt, from_featurizer)
            return z.reshape(bs, seqlen, g * dg)
        h = self._filter(seqlen)
        cast = self.cgcg_dtype != dtype and not self._fp32_inside(dtype, features)
        if cast:
            features = features.to(self.cgcg_dtype)
        z = two_pass_chunked_gate_conv_gate_interleaved(features, h.to(self.cgcg_dtype), bs, seqlen, g, dg,
                                                        keep_dfeatures=from_featurizer)
        z = z.reshape(bs, seqlen, g * dg)
        return z.to(dtype) if cast else z


class HyenaMROperator(_CgcgOperatorBase):
    """Hyena-MR: explicit decayed filter of length ``hyena_mr_len`` (128 in the 7B configs)."""

    def __init__(self, hidden_size: int, num_groups: int, hyena_mr_len: int = 128, cfg: Optional[CgcgConfig] = None,
                 decay_preset: str = "strong", small_init: bool = True, device=None, fuse_filter: bool = True):
        super().__init__(hidden_size, num_groups, cfg)
        self.hyena_mr_len = hyena_mr_len
        self.fuse_filter = fuse_filter       # form the filter inside the convolution kernels where they can
        self.filter = ExplicitSingleDecayFilter(self.num_groups, hyena_mr_len, decay_preset=decay_preset,
                                                small_init=small_init, device=device)

    def _filter_in_kernel(self, L, g, dg, dtype, *tensors):
        w = self.filter.h
        if not (self.fuse_filter and w.is_cuda and w.dtype == torch.float32 and all(t.is_cuda for t in tensors)):
            return None
        if self.cgcg_dtype != dtype and not self._fp32_inside(dtype, tensors[0]):
            return None                                             # a cast the kernels do not fold
        hl = min(self.hyena_mr_len, L)
        if not _lib.decay_supported(g, dg, hl, *tensors):
            return None
        if len(tensors) == 3 and not torch.compiler.is_compiling() and \
                planar_source(tensors[2], tensors[1], tensors[0]) is not None:
            return None         # the split without interleaving: the planar entry points take an explicit filter
        return hl, self.cgcg_dtype

    def _filter(self, L: int) -> torch.Tensor:
        hl = min(self.hyena_mr_len, L)                              # hyena.py:440-441, :503
        if self.filter.h.is_cuda and self.filter.h.dtype == torch.float32:
            return self.filter.fused(hl, self.cgcg_dtype)
        return self.filter(hl)[:, None]


class HyenaSEOperator(_CgcgOperatorBase):
    """Hyena-SE: short explicit filter (g, 1, hl), hl = ``hyena_se_len`` (7 in the 7B configs);
    initialised uniform(+-sqrt(1/hl)) like short_conv_weight (hyena.py:120-130)."""

    def __init__(self, hidden_size: int, num_groups: int, hyena_se_len: int = 7, cfg: Optional[CgcgConfig] = None,
                 device=None):
        super().__init__(hidden_size, num_groups, cfg)
        bound = math.sqrt(1.0 / hyena_se_len)
        self.short_conv_weight = nn.Parameter(
            torch.empty(self.num_groups, 1, hyena_se_len, device=device).uniform_(-bound, bound))

    def _filter(self, L: int) -> torch.Tensor:
        return self.short_conv_weight


class _CausalDepthwiseConv(torch.autograd.Function):
    """y[b, t, c] = sum_k w[c / dg, 0, k] x[b, t - (K-1) + k, c] on (b, l, g, dg) tensors."""

    @staticmethod
    def forward(ctx, x, w, feeds_operator=False):
        x = x if x.is_contiguous() else x.contiguous()
        w = w if w.is_contiguous() else w.contiguous()
        ctx.save_for_backward(x, w)
        return _lib.dwconv_fwd(x, w, keep_output=feeds_operator)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        return _lib.dwconv_bwd(dy if dy.is_contiguous() else dy.contiguous(), x, w) + (None,)


class CausalDepthwiseConv1d(nn.Module):
    """The featurizer conv of the hyena blocks: counterpart of ParallelCausalDepthwiseConv1d
    (savanna/model/operators/hyena/hyena.py:76-181) on its torch path (:159-176), i.e. left
    zero padding of K-1 and a cross-correlation, one filter per channel unless ``num_groups``
    shares them ((num_groups, 1, K) weight, hyena.py:99-110, uniform(+-sqrt(1/K)) init, :128-130).

    The reference module works on (B, D, L) and the block permutes around it (block.py:867-876);
    ``forward_bld`` takes and returns (B, L, D) -- the layout of the projection before it and of
    the interleaved operator after it -- and ``forward`` keeps the reference's (B, D, L) contract.
    """

    def __init__(self, d_model: int, kernel_size: int = 3, num_groups: Optional[int] = None,
                 dtype=torch.float32, device=None):
        super().__init__()
        self.d_model, self.kernel_size = d_model, kernel_size
        self.num_groups = d_model if num_groups is None else num_groups
        assert d_model % self.num_groups == 0
        self.group_dim = d_model // self.num_groups
        bound = math.sqrt(1.0 / kernel_size)
        w = torch.empty(self.num_groups, 1, kernel_size, dtype=dtype, device=device).uniform_(-bound, bound)
        self.short_conv_weight = nn.Parameter(w)

    def forward_bld(self, x: torch.Tensor, feeds_operator: bool = False) -> torch.Tensor:
        """``feeds_operator``: the result goes straight into the interleaved operator; it is then stored
        through the cache, where part of it still is when that kernel starts (same values either way)."""
        b, l, d = x.shape
        assert d == self.d_model
        y = _CausalDepthwiseConv.apply(x.reshape(b, l, self.num_groups, self.group_dim),
                                       self.short_conv_weight.to(x.dtype), feeds_operator)
        return y.reshape(b, l, d)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.forward_bld(x.permute(0, 2, 1)).permute(0, 2, 1)


class _FeaturizedShortGateConvGate(torch.autograd.Function):
    """z = gated short convolution of the featurized projection, raw (b, l, g, dg, 3) -> (b, l, g, dg),
    in one kernel each way; the featurized tensor exists in registers only.  ``planar``: raw is (b, l, 3, g, dg)."""

    @staticmethod
    def forward(ctx, raw, wf, h, planar=False):
        raw, wf, h = (t if t.is_contiguous() else t.contiguous() for t in (raw, wf, h))
        ctx.save_for_backward(raw, wf, h)
        ctx.planar = planar
        return _lib.mixer_se_fwd(raw, wf, h, planar)

    @staticmethod
    def backward(ctx, dz):
        raw, wf, h = ctx.saved_tensors
        return _lib.mixer_se_bwd(dz if dz.is_contiguous() else dz.contiguous(), raw, wf, h, ctx.planar) + (None,)


class _FeaturizedGateConvGate(torch.autograd.Function):
    """z = gated Hyena-MR convolution of the featurized projection, raw (b, l, g, dg, 3) -> (b, l, g, dg), without
    the featurized tensor: the forward makes its rows on the way, the backward recomputes them from raw and hands
    their gradient to the featurizer's backward inside the same call.  Only raw, wf and h are saved.
    ``planar``: raw is (b, l, 3, g, dg)."""

    @staticmethod
    def forward(ctx, raw, wf, h, planar=False):
        raw, wf, h = (t if t.is_contiguous() else t.contiguous() for t in (raw, wf, h))
        ctx.save_for_backward(raw, wf, h)
        ctx.planar = planar
        return _lib.mixer_mr_fwd(raw, wf, h, planar)

    @staticmethod
    def backward(ctx, dz):
        raw, wf, h = ctx.saved_tensors
        return _lib.mixer_mr_bwd(dz if dz.is_contiguous() else dz.contiguous(), raw, wf, h, ctx.planar) + (None,)


class _FeaturizedDecayedGateConvGate(torch.autograd.Function):
    """_FeaturizedGateConvGate with the filter F(w * decay)[:, :hl] formed inside the kernels, F the cast to ``filt``
    (ExplicitSingleDecayFilter.filter, explicit.py:68-75; hyena.py:499-503): a Hyena-MR layer's convolutional
    part is one kernel each way, and the backward returns the gradient of the filter parameter itself."""

    @staticmethod
    def forward(ctx, raw, wf, w, decay, hl, filt, planar=False):
        raw, wf, w, decay = (t if t.is_contiguous() else t.contiguous() for t in (raw, wf, w, decay))
        ctx.save_for_backward(raw, wf, w, decay)
        ctx.hl, ctx.filt, ctx.planar = hl, filt, planar
        return _lib.mixer_mr_fwd_decay(raw, wf, w, decay, hl, filt, planar)

    @staticmethod
    def backward(ctx, dz):
        raw, wf, w, decay = ctx.saved_tensors
        draw, dwf, dw = _lib.mixer_mr_bwd_decay(dz if dz.is_contiguous() else dz.contiguous(), raw, wf, w, decay,
                                                ctx.hl, ctx.filt, ctx.planar)
        return draw, dwf, dw, None, None, None, None


class HyenaMixer(nn.Module):
    """The convolutional part of ParallelSequenceMixer.forward for the hyena operators
    (savanna/model/block.py:865-890): featurizer conv on the projected features, interleaved split,
    gated convolution.  Input (b, l, 3*hidden) -- what the dense projection writes -- output
    (b, l, hidden) for the output projection; no permute, gather or split copy in between.

    With a short operator filter (Hyena-SE: at most 8 taps, featurizer of at most 4, one filter per
    feature channel) the two convolutions run as one kernel each way (``fuse_short``); the result
    differs from the two-kernel chain by the rounding of fp32 sums only.  With a Hyena-MR filter
    (9 to 128 taps) and a featurizer of at most 3 taps the featurized tensor is never stored (``fuse_medium``):
    the operator's kernels make its rows from the projection output, forward and backward, with the chain's results,
    and form the decayed filter themselves where the operator allows it (``HyenaMROperator.fuse_filter``).
    ``interleave_projections=False`` takes the features laid out "(p g dg)" instead (block.py:881-884)."""

    def __init__(self, operator: _CgcgOperatorBase, short_conv_L: int = 3, dtype=torch.float32, device=None,
                 fuse_short: bool = True, fuse_medium: bool = True, interleave_projections: bool = True):
        super().__init__()
        self.mixer = operator
        self.fuse_short = fuse_short
        self.fuse_medium = fuse_medium
        self.interleave_projections = interleave_projections        # global_config.py:270
        self.hyena_proj_conv = CausalDepthwiseConv1d(3 * operator.hidden_size, short_conv_L, dtype=dtype, device=device)

    def _fusable(self, features: torch.Tensor, hl: int) -> bool:
        conv, op = self.hyena_proj_conv, self.mixer
        return (self.fuse_short and features.is_cuda and hl <= 8 and conv.kernel_size <= 4 and conv.group_dim == 1
                and op.group_dim % 2 == 0)

    def _fused_short(self, features: torch.Tensor, h: torch.Tensor, planar: bool) -> torch.Tensor:
        """Featurizer and Hyena-SE operator in one kernel each way.  16-bit features with ``cgcg_dtype`` float32 stay
        16-bit: the kernels round the featurizer's output to the features' type, as the conv of block.py:873 stores
        it before the casts of hyena.py:812-816, and keep the filter and the operator's arithmetic in fp32."""
        op = self.mixer
        bs, seqlen, _ = features.shape
        g, dg = op.num_groups, op.group_dim
        dtype = features.dtype
        inside = op.cgcg_dtype != dtype and op._fp32_inside(dtype, features)
        cast = op.cgcg_dtype != dtype and not inside
        if cast:
            features = features.to(op.cgcg_dtype)
        shape = (bs, seqlen, 3, g, dg) if planar else (bs, seqlen, g, dg, 3)
        z = _FeaturizedShortGateConvGate.apply(features.reshape(shape),
                                               self.hyena_proj_conv.short_conv_weight.to(features.dtype),
                                               h.to(op.cgcg_dtype), planar)
        z = z.reshape(bs, seqlen, g * dg)
        return z.to(dtype) if cast else z

    def _mixer_code(self, features: torch.Tensor) -> int:
        """The library's dtype code for the mixer's call on these features: their own type, or 16-bit tensors with
        fp32 arithmetic, or -- features cast to ``cgcg_dtype`` around the call -- that type."""
        op = self.mixer
        if op.cgcg_dtype == features.dtype:
            return _lib.dtype_code(features.dtype)
        if op._fp32_inside(features.dtype, features):
            return _lib.GCG_BF16_F32 if features.dtype == torch.bfloat16 else _lib.GCG_F16_F32
        return _lib.dtype_code(op.cgcg_dtype)

    def _medium(self, features: torch.Tensor, hl: int) -> bool:
        """Whether the one-kernel Hyena-MR mixer takes these features with a filter of ``hl`` taps.  Planar features
        ("(p g dg)" rows) run in the one-kernel form only, which has 16-bit arithmetic."""
        conv, op = self.hyena_proj_conv, self.mixer
        if not (self.fuse_medium and features.is_cuda and conv.group_dim == 1 and
                _lib.mixer_mr_supported(op.group_dim, hl, conv.kernel_size, features,
                                        planar=not self.interleave_projections,
                                        sizes=(features.shape[0], features.shape[1], op.num_groups,
                                               self._mixer_code(features)))):
            return False
        if self.interleave_projections:
            return op.cgcg_dtype == features.dtype or op._fp32_inside(features.dtype, features)
        return op.cgcg_dtype == features.dtype and features.dtype in (torch.bfloat16, torch.float16)

    def forward(self, features: torch.Tensor) -> torch.Tensor:
        op, conv = self.mixer, self.hyena_proj_conv
        bs, seqlen, d3 = features.shape
        g, dg = op.num_groups, op.group_dim
        assert d3 == 3 * g * dg
        planar = not self.interleave_projections
        shape = (bs, seqlen, 3, g, dg) if planar else (bs, seqlen, g, dg, 3)
        # Hyena-MR: one kernel each way, with the decayed filter formed inside it where the operator allows that
        fused = op._filter_in_kernel(seqlen, g, dg, features.dtype, features)
        if fused is not None and self._medium(features, fused[0]):
            z = _FeaturizedDecayedGateConvGate.apply(features.reshape(shape), conv.short_conv_weight.to(features.dtype),
                                                     op.filter.h, op.filter.decay, fused[0], fused[1], planar)
            return z.reshape(bs, seqlen, g * dg)
        h = op._filter(seqlen)
        if self._medium(features, h.shape[-1]):
            z = _FeaturizedGateConvGate.apply(features.reshape(shape), conv.short_conv_weight.to(features.dtype),
                                              h.to(op.cgcg_dtype), planar)
            return z.reshape(bs, seqlen, g * dg)
        # Hyena-SE: one kernel each way
        if self._fusable(features, h.shape[-1]):
            return self._fused_short(features, h, planar)
        # otherwise the featurizer kernel, then the operator on its output where it lies (two kernels each way)
        return op.forward_features(conv.forward_bld(features, feeds_operator=True), from_featurizer=True,
                                   interleaved=not planar)
