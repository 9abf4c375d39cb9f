"""Synthetic workloads: the five benchmark configurations and their input recipe.

Naming: the workload descriptions speak of q, k (pre-gate pair) and v (post-gate);
the kernel arguments are B = q, x = k, C = v  (y = v * conv(q * k, h)).

Inputs are drawn on the CPU from ``torch.Generator().manual_seed(seed)`` in fp32 in the
fixed order q, k, v, filter noise w, filter decay a, dy, then cast and copied, so a
CPU checker and the GPU see bit-identical values.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    bs: int
    L: int
    g: int
    dg: int
    filters: Tuple[int, ...]      # filter lengths of the ops applied in sequence
    dtype: torch.dtype
    backward: bool
    about: str
    # "planar": q, k, v are the thirds of the rows of one (bs, L, 3, g, dg) tensor, read in place.
    # "separate": q, k, v are three contiguous tensors.  "interleaved": they are the thirds of one
    # (bs, L, g, dg, 3) projected-features tensor and the kernels read it as it is.  "gathered": same
    # features tensor, handled the way the reference does (three strided gathers before the forward,
    # re-assembly of the feature gradient after the backward) around the separate-tensor kernels.
    # "dwconv": the ungated featurizer conv on one (bs, L, g, dg) tensor.
    # "mixer": featurizer conv then the operator on the interleaved features, all on (bs, L, 3d);
    # "mixer_fused": the same result from the one-pass kernels (short operator filters only);
    # "mixer_reference_flow": the same chain as block.py:865-890 runs it -- permute to (B, 3D, L),
    # F.pad + F.conv1d, permute back, interleaved split, three gathers -- around the separate-tensor
    # kernels, with autograd doing the backward of the torch part.
    layout: str = "separate"
    # the filter's dtype where it is not the tensors': float32 with 16-bit tensors = cgcg_dtype float32 on 16-bit
    # activations (fp32 filter, arithmetic and filter gradient; hyena.py:499-503, :812-816)
    filt_dtype: Optional[torch.dtype] = None

    @property
    def d(self) -> int:
        return self.g * self.dg

    @property
    def tokens(self) -> int:
        return self.bs * self.L

    @property
    def elem_bytes(self) -> int:
        return torch.empty((), dtype=self.dtype).element_size()

    def algorithmic_bytes(self) -> int:
        if self.layout.startswith("mixer"):
            # forward: read raw features 3N, write y N; backward: read dy N and raw features 3N, write d features 3N
            return (11 if self.backward else 4) * self.bs * self.L * self.d * self.elem_bytes * len(self.filters)
        if self.layout == "dwconv":      # ungated: forward reads x, writes y; backward reads dy, x, writes dx
            return (5 if self.backward else 2) * self.bs * self.L * self.d * self.elem_bytes * len(self.filters)
        return self._gated_bytes()

    def _gated_bytes(self) -> int:
        """Compulsory HBM traffic of one pass: forward reads q, k, v and writes y (4
        tensors); forward+backward adds reads of dy, q, k, v and writes of dq, dk, dv
        (11 tensors).  Filter and filter-gradient traffic (<= 256 KB) is not counted."""
        per_op = 11 if self.backward else 4
        return per_op * self.bs * self.L * self.d * self.elem_bytes * len(self.filters)

    def algorithmic_flops(self) -> int:
        """2*bs*L*hl*d per convolution pass, three passes for forward+backward
        (savanna/mfu.py:423-431, :113-124)."""
        passes = 3 if self.backward else 1
        return sum(2 * self.bs * self.L * hl * self.d * passes for hl in self.filters)


WORKLOADS = {
    "se_fwd_fp32": Workload("se_fwd_fp32", 1, 2048, 16, 16, (7,), torch.float32, False,
                            "Hyena-SE forward, fp32, B=1 L=2048 D=256 G=16 hl=7"),
    "mr_fwd_7b": Workload("mr_fwd_7b", 2, 8192, 256, 16, (128,), torch.bfloat16, False,
                          "Hyena-MR forward, bf16, Evo2-7B layer shape B=2 L=8192 D=4096 G=256 hl=128"),
    "mr_fwdbwd_7b": Workload("mr_fwdbwd_7b", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                             "Hyena-MR forward+backward, bf16, Evo2-7B layer shape B=2 L=8192 D=4096 G=256 hl=128"),
    "se_mr_fwdbwd_40b": Workload("se_mr_fwdbwd_40b", 1, 32768, 512, 16, (7, 128), torch.bfloat16, True,
                                 "Hyena-SE then Hyena-MR forward+backward, bf16, B=1 L=32768 D=8192 G=512"),
    "mr_fwd_1m": Workload("mr_fwd_1m", 1, 1048576, 256, 16, (128,), torch.bfloat16, False,
                          "Hyena-MR forward, bf16, B=1 L=1048576 D=4096 G=256 hl=128"),
    # the shapes the reference's own benchmark scripts use (cgcg/tests/benchmark-7b.sh, benchmark-40b.sh)
    "ref_bench_7b": Workload("ref_bench_7b", 8, 8192, 256, 16, (128,), torch.bfloat16, True,
                             "Hyena-MR forward+backward, bf16, B=8 L=8192 D=4096 G=256 hl=128"),
    "ref_bench_40b": Workload("ref_bench_40b", 2, 8192, 512, 16, (7,), torch.bfloat16, True,
                              "Hyena-SE forward+backward, bf16, B=2 L=8192 D=8192 G=512 hl=7"),
    # Hyena-MR at the 7B layer shape fed from the interleaved projected features (block.py:886-890)
    "mr_fwdbwd_7b_interleaved": Workload("mr_fwdbwd_7b_interleaved", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                                         "Hyena-MR forward+backward on interleaved features, bf16, B=2 L=8192 D=4096 "
                                         "G=256 hl=128", layout="interleaved"),
    "mr_fwdbwd_7b_gathered": Workload("mr_fwdbwd_7b_gathered", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                                      "the same with the reference's data flow: three gathers, separate-tensor "
                                      "kernels, feature gradient re-assembled", layout="gathered"),
    "se_fwdbwd_40b_interleaved": Workload("se_fwdbwd_40b_interleaved", 1, 32768, 512, 16, (7,), torch.bfloat16, True,
                                          "Hyena-SE forward+backward on interleaved features, bf16, B=1 L=32768 "
                                          "D=8192 G=512 hl=7", layout="interleaved"),
    # the same two on planar features, the split without interleaving (block.py:881-884, interleave_projections = false)
    "mr_fwdbwd_7b_planar": Workload("mr_fwdbwd_7b_planar", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                                    "Hyena-MR forward+backward on planar features (the thirds of each row read in "
                                    "place), bf16, B=2 L=8192 D=4096 G=256 hl=128", layout="planar"),
    "se_fwdbwd_40b_planar": Workload("se_fwdbwd_40b_planar", 1, 32768, 512, 16, (7,), torch.bfloat16, True,
                                     "Hyena-SE forward+backward on planar features, bf16, B=1 L=32768 D=8192 G=512 "
                                     "hl=7", layout="planar"),
    "se_fwdbwd_40b_gathered": Workload("se_fwdbwd_40b_gathered", 1, 32768, 512, 16, (7,), torch.bfloat16, True,
                                       "the same with three gathers, separate-tensor kernels and re-assembly",
                                       layout="gathered"),
    # the featurizer conv of a 7B layer: 3 * 4096 channels, one 3-tap filter per channel (block.py:873)
    "featurizer_fwdbwd_7b": Workload("featurizer_fwdbwd_7b", 2, 8192, 12288, 1, (3,), torch.bfloat16, True,
                                     "featurizer conv forward+backward, bf16, B=2 L=8192 channels=12288, one 3-tap "
                                     "filter per channel", layout="dwconv"),
    "mixer_fwdbwd_7b": Workload("mixer_fwdbwd_7b", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                                "featurizer conv + Hyena-MR on interleaved features, forward+backward, bf16, B=2 L=8192 "
                                "D=4096 G=256 hl=128", layout="mixer"),
    "mixer_fwdbwd_7b_fused": Workload("mixer_fwdbwd_7b_fused", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                                      "the same without the featurized tensor: the operator's kernels make its rows "
                                      "from the projection output, forward and backward", layout="mixer_fused"),
    "mixer_fwdbwd_7b_fused_planar": Workload("mixer_fwdbwd_7b_fused_planar", 2, 8192, 256, 16, (128,), torch.bfloat16,
                                             True, "the same on planar features (interleave_projections = false): "
                                             "gcg_mixer_mr_fwd_planar / _bwd_planar", layout="mixer_fused_planar"),
    "mr_fwdbwd_7b_fp32_arith": Workload("mr_fwdbwd_7b_fp32_arith", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                                        "Hyena-MR forward+backward with cgcg_dtype float32 on bf16 tensors (fp32 filter and "
                                        "arithmetic, dtype code GCG_BF16_F32), B=2 L=8192 D=4096 G=256 hl=128",
                                        filt_dtype=torch.float32),
    "mr_fwdbwd_7b_interleaved_fp32_arith": Workload("mr_fwdbwd_7b_interleaved_fp32_arith", 2, 8192, 256, 16, (128,),
                                                    torch.bfloat16, True, "the same on interleaved features",
                                                    layout="interleaved", filt_dtype=torch.float32),
    "mixer_fwdbwd_7b_fp32_arith": Workload("mixer_fwdbwd_7b_fp32_arith", 2, 8192, 256, 16, (128,), torch.bfloat16, True,
                                           "featurizer conv + Hyena-MR with cgcg_dtype float32 on the bf16 features (the "
                                           "reference's default precision): two kernels each way", layout="mixer",
                                           filt_dtype=torch.float32),
    "mixer_fwdbwd_7b_fused_fp32_arith": Workload("mixer_fwdbwd_7b_fused_fp32_arith", 2, 8192, 256, 16, (128,),
                                                 torch.bfloat16, True, "the same through gcg_mixer_mr_fwd / _bwd",
                                                 layout="mixer_fused", filt_dtype=torch.float32),
    "mixer_fwd_7b": Workload("mixer_fwd_7b", 2, 8192, 256, 16, (128,), torch.bfloat16, False,
                             "featurizer conv + Hyena-MR on interleaved features, forward only (prefill), bf16, "
                             "B=2 L=8192 D=4096 G=256 hl=128", layout="mixer"),
    "mixer_fwd_7b_fused": Workload("mixer_fwd_7b_fused", 2, 8192, 256, 16, (128,), torch.bfloat16, False,
                                   "the same as one kernel (the featurized tensor is never stored)",
                                   layout="mixer_fused"),
    "mixer_fwdbwd_7b_reference_flow": Workload("mixer_fwdbwd_7b_reference_flow", 2, 8192, 256, 16, (128,),
                                               torch.bfloat16, True,
                                               "the same chain with the reference's data flow (permutes, F.conv1d on "
                                               "(B, 3D, L), gathers) around the separate-tensor kernels",
                                               layout="mixer_reference_flow"),
    # the Hyena-SE layer of the 40B shape from the dense projection's output to the operator's output
    "mixer_se_fwdbwd_40b": Workload("mixer_se_fwdbwd_40b", 1, 32768, 512, 16, (7,), torch.bfloat16, True,
                                    "featurizer conv + Hyena-SE on interleaved features as two kernels each way, "
                                    "forward+backward, bf16, B=1 L=32768 D=8192 G=512 hl=7", layout="mixer"),
    "mixer_se_fwdbwd_40b_fused": Workload("mixer_se_fwdbwd_40b_fused", 1, 32768, 512, 16, (7,), torch.bfloat16, True,
                                          "the same as one kernel each way (the featurized tensor stays in "
                                          "registers)", layout="mixer_fused"),
    "mixer_se_fwdbwd_40b_fp32_arith": Workload("mixer_se_fwdbwd_40b_fp32_arith", 1, 32768, 512, 16, (7,), torch.bfloat16,
                                               True, "the two-kernel chain with cgcg_dtype float32 on the bf16 features "
                                               "(fp32 filter and arithmetic inside the operator's kernels)",
                                               layout="mixer", filt_dtype=torch.float32),
    "mixer_se_fwdbwd_40b_fused_fp32_arith": Workload("mixer_se_fwdbwd_40b_fused_fp32_arith", 1, 32768, 512, 16, (7,),
                                                     torch.bfloat16, True, "the same as one kernel each way",
                                                     layout="mixer_fused", filt_dtype=torch.float32),
    "mixer_se_fwdbwd_40b_fused_planar": Workload("mixer_se_fwdbwd_40b_fused_planar", 1, 32768, 512, 16, (7,),
                                                 torch.bfloat16, True,
                                                 "the same on planar features (interleave_projections = false): "
                                                 "gcg_mixer_se_fwd_planar / _bwd_planar", layout="mixer_fused_planar"),
}
# the order in which the benchmark reports them
WORKLOAD_ORDER = ("se_fwd_fp32", "mr_fwd_7b", "mr_fwdbwd_7b", "se_mr_fwdbwd_40b", "mr_fwd_1m")


def se_filter(g: int, hl: int, gen: torch.Generator) -> torch.Tensor:
    """Short explicit filter: h ~ N(0, 1/hl), shape (g, 1, hl), fp32."""
    return torch.randn(g, 1, hl, generator=gen) / math.sqrt(hl)


def mr_filter(g: int, hl: int, gen: torch.Generator) -> torch.Tensor:
    """Medium explicit filter with exponential decay: h[g,t] = w[g,t] * exp(-a_g * t),
    w ~ N(0, 1/hl), a_g log-uniform in [1e-3, 1e-1]; shape (g, 1, hl), fp32.
    Same family as ExplicitSingleDecayFilter
    (savanna/model/operators/hyena/parametrization/explicit.py:40-75)."""
    w = torch.randn(g, hl, generator=gen) / math.sqrt(hl)
    lo, hi = math.log(1e-3), math.log(1e-1)
    a = torch.exp(lo + (hi - lo) * torch.rand(g, generator=gen))
    t = torch.arange(hl, dtype=torch.float32)
    return (w * torch.exp(-a[:, None] * t[None, :])).unsqueeze(1)


def make_inputs(bs: int, L: int, g: int, dg: int, hl: int, dtype: torch.dtype, seed: int = 0,
                decay: Optional[bool] = None, device="cpu", with_dy: bool = True):
    """Returns dict(q, k, v, h, dy) of tensors in ``dtype`` on ``device``.

    ``decay``: True = mr_filter, False = se_filter, None = by length (hl > 8 decays).
    """
    gen = torch.Generator().manual_seed(seed)
    shape = (bs, L, g, dg)
    q = torch.randn(shape, generator=gen)
    k = torch.randn(shape, generator=gen)
    v = torch.randn(shape, generator=gen)
    use_decay = (hl > 8) if decay is None else decay
    h = mr_filter(g, hl, gen) if use_decay else se_filter(g, hl, gen)
    out = {"q": q, "k": k, "v": v, "h": h}
    if with_dy:
        out["dy"] = torch.randn(shape, generator=gen)
    return {n: t.to(dtype).to(device) for n, t in out.items()}


def make_inputs_device(bs: int, L: int, g: int, dg: int, hl: int, dtype: torch.dtype, device,
                       seed: int = 0, with_dy: bool = True, slab_rows: int = 65536):
    """Same distributions generated on the device in time slabs, for shapes too large
    to stage through host memory (the 2^32-element case).  Values differ from
    make_inputs; a slab is reproducible from (seed, slab index)."""
    names = ["q", "k", "v"] + (["dy"] if with_dy else [])
    out = {n: torch.empty((bs, L, g, dg), dtype=dtype, device=device) for n in names}
    gen = torch.Generator(device=device)
    for i, n in enumerate(names):
        for s, t0 in enumerate(range(0, L, slab_rows)):
            t1 = min(L, t0 + slab_rows)
            gen.manual_seed(seed * 1000003 + i * 10007 + s)
            out[n][:, t0:t1].normal_(generator=gen)
    hgen = torch.Generator().manual_seed(seed)
    h = mr_filter(g, hl, hgen) if hl > 8 else se_filter(g, hl, hgen)
    out["h"] = h.to(dtype).to(device)
    return out
