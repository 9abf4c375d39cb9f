#!/usr/bin/env python3
"""Benchmark of the gated chunked causal convolution on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only] [--all] [--kernels]

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM: forward, plus backward for the forward+backward workloads.  The default
workload is the one the headline metric is quoted on (Hyena-MR forward+backward at the
Evo2-7B layer shape).  One JSON line is printed; it carries the whole-job throughput in
tokens/s, the roofline position of the dominant kernel (algorithmic bytes over the HIP-event
duration of that launch), the same figures for the other four configurations (`all_configs`;
`--only` leaves them out) and a CPU baseline timed on the host cores in the same run.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from savanna_amd import _lib  # noqa: E402
from savanna_amd.synthetic import WORKLOAD_ORDER, WORKLOADS, make_inputs, make_inputs_device  # noqa: E402,F401

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16, published

# HBM bytes per launch of the dominant kernel as counted by rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script (scaled by a plain copy of known size in the same run).  Counters cannot be read from inside the process, so
# the figures are kept in a data file that is rewritten whenever the counter profile is; a workload without an
# entry (or a checkout without the file) reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(workload, kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    entry = table.get(workload, {}).get(kernel)
    return entry["bytes"] if entry else None


KEEP_INTERMEDIATES = True      # mixer workloads: the chain's two intermediates stored through the cache (--no-keep-output)


class KernelEvents:
    """Pairs of hipEvent_t for gcg_time_next_kernel: the runtime stamps a pair at the start and the end of one
    kernel, so the elapsed time is that kernel's launch duration (what a profiler's kernel trace reports),
    without the small reduction kernel and the dispatch gap that a bracket around the whole call also holds."""

    def __init__(self, n):
        import ctypes

        path = None
        with open("/proc/self/maps") as f:          # the HIP runtime this process already uses
            for line in f:
                if "libamdhip64" in line:
                    path = line.split()[-1]
                    break
        if path is None:
            raise RuntimeError("HIP runtime not loaded")
        self.ct = ctypes
        self.hip = ctypes.CDLL(path)
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.pairs = []
        for _ in range(n):
            a, b = ctypes.c_void_p(), ctypes.c_void_p()
            if self.hip.hipEventCreate(ctypes.byref(a)) or self.hip.hipEventCreate(ctypes.byref(b)):
                raise RuntimeError("hipEventCreate failed")
            self.pairs.append((a, b))

    def mean_ms(self, which=None):
        """Mean over the pairs (or those with the given indices), or None if one of them was never stamped."""
        pairs = self.pairs if which is None else [self.pairs[i] for i in which]
        tot = 0.0
        for a, b in pairs:
            ms = self.ct.c_float()
            if self.hip.hipEventElapsedTime(self.ct.byref(ms), a, b):
                return None
            tot += ms.value
        return tot / len(pairs)

    def close(self):
        for a, b in self.pairs:
            self.hip.hipEventDestroy(a)
            self.hip.hipEventDestroy(b)
        self.pairs = []


class Op:
    """One convolution of a workload with its resident inputs, rotated over `nsets` copies so that
    no step finds its inputs in the 256 MB last-level cache."""

    def __init__(self, wl, hl, device, rotate_bytes=512 << 20):
        n_in = 5 if wl.backward else 3
        set_bytes = n_in * wl.bs * wl.L * wl.d * wl.elem_bytes
        # at least two sets (up to 4 GB each): part of a single one is still in the last-level cache a step later
        self.nsets = int(max(2 if set_bytes <= (4 << 30) else 1, min(64, -(-rotate_bytes // set_bytes))))
        self.sets = []
        for i in range(self.nsets):
            # drawn on the device (same distributions as the CPU recipe; the values are not compared here)
            t = make_inputs_device(wl.bs, wl.L, wl.g, wl.dg, hl, wl.dtype, device, seed=i, with_dy=wl.backward)
            if wl.layout == "dwconv":
                t = {"x": t["k"], "h": t["h"], "dy": t.get("dy")}
            elif wl.layout.startswith("mixer"):
                raw = torch.stack([t.pop("v"), t.pop("q"), t.pop("k")], dim=-1).reshape(wl.bs, wl.L, 3 * wl.d)
                wf = (torch.randn(3 * wl.d, 1, 3, generator=torch.Generator().manual_seed(i)) / 3 ** 0.5)
                t["raw"] = raw.contiguous().requires_grad_(True)
                t["wf"] = wf.to(wl.dtype).to(device).requires_grad_(True)
                t["h"] = (t["h"].to(wl.filt_dtype) if wl.filt_dtype else t["h"]).requires_grad_(True)
            elif wl.layout == "planar":
                t["feat"] = torch.stack([t.pop("v"), t.pop("q"), t.pop("k")], dim=2).contiguous()
            elif wl.layout != "separate":
                # kernel names: C = v, B = q, x = k
                t["feat"] = torch.stack([t.pop("v"), t.pop("q"), t.pop("k")], dim=-1).contiguous()
            if wl.filt_dtype and not wl.layout.startswith("mixer"):
                t["h"] = t["h"].to(wl.filt_dtype)
            self.sets.append(t)
        self.layout = wl.layout
        self.wl = wl
        self.hl = hl
        self.backward = wl.backward
        self.i = 0
        n = wl.bs * wl.L * wl.d * wl.elem_bytes
        self.fwd_bytes, self.bwd_bytes = (2 * n, 3 * n) if wl.layout == "dwconv" else (4 * n, 7 * n)

    def run_mixer(self, t, ev):
        """Featurizer conv + operator through autograd, ours or with the reference's data flow."""
        import torch.nn.functional as F
        from einops import rearrange

        from savanna_amd.kernels.cgcg.interface import (two_pass_chunked_gate_conv_gate,
                                                        two_pass_chunked_gate_conv_gate_interleaved)
        from savanna_amd.kernels.cgcg.src.kernel_utils import FwdKernelConfigRefactor
        from savanna_amd.operators.hyena import (_CausalDepthwiseConv, _FeaturizedGateConvGate,
                                                 _FeaturizedShortGateConvGate)

        wl = self.wl
        raw, wf, h = t["raw"], t["wf"], t["h"]
        raw.grad = wf.grad = h.grad = None
        if ev is not None:
            ev[0].record()
        if self.layout == "mixer_fused":
            fused = _FeaturizedShortGateConvGate if self.hl <= 8 else _FeaturizedGateConvGate
            y = fused.apply(raw.reshape(wl.bs, wl.L, wl.g, wl.dg, 3), wf, h)
        elif self.layout == "mixer_fused_planar":       # the same values read as (bs, L, 3, g, dg)
            fused = _FeaturizedShortGateConvGate if self.hl <= 8 else _FeaturizedGateConvGate
            y = fused.apply(raw.reshape(wl.bs, wl.L, 3, wl.g, wl.dg), wf, h, True)
        elif self.layout == "mixer":
            f = _CausalDepthwiseConv.apply(raw.reshape(wl.bs, wl.L, 3 * wl.d, 1), wf, KEEP_INTERMEDIATES)
            y = two_pass_chunked_gate_conv_gate_interleaved(f, h, wl.bs, wl.L, wl.g, wl.dg,
                                                            keep_dfeatures=KEEP_INTERMEDIATES)
        else:
            u = raw.permute(0, 2, 1)                                               # block.py:867
            f = F.conv1d(F.pad(u, (2, 0)), wf, groups=3 * wl.d)[..., :wl.L]        # hyena.py:139, :168-175
            f = f.permute(0, 2, 1)                                                 # block.py:875
            x1, x2, v = rearrange(f, "b l (g dg p) -> b l g p dg", p=3, g=wl.g).unbind(dim=3)
            y = two_pass_chunked_gate_conv_gate(v.contiguous(), x2.contiguous(), x1.contiguous(), h, wl.bs, wl.L,
                                                wl.g, wl.dg, fwd_kernel_cfg=FwdKernelConfigRefactor(CHUNK_SIZE=128, BLOCK_D=16, THREADBLOCK_SWIZZLE="row"),
                                                bwd_autotune=True)
        if self.backward:
            y.backward(t["dy"])
        if ev is not None:
            ev[1].record()
        return y

    def run_features(self, t, ev):
        """Workloads whose inputs are one interleaved features tensor.  The whole op is bracketed:
        for "gathered" the gathers and the re-assembly of the feature gradient are part of it."""
        if self.layout == "dwconv":
            if ev is not None:
                ev[0].record()
            y = _lib.dwconv_fwd(t["x"], t["h"])
            if self.backward:
                _lib.dwconv_bwd(t["dy"], t["x"], t["h"])
            if ev is not None:
                ev[1].record()
            return y
        feat, h = t["feat"], t["h"]
        if ev is not None:
            ev[0].record()
        if self.layout == "interleaved":
            y = _lib.fwd_interleaved(feat, h)
            if self.backward:
                _lib.bwd_interleaved(t["dy"], feat, h)
        elif self.layout == "planar":
            y = _lib.fwd_planar(feat, h)
            if self.backward:
                _lib.bwd_planar(t["dy"], feat, h)
        else:
            C, B, x = (feat[..., i].contiguous() for i in range(3))     # cgcg/interface.py:51-54
            _, _, y = _lib.fwd(x, B, C, h)
            if self.backward:
                dx, dB, dC, _ = _lib.bwd(t["dy"], x, B, C, h)
                torch.stack([dC, dB, dx], dim=-1)                        # autograd of unbind (block.py:886-890)
        if ev is not None:
            ev[1].record()
        return y

    def run(self, ev=None, kev=None):
        """ev: torch events recorded around the dominant call; kev: a hipEvent_t pair armed for its main kernel."""
        t = self.sets[self.i % self.nsets]
        self.i += 1
        if self.layout.startswith("mixer"):
            return self.run_mixer(t, ev)
        if self.layout != "separate":
            return self.run_features(t, ev)
        # kernel names: B = q, x = k, C = v
        if ev is not None and not self.backward:
            ev[0].record()
        if kev is not None and not self.backward:
            _lib.time_next_kernel(kev[0], kev[1])
        _, _, y = _lib.fwd(t["k"], t["q"], t["v"], t["h"])
        if ev is not None and not self.backward:
            ev[1].record()
        if self.backward:
            if ev is not None:
                ev[0].record()
            if kev is not None:
                _lib.time_next_kernel(kev[0], kev[1])
            _lib.bwd(t["dy"], t["k"], t["q"], t["v"], t["h"])
            if ev is not None:
                ev[1].record()
        return y


def time_graph(ops, steps, warmup):
    """One HIP graph holding a full rotation over the input sets, replayed; ms per step.
    For launch-bound shapes this is how a caller would run the op."""
    rounds = max(o.nsets for o in ops)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(rounds):
            for op in ops:
                op.run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(rounds):
            for op in ops:
                op.run()
    replays = max(1, -(-steps // rounds))
    for _ in range(max(1, warmup // rounds)):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / (replays * rounds)


SETTLE_S = 0.3     # untimed steps before the warm-up steps, by wall time (--settle)


def time_workload(wl, device, steps, warmup, graph=False):
    ops = [Op(wl, hl, device) for hl in wl.filters]
    dom = max(range(len(ops)), key=lambda i: ops[i].hl)     # dominant launch: longest filter
    # The device needs a few hundred milliseconds of load before its clocks and the translation caches of the
    # input sets are where a training run keeps them: with only a handful of warm-up steps the same step
    # measures 3 % slower (0.282 against 0.273 ms at the headline shape).  So the step is first repeated,
    # untimed, for SETTLE_S of wall time; the W warm-up steps and the K timed steps follow as asked.
    t_settle = time.perf_counter()
    n_settle = 0
    while SETTLE_S > 0 and time.perf_counter() - t_settle < SETTLE_S:
        for _ in range(8):
            for op in ops:
                op.run()
        torch.cuda.synchronize()
        n_settle += 8
    for _ in range(warmup):
        for op in ops:
            op.run()
    torch.cuda.synchronize()
    # Instrumented steps cost time themselves: a launch that carries a pair of kernel events about 5 us, a bracket
    # of torch events around the call about 9 us more (measured at the headline shape).  So inside the timed region
    # one or two steps carry kernel events only (workloads whose dominant call is one library launch), or the bracket where
    # the bracket is the measurement (whole-op workloads); the instrumented step is then repeated after the timed
    # region, with both kinds of events, for a steadier mean.  Both sample sets are reported.
    n_in = min(2, max(1, steps // 25))      # one instrumented step in a region of fewer than 50 steps, else two
    marks = {(steps * (2 * j + 1)) // (2 * n_in): j for j in range(n_in)}       # spread over the region, not step 0
    n_after = min(16, max(4, steps))
    nsamp = n_in + n_after
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(nsamp)]
    kevents = KernelEvents(nsamp) if wl.layout == "separate" else None
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        j = marks.get(k)
        for i, op in enumerate(ops):
            if i == dom and j is not None:
                op.run(None if kevents else events[j], kevents.pairs[j] if kevents else None)
            else:
                op.run()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps
    for j in range(n_in, nsamp):
        for i, op in enumerate(ops):
            if i == dom:
                op.run(events[j], kevents.pairs[j] if kevents else None)
            else:
                op.run()
    torch.cuda.synchronize()
    bracketed = events[n_in:] if kevents else events
    call_ms = sum(a.elapsed_time(b) for a, b in bracketed) / len(bracketed)   # bracket around the whole entry point
    kern_ms = kevents.mean_ms() if kevents else None                 # the main kernel alone
    kern_ms_in = kevents.mean_ms(range(n_in)) if kevents else None
    if kevents:
        kevents.close()
    if kern_ms is None:
        kern_ms = call_ms
    op = ops[dom]
    kern_bytes = op.bwd_bytes if op.backward else op.fwd_bytes
    kern_name = ("gcg_bwd" if op.backward else "gcg_fwd") + f" hl={op.hl} " + _lib.select_algo(
        wl.bs, wl.L, wl.g, wl.dg, op.hl, wl.dtype, op.backward)
    if wl.layout != "separate":      # the bracket holds the whole op, not one launch
        kern_bytes = op.fwd_bytes + (op.bwd_bytes if op.backward else 0)
        kern_name = f"whole op ({wl.layout}) hl={op.hl}"
    achieved = kern_bytes / (kern_ms * 1e-3) / 1e9
    res = {
        "workload": wl.name,
        "ms_per_step": ms_per_step,
        "tokens_per_s": wl.tokens / (ms_per_step * 1e-3),
        "step_gbs": wl.algorithmic_bytes() / (ms_per_step * 1e-3) / 1e9,
        "step_hbm_frac": wl.algorithmic_bytes() / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "step_tflops": wl.algorithmic_flops() / (ms_per_step * 1e-3) / 1e12,
        "kernel": kern_name,
        "kernel_ms": kern_ms,
        "kernel_ms_timed_region": kern_ms_in,
        "kernel_samples": {"timed_region": n_in, "after": n_after},
        "call_ms": call_ms,
        "kernel_bytes": kern_bytes,
        "kernel_gbs": achieved,
        "kernel_hbm_frac": achieved / HBM_PEAK_GBS,
        "input_sets": [o.nsets for o in ops],
        "settle_steps": n_settle,
    }
    if graph:
        g_ms = time_graph(ops, steps, warmup)
        res["graph_ms_per_step"] = g_ms
        res["graph_tokens_per_s"] = wl.tokens / (g_ms * 1e-3)
        res["graph_hbm_frac"] = wl.algorithmic_bytes() / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
    del ops
    torch.cuda.empty_cache()
    return res


def cpu_baseline(wl, budget_s=20.0):
    """The CPU port (oracle/: depthwise F.conv1d formulation + autograd, fp32) timed on this
    host's cores on a bounded sample of the workload: one batch row and as many whole filter
    groups as fit the time budget, scaled to full width (the cost is linear in channels)."""
    import oracle  # the checker, timed here only as the reported baseline

    threads = torch.get_num_threads()
    hl = max(wl.filters)
    L = min(wl.L, 8192)
    g_s = min(wl.g, 32)

    def once(g_use):
        t = make_inputs(1, L, g_use, wl.dg, hl, torch.float32, seed=0, with_dy=wl.backward)
        t0 = time.perf_counter()
        if wl.backward:
            oracle.gcg_bwd_ref_torch(t["dy"], t["k"], t["q"], t["v"], t["h"], dtype=torch.float32)
        else:
            oracle.gcg_fwd_ref_torch(t["k"], t["q"], t["v"], t["h"])
        return time.perf_counter() - t0

    once(g_s)                                   # warm-up (thread pool, mkldnn primitives)
    dt = once(g_s)
    # grow the sample until three timed runs of it fill the budget
    while g_s * 2 <= wl.g and dt * 2 * 4 < budget_s:
        g_s *= 2
        dt = once(g_s)
    runs = sorted([dt, once(g_s), once(g_s)])
    dt = runs[1]                                # median of three
    tokens_per_s = L / dt * (g_s / wl.g) / len(wl.filters)
    return {
        "value": tokens_per_s,
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": f"1 batch row x {L} tokens x {g_s * wl.dg} of {wl.d} channels, hl={hl}, fp32, "
                  f"{'fwd+bwd' if wl.backward else 'fwd'}; median of 3 runs; scaled linearly to {wl.d} channels"
                  + (f" and {len(wl.filters)} ops" if len(wl.filters) > 1 else ""),
    }


# (label, layout, bs, L, g, dg, hl, tensor dtype, filter dtype) of the single-kernel table (--kernels)
KERNEL_TABLE = (
    ("mfma bf16 hl=128, 7B", "sep", 2, 8192, 256, 16, 128, torch.bfloat16, torch.bfloat16),
    ("mfma interleaved bf16 hl=128, 7B", "il", 2, 8192, 256, 16, 128, torch.bfloat16, torch.bfloat16),
    ("mfma fp32 hl=128, 7B", "sep", 2, 8192, 256, 16, 128, torch.float32, torch.float32),
    ("mfma interleaved fp32 hl=128, 7B", "il", 2, 8192, 256, 16, 128, torch.float32, torch.float32),
    ("mfma bf16 tensors + fp32 filter hl=128, 7B", "sep", 2, 8192, 256, 16, 128, torch.bfloat16, torch.float32),
    ("mfma interleaved bf16 tensors + fp32 filter hl=128, 7B", "il", 2, 8192, 256, 16, 128, torch.bfloat16, torch.float32),
    ("mfma bf16 hl=128, 40B", "sep", 1, 32768, 512, 16, 128, torch.bfloat16, torch.bfloat16),
    ("window bf16 hl=7, 40B", "sep", 1, 32768, 512, 16, 7, torch.bfloat16, torch.bfloat16),
    ("window interleaved bf16 hl=7, 40B", "il", 1, 32768, 512, 16, 7, torch.bfloat16, torch.bfloat16),
    ("window bf16 hl=7, 7B", "sep", 2, 8192, 256, 16, 7, torch.bfloat16, torch.bfloat16),
    ("window fp32 hl=7, 7B", "sep", 2, 8192, 256, 16, 7, torch.float32, torch.float32),
    ("window interleaved fp32 hl=7, 7B", "il", 2, 8192, 256, 16, 7, torch.float32, torch.float32),
    # a tensor-parallel rank's share of the 40B layer at TP = 8 (get_groups_and_group_sizes: g = 64, d = 1024)
    ("mfma bf16 hl=128, 40B / 8 ranks, L=8192", "sep", 1, 8192, 64, 16, 128, torch.bfloat16, torch.bfloat16),
    ("mfma interleaved bf16 hl=128, 40B / 8 ranks, L=8192", "il", 1, 8192, 64, 16, 128, torch.bfloat16, torch.bfloat16),
    ("window bf16 hl=7, 40B / 8 ranks, L=8192", "sep", 1, 8192, 64, 16, 7, torch.bfloat16, torch.bfloat16),
)


def kernel_table(device, n=30, nsets=4):
    """Forward and backward kernel of the gated entry points alone: each launch between two HIP events that the
    runtime stamps at its start and end (gcg_time_next_kernel), inputs rotated over `nsets` sets, mean of n."""
    rows = []
    for label, layout, bs, L, g, dg, hl, dt, fdt in KERNEL_TABLE:
        gen = torch.Generator(device=device).manual_seed(1)
        sets = []
        for _ in range(nsets):
            feat = torch.randn(bs, L, g, dg, 3, generator=gen, device=device).to(dt)
            dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=device)).to(dt)
            h = (torch.randn(g, 1, hl, generator=gen, device=device) / hl ** 0.5).to(fdt)
            if layout == "sep":
                C, B, x = (feat[..., j].contiguous() for j in range(3))
                sets.append((x, B, C, dy, h))
            else:
                sets.append((feat, dy, h))
        if layout == "sep":
            fwd = lambda s: _lib.fwd(s[0], s[1], s[2], s[4])                    # noqa: E731
            bwd = lambda s: _lib.bwd(s[3], s[0], s[1], s[2], s[4])              # noqa: E731
        else:
            fwd = lambda s: _lib.fwd_interleaved(s[0], s[2])                    # noqa: E731
            bwd = lambda s: _lib.bwd_interleaved(s[1], s[0], s[2])              # noqa: E731
        t0 = time.perf_counter()
        i = 0
        while i < 8 or time.perf_counter() - t0 < SETTLE_S:
            fwd(sets[i % nsets]), bwd(sets[i % nsets])
            torch.cuda.synchronize()
            i += 1
        kf, kb = KernelEvents(n), KernelEvents(n)
        for i in range(n):
            s = sets[i % nsets]
            _lib.time_next_kernel(*kf.pairs[i])
            fwd(s)
            _lib.time_next_kernel(*kb.pairs[i])
            bwd(s)
        torch.cuda.synchronize()
        fms, bms = kf.mean_ms(), kb.mean_ms()
        kf.close(), kb.close()
        nbytes = bs * L * g * dg * dy.element_size()
        rows.append({"kernel": label, "shape": [bs, L, g, dg], "hl": hl,
                     "fwd_us": fms * 1e3, "fwd_gbs": 4 * nbytes / fms / 1e6, "fwd_hbm_frac": 4 * nbytes / fms / 1e6 / HBM_PEAK_GBS,
                     "bwd_us": bms * 1e3, "bwd_gbs": 7 * nbytes / bms / 1e6, "bwd_hbm_frac": 7 * nbytes / bms / 1e6 / HBM_PEAK_GBS})
        del sets
        torch.cuda.empty_cache()
    return rows


class BoardSensors:
    """Shader clock and board power of card 0 from sysfs (pp_dpm_sclk, hwmon power1_input), sampled by a thread."""

    def __init__(self, period_s=0.05):
        import glob
        import threading
        dev = "/sys/class/drm/card0/device"
        power = sorted(glob.glob(dev + "/hwmon/hwmon*/power1_input") + glob.glob(dev + "/hwmon/hwmon*/power1_average"))
        self.paths = {"sclk": dev + "/pp_dpm_sclk", "power": power[0] if power else None}
        self.period_s, self.samples, self.stop = period_s, [], False
        self.thread = threading.Thread(target=self._poll, daemon=True)
        self.thread.start()

    def _read(self):
        out = {}
        try:
            cur = [ln for ln in open(self.paths["sclk"]).read().splitlines() if ln.rstrip().endswith("*")]
            out["sclk_mhz"] = float(cur[0].split(":")[1].strip().rstrip("*").strip().lower().replace("mhz", ""))
        except (OSError, IndexError, ValueError):
            out["sclk_mhz"] = None
        try:
            out["power_w"] = int(open(self.paths["power"]).read()) / 1e6
        except (OSError, TypeError, ValueError):
            out["power_w"] = None
        return out

    def _poll(self):
        while not self.stop:
            self.samples.append((time.perf_counter(), self._read()))
            time.sleep(self.period_s)

    def between(self, t0, t1):
        """Median reading over [t0, t1) (perf_counter times)."""
        rows = [r for t, r in self.samples if t0 <= t < t1]
        out = {}
        for key in ("sclk_mhz", "power_w"):
            v = sorted(r[key] for r in rows if r[key] is not None)
            out[key] = v[len(v) // 2] if v else None
        return out

    def close(self):
        self.stop = True
        self.thread.join()


def power_table(device, secs=2.0):
    """Each kernel of the Hyena-MR paths launched back to back for `secs` seconds at the 7B and 40B layer shapes:
    median time per call (HIP events around groups of five) with the shader clock and board power meanwhile."""
    sensors = BoardSensors()
    rows = []
    for shape_name, bs, L, g, dg in (("7B", 2, 8192, 256, 16), ("40B", 1, 32768, 512, 16)):
        gen = torch.Generator(device=device).manual_seed(1)
        sets = []
        for _ in range(2):
            feat = torch.randn(bs, L, g, dg, 3, generator=gen, device=device).to(torch.bfloat16)
            dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen, device=device)).to(torch.bfloat16)
            sets.append((feat, dy))
        x, B, C = (torch.randn(bs, L, g, dg, generator=gen, device=device).to(torch.bfloat16) for _ in range(3))
        h = (torch.randn(g, 1, 128, generator=gen, device=device) / 128 ** 0.5).to(torch.bfloat16)
        hs = (torch.randn(g, 1, 7, generator=gen, device=device) / 7 ** 0.5).to(torch.bfloat16)
        hf = h.float()                                    # fp32 filter: fp32 arithmetic on the bf16 tensors
        wf = (torch.randn(3 * g * dg, 1, 3, generator=gen, device=device) / 3 ** 0.5).to(torch.bfloat16)
        calls = (
            ("gcg_fwd hl=128", lambda s: _lib.fwd(x, B, C, h)),
            ("gcg_bwd hl=128", lambda s: _lib.bwd(s[1], x, B, C, h)),
            ("gcg_fwd_interleaved hl=128", lambda s: _lib.fwd_interleaved(s[0], h)),
            ("gcg_bwd_interleaved hl=128", lambda s: _lib.bwd_interleaved(s[1], s[0], h)),
            ("gcg_mixer_mr_fwd", lambda s: _lib.mixer_mr_fwd(s[0], wf, h)),
            ("gcg_mixer_mr_bwd", lambda s: _lib.mixer_mr_bwd(s[1], s[0], wf, h)),
            ("gcg_bwd hl=7", lambda s: _lib.bwd(s[1], x, B, C, hs)),
            ("gcg_fwd hl=128, fp32 arithmetic", lambda s: _lib.fwd(x, B, C, hf)),
            ("gcg_bwd hl=128, fp32 arithmetic", lambda s: _lib.bwd(s[1], x, B, C, hf)),
        )
        for name, fn in calls:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            groups, i = [], 0
            while time.perf_counter() - t0 < secs:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(5):
                    fn(sets[i % 2])
                    i += 1
                e1.record()
                torch.cuda.synchronize()
                groups.append(e0.elapsed_time(e1) / 5 * 1e3)
            t1 = time.perf_counter()
            late = sorted(groups[len(groups) // 2:])           # the second half: clocks and power have settled
            rows.append({"kernel": name, "shape": shape_name, "us": late[len(late) // 2], "us_min": late[0],
                         "us_max": late[-1], **sensors.between(t0 + 0.5 * (t1 - t0), t1)})
        del sets, x, B, C
        torch.cuda.empty_cache()
    time.sleep(0.5)
    t_idle = time.perf_counter()
    time.sleep(0.5)
    idle = sensors.between(t_idle, time.perf_counter())
    sensors.close()
    return {"kernels": rows, "idle": idle}


TRACE_LIB = os.path.join(ROOT, "savanna_amd", "csrc", "libgcg_hip_trace.so")


def timeline_table(device, workload="mr_fwdbwd_7b", reps=5):
    """Per-workgroup timestamps inside the two matrix-core kernels of a separate-tensor workload: where a launch's
    time goes (start, prologue, walk, spread between the first and the last workgroup to finish, filter-gradient
    tail).  Uses the trace build of the library (`make -C savanna_amd/csrc trace`: libgcg_hip_trace.so, the same
    kernels with thread 0 of every workgroup storing the 100 MHz constant clock at its start, at the start and end
    of its walk and at its end) through the C ABI; one launch of each kernel per repetition, after warm-up, inputs
    rotated.  Times are microseconds from the first start on the workgroup's own XCD (the XCDs' clocks are offset
    against each other).  The stamps cost the forward about 3 us per launch (it is sensitive to any further store)
    and the backward nothing measurable; the same launch's duration by HIP events is reported beside them."""
    import ctypes
    import statistics

    if not os.path.exists(TRACE_LIB):
        raise SystemExit(f"bench.py --timeline needs {TRACE_LIB}: run `make -C savanna_amd/csrc trace`")
    wl = WORKLOADS[workload]
    if wl.layout != "separate" or len(wl.filters) != 1:
        raise SystemExit("--timeline takes a separate-tensor workload with one filter")
    lib = ctypes.CDLL(TRACE_LIB)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32
    lib.gcg_fwd.argtypes = [vp] * 7 + [i64, i64, i32, i32, i32, i32, i32, vp]
    lib.gcg_bwd.argtypes = [vp] * 10 + [ctypes.c_size_t, i64, i64, i32, i32, i32, i32, i32, vp]
    lib.gcg_bwd_workspace_bytes.argtypes = [i64, i64, i32, i32, i32, i32, i32]
    lib.gcg_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.gcg_trace_buffer.argtypes = [ctypes.POINTER(ctypes.c_size_t)]
    lib.gcg_trace_buffer.restype = vp
    hl = wl.filters[0]
    code = _lib.dtype_code(wl.dtype)
    sets = [make_inputs_device(wl.bs, wl.L, wl.g, wl.dg, hl, wl.dtype, device, seed=i, with_dy=True) for i in range(3)]
    y, dx, dB, dC = (torch.empty_like(sets[0]["k"]) for _ in range(4))
    dh = torch.empty_like(sets[0]["h"])
    nws = lib.gcg_bwd_workspace_bytes(wl.bs, wl.L, wl.g, wl.dg, hl, code, 0)
    ws = torch.empty(nws + 256, dtype=torch.uint8, device=device)
    st = torch.cuda.current_stream().cuda_stream
    dims = (wl.bs, wl.L, wl.g, wl.dg, hl, code, 0, st)

    def fwd(t):
        rc = lib.gcg_fwd(t["k"].data_ptr(), t["q"].data_ptr(), t["v"].data_ptr(), t["h"].data_ptr(), y.data_ptr(), None, None, *dims)
        assert rc == 0, rc

    def bwd(t):
        rc = lib.gcg_bwd(t["dy"].data_ptr(), t["k"].data_ptr(), t["q"].data_ptr(), t["v"].data_ptr(), t["h"].data_ptr(),
                         dx.data_ptr(), dB.data_ptr(), dC.data_ptr(), dh.data_ptr(), ws.data_ptr(), nws, *dims)
        assert rc == 0, rc

    nbytes = ctypes.c_size_t()
    tptr = lib.gcg_trace_buffer(ctypes.byref(nbytes))
    hip = KernelEvents(0).hip
    hip.hipMemset.argtypes = [vp, ctypes.c_int, ctypes.c_size_t]
    hip.hipMemcpy.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int]
    # workgroup counts from the library's own plan: the table is cleared, and the slots that a launch stamped are its workgroups
    take = 4096 * 16 * 8
    host = (ctypes.c_uint64 * (take // 8))()
    t_end = time.perf_counter() + 0.4
    i = 0
    while time.perf_counter() < t_end:
        fwd(sets[i % 3]); bwd(sets[i % 3]); i += 1
        torch.cuda.synchronize()
    out = {}
    for name, run in (("forward", fwd), ("backward", bwd)):
        rows = []
        for rep in range(reps):
            for k in range(4):
                fwd(sets[(i + k) % 3]); bwd(sets[(i + k) % 3])
            torch.cuda.synchronize()
            assert hip.hipMemset(tptr, 0, take) == 0
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(); run(sets[(i + rep) % 3]); e1.record()
            torch.cuda.synchronize()
            assert hip.hipMemcpy(host, tptr, take, 2) == 0
            import numpy as np
            a = np.frombuffer(host, dtype=np.uint64).reshape(-1, 16).astype(np.int64)
            a = a[a[:, 0] != 0]
            t = a / 100.0
            xcd = np.arange(len(t)) % 8
            base = np.array([t[xcd == x, 0].min() for x in range(8)])
            t = t - base[xcd][:, None]
            last = 7 if (a[:, 7] != 0).all() else 6
            rows.append({
                "workgroups": int(len(t)), "event_us": e0.elapsed_time(e1) * 1e3,
                "start_median": float(np.median(t[:, 0])), "start_last": float(t[:, 0].max()),
                "prologue_median": float(np.median(t[:, 5] - t[:, 0])),
                "walk_min": float((t[:, 6] - t[:, 5]).min()), "walk_median": float(np.median(t[:, 6] - t[:, 5])),
                "walk_max": float((t[:, 6] - t[:, 5]).max()),
                "walk_end_median": float(np.median(t[:, 6])), "walk_end_last": float(t[:, 6].max()),
                "tail_median": float(np.median(t[:, last] - t[:, 6])), "tail_max": float((t[:, last] - t[:, 6]).max()),
                "end_median": float(np.median(t[:, last])), "end_last": float(t[:, last].max()),
                "walk_end_mean_by_xcd": [round(float(t[xcd == x, 6].mean()), 2) for x in range(8)],
            })
        out[name] = {k: (round(statistics.median(r[k] for r in rows), 2) if not isinstance(rows[0][k], list) else rows[len(rows) // 2][k])
                     for k in rows[0]}
        out[name]["launches"] = reps
    return out


def main():
    global KEEP_INTERMEDIATES, SETTLE_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="mr_fwdbwd_7b", choices=list(WORKLOADS))
    ap.add_argument("--only", action="store_true", help="time the chosen workload alone (no all_configs block)")
    ap.add_argument("--all", action="store_true", help="also time the rows next to the hot path (interleaved "
                                                       "features, featurizer conv, mixer chains)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-keep-output", action="store_true",
                    help="mixer workloads: store the chain's intermediates past the cache like every other output")
    ap.add_argument("--graph", action="store_true",
                    help="also time the step replayed from a captured HIP graph (launch-bound shapes)")
    ap.add_argument("--settle", type=float, default=SETTLE_S,
                    help="seconds of untimed steps before the warm-up steps, so that clocks have settled (0: none)")
    ap.add_argument("--kernels", action="store_true",
                    help="print the single-kernel table instead (forward and backward kernel of the gated entry "
                         "points alone at the 7B and 40B layer shapes, one JSON line) and exit")
    ap.add_argument("--power", action="store_true",
                    help="print shader clock and board power (sysfs) under each Hyena-MR kernel launched back to "
                         "back, with the time per call, as one JSON line, and exit")
    ap.add_argument("--timeline", action="store_true",
                    help="print per-workgroup timestamps inside the two matrix-core kernels of the workload (start, "
                         "prologue, walk, finishing spread, filter-gradient tail) from the trace build of the library "
                         "(make -C savanna_amd/csrc trace), as one JSON line, and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy three times, so a counter profile of this "
                         "command holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    KEEP_INTERMEDIATES = not args.no_keep_output
    SETTLE_S = args.settle
    if args.gpus != 1:
        print("bench.py: this build is single-GPU; the path has no collective or sharded variant, "
              "so --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU path", file=sys.stderr)
        sys.exit(3)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    _lib.load()

    if args.kernels:
        print(json.dumps({"single_kernels": kernel_table(device, n=max(10, args.steps)), "unit": "us, GB/s of algorithmic "
                          "bytes (4 tensors forward, 7 backward), fraction of 8 TB/s"}), flush=True)
        return

    if args.timeline:
        print(json.dumps({"timeline": timeline_table(device, args.workload), "workload": args.workload,
                          "unit": "us from the first workgroup start on the same XCD; medians over the launches"}), flush=True)
        return

    if args.power:
        print(json.dumps({"power": power_table(device), "unit": "us per call (median, min, max of the settled half), "
                          "MHz, W"}), flush=True)
        return

    wl = WORKLOADS[args.workload]
    res = time_workload(wl, device, args.steps, args.warmup, graph=args.graph)
    line = {
        "metric": "Hyena-MR fwd+bwd tokens/s and HBM GB/s (% roofline) at 1 MI355X",
        "value": res["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": str(wl.dtype).replace("torch.", "").replace("bfloat16", "bf16").replace("float32", "f32"),
        "data": "synthetic",
        "config": {"workload": wl.name, "about": wl.about, "bs": wl.bs, "L": wl.L, "d": wl.d, "g": wl.g,
                   "filters": list(wl.filters), "backward": wl.backward,
                   "step_algorithmic_bytes": wl.algorithmic_bytes(), "step_gbs": res["step_gbs"],
                   "step_hbm_frac": res["step_hbm_frac"], "step_tflops": res["step_tflops"],
                   "step_mfma_frac": res["step_tflops"] / MFMA_BF16_PEAK_TFLOPS,
                   "settle_s": SETTLE_S, "settle_steps": res["settle_steps"]},
        "roofline": {"bound": "hbm", "kernel": res["kernel"], "achieved": res["kernel_gbs"],
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": res["kernel_hbm_frac"],
                     "kernel_ms": res["kernel_ms"], "call_ms": res["call_ms"], "algorithmic_bytes": res["kernel_bytes"],
                     "kernel_ms_timed_region": res["kernel_ms_timed_region"], "kernel_samples": res["kernel_samples"],
                     "traffic": measured_traffic(wl.name, res["kernel"])},
    }
    if args.graph:
        line["graph"] = {k: res[k] for k in ("graph_ms_per_step", "graph_tokens_per_s", "graph_hbm_frac")}
    if not args.only:
        # the other four configurations, each with its own roofline position (fewer steps where a step is long)
        others = {}
        for name in WORKLOAD_ORDER:
            if name == wl.name:
                continue
            w = WORKLOADS[name]
            n = w.bs * w.L * w.d
            k = max(100, args.steps) if n < (1 << 22) else args.steps if n < (1 << 28) else \
                max(5, args.steps // 2) if n < (1 << 30) else 3
            small = w.algorithmic_bytes() < (64 << 20)       # launch-bound: also report graph replay
            r = time_workload(w, device, k, max(2, min(args.warmup, k // 2)), graph=small)
            r["steps"] = k
            r["traffic"] = measured_traffic(w.name, r["kernel"])
            others[name] = r
        line["all_configs"] = others
    if args.all:
        # the rows next to the hot path: the operator fed from the interleaved projected features, the
        # featurizer conv, and the two chained through autograd
        extra = {}
        for name in ("mr_fwdbwd_7b_interleaved", "se_fwdbwd_40b_interleaved", "mr_fwdbwd_7b_planar", "se_fwdbwd_40b_planar",
                     "featurizer_fwdbwd_7b", "mixer_fwdbwd_7b",
                     "mixer_fwdbwd_7b_fused", "mixer_fwdbwd_7b_fused_planar", "mixer_fwd_7b", "mixer_fwd_7b_fused",
                     "mixer_se_fwdbwd_40b", "mixer_se_fwdbwd_40b_fused", "mixer_se_fwdbwd_40b_fused_planar",
                     "mixer_se_fwdbwd_40b_fp32_arith", "mixer_se_fwdbwd_40b_fused_fp32_arith",
                     "mixer_fwdbwd_7b_fp32_arith", "mixer_fwdbwd_7b_fused_fp32_arith",
                     "mr_fwdbwd_7b_fp32_arith", "mr_fwdbwd_7b_interleaved_fp32_arith"):
            r = time_workload(WORKLOADS[name], device, max(10, args.steps // 2), 4)
            extra[name] = {k: r[k] for k in ("ms_per_step", "tokens_per_s", "step_gbs", "step_hbm_frac")}
        line["next_rows"] = extra
    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        line["copy_calibration"] = {"bytes_read": src.numel(), "bytes_written": dst.numel(), "launches": 3}
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
