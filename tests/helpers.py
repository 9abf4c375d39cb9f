"""Shared pieces of the parity tests."""
import torch

import oracle

# Parity bars (max |out - ref| / max |ref|), from the workload definition:
# bf16 / f16 I/O with fp32 accumulation <= 1e-2; fp32 mode <= 1e-5.
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}
# dh sums up to bs*L*dg products per tap and is stored in the I/O dtype
TOL_DH = {torch.float32: 2e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}


def rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    out = out.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert out.shape == ref.shape, (out.shape, ref.shape)
    assert torch.isfinite(out).all(), "non-finite values in kernel output"
    scale = ref.abs().max().item()
    return (out - ref).abs().max().item() / (scale if scale > 0 else 1.0)


def assert_close(out, ref, tol, what):
    e = rel_err(out, ref)
    assert e <= tol, f"{what}: max relative error {e:.3e} > {tol:.1e}"


def inputs(bs, L, g, dg, hl, dtype, seed=0, dy_scale=1.0):
    """x, B, C, h, dy in ``dtype`` on the CPU (values already rounded to ``dtype``)."""
    gen = torch.Generator().manual_seed(seed)
    x, B, C, dy = (torch.randn(bs, L, g, dg, generator=gen).to(dtype) for _ in range(4))
    h = (torch.randn(g, 1, hl, generator=gen) / max(1.0, hl ** 0.5)).to(dtype)
    return x, B, C, h, (dy_scale * dy.float()).to(dtype)


def oracle_fwd(x, B, C, h):
    """fp64-accumulated (bx, y2, y) on the dtype-rounded inputs."""
    return oracle.gcg_fwd_oracle(x.float(), B.float(), C.float(), h.float(), return_intermediates=True)


def oracle_bwd(dy, x, B, C, h):
    return oracle.gcg_bwd_oracle(dy.float(), x.float(), B.float(), C.float(), h.float())
