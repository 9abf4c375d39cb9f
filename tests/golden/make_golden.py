"""Writes tests/golden/*.npz: small input/output vectors of the gated convolution.

The expected values come from the library formulation the reference uses as its ground
truth -- depthwise F.conv1d cross-correlation with left pad hl-1 on B*x, times C
(savanna/kernels/triton_src/cgcg/ref_fwd.py:109-129) and autograd of it
(tests/test_bwd_refactor.py:95-103) -- evaluated in float64 by oracle.gcg_fwd_ref_torch /
gcg_bwd_ref_torch on inputs drawn from a CPU generator with seed 0.  The reference has no
stored vectors for this path (its tests draw randn on the CUDA generator), and nothing of
the reference is imported here.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

# name -> (bs, L, g, dg, hl, dtype the inputs are rounded to)
CASES = {
    "se_fp32_small": (1, 96, 4, 16, 7, torch.float32),       # Hyena-SE shape family, fp32
    "mr_bf16_small": (2, 320, 2, 16, 128, torch.bfloat16),    # Hyena-MR, crosses two 128-chunks, ragged tail
    "mr_f16_hl32": (1, 200, 3, 16, 32, torch.float16),
    "arange_filter": (1, 40, 2, 16, 4, torch.float32),        # h = arange, the reference's Toeplitz KAT input
}


def featurizer_case():
    """The featurizer conv as ParallelCausalDepthwiseConv1d.forward computes it on (B, D, L)
    (savanna/model/operators/hyena/hyena.py:139,159,168-175: left pad K-1, F.conv1d with one group per
    channel, first L samples), in float64, stored channel-last as (bs, L, D, 1) / (D, 1, K)."""
    import torch.nn.functional as F

    bs, L, D, K, dtype = 2, 150, 24, 3, torch.bfloat16
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(bs, D, L, generator=gen).to(dtype).double().requires_grad_(True)
    dy = torch.randn(bs, D, L, generator=gen).to(dtype).double()
    w = (torch.randn(D, 1, K, generator=gen) / K ** 0.5).to(dtype).double().requires_grad_(True)
    y = F.conv1d(F.pad(x, (K - 1, 0)), w, bias=None, stride=1, padding=0, groups=D)[..., :L]
    y.backward(dy)
    cl = lambda t: t.detach().permute(0, 2, 1).unsqueeze(-1).contiguous()   # (bs, L, D, 1)
    np.savez_compressed(
        os.path.join(HERE, "featurizer_bf16_small.npz"),
        x=cl(x).float().numpy(), dy=cl(dy).float().numpy(), w=w.detach().float().numpy(),
        y=cl(y).numpy(), dx=cl(x.grad).numpy(), dw=w.grad.numpy(), dtype=np.array(str(dtype)),
    )
    print("featurizer_bf16_small written")


def mixer_se_case():
    """The convolutional part of a Hyena-SE layer as the reference chains it, in float64 with its
    bf16 tensors emulated: permute, ParallelCausalDepthwiseConv1d on (B, 3D, L), permute
    (savanna/model/block.py:867-876), the interleaved split (block.py:886-890), and
    y = x1 * conv(x2 * v, h) (hyena.py:825-840 -> ref_fwd.py:109-129).  The featurized tensor is a
    bf16 tensor there, so it is rounded on the way forward and its gradient on the way back."""
    import torch.nn.functional as F
    from einops import rearrange

    bs, L, g, dg, hl, K, dtype = 2, 150, 3, 8, 7, 3, torch.bfloat16
    D = g * dg
    gen = torch.Generator().manual_seed(0)
    raw = torch.randn(bs, L, 3 * D, generator=gen).to(dtype).double().requires_grad_(True)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype).double()
    wf = (torch.randn(3 * D, 1, K, generator=gen) / K ** 0.5).to(dtype).double().requires_grad_(True)
    h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype).double().requires_grad_(True)
    u = raw.permute(0, 2, 1)
    f = F.conv1d(F.pad(u, (K - 1, 0)), wf, bias=None, stride=1, padding=0, groups=3 * D)[..., :L].permute(0, 2, 1)
    f = f + (f.to(dtype).double() - f).detach()                  # stored as bf16
    f.register_hook(lambda gr: gr.to(dtype).double())            # and so is its gradient
    x1, x2, v = rearrange(f, "b l (g dg p) -> b l g p dg", p=3, g=g).unbind(dim=3)
    y = oracle.gcg_fwd_ref_torch(v.contiguous(), x2.contiguous(), x1.contiguous(), h)
    y.backward(dy)
    np.savez_compressed(
        os.path.join(HERE, "mixer_se_bf16_small.npz"),
        raw=raw.detach().reshape(bs, L, g, dg, 3).float().numpy(), dy=dy.float().numpy(),
        wf=wf.detach().float().numpy(), h=h.detach().float().numpy(), y=y.detach().numpy(),
        draw=raw.grad.reshape(bs, L, g, dg, 3).numpy(), dwf=wf.grad.numpy(), dh=h.grad.numpy(),
        dtype=np.array(str(dtype)),
    )
    print("mixer_se_bf16_small written")


def mixer_mr_case():
    """The convolutional part of a Hyena-MR layer as the reference chains it, in float64 with its bf16 tensors
    emulated: the decayed filter h = (w * decay)[:, :hl] cast to the tensors' type
    (savanna/model/operators/hyena/parametrization/explicit.py:68-75, hyena.py:440-441, :499-503), the featurizer
    conv and interleaved split as in mixer_se_case (block.py:867-890), and y = x1 * conv(x2 * v, h)
    (hyena.py:517-531 -> ref_fwd.py:109-129).  The gradient of the filter is stored in the filter's type before
    it reaches w, as autograd of the cast does."""
    import torch.nn.functional as F
    from einops import rearrange

    bs, L, g, dg, hl, lc, K, dtype = 2, 300, 3, 16, 128, 160, 3, torch.bfloat16
    D = g * dg
    gen = torch.Generator().manual_seed(0)
    raw = torch.randn(bs, L, 3 * D, generator=gen).to(dtype).double().requires_grad_(True)
    dy = (0.1 * torch.randn(bs, L, g, dg, generator=gen)).to(dtype).double()
    wf = (torch.randn(3 * D, 1, K, generator=gen) / K ** 0.5).to(dtype).double().requires_grad_(True)
    w = (torch.randn(g, lc, generator=gen) / lc ** 0.5).float().double().requires_grad_(True)
    decay = torch.exp(-torch.logspace(0, 2, g)[:, None] * torch.linspace(0, 1, lc)[None]).float().double()
    hfull = (w * decay)[:, :hl]
    h = hfull + (hfull.to(dtype).double() - hfull).detach()       # the cast to the tensors' type
    h.register_hook(lambda gr: gr.to(dtype).double())             # whose gradient is stored in that type
    h = h[:, None]
    u = raw.permute(0, 2, 1)
    f = F.conv1d(F.pad(u, (K - 1, 0)), wf, bias=None, stride=1, padding=0, groups=3 * D)[..., :L].permute(0, 2, 1)
    f = f + (f.to(dtype).double() - f).detach()
    f.register_hook(lambda gr: gr.to(dtype).double())
    x1, x2, v = rearrange(f, "b l (g dg p) -> b l g p dg", p=3, g=g).unbind(dim=3)
    y = oracle.gcg_fwd_ref_torch(v.contiguous(), x2.contiguous(), x1.contiguous(), h)
    y.backward(dy)
    np.savez_compressed(
        os.path.join(HERE, "mixer_mr_bf16_small.npz"),
        raw=raw.detach().reshape(bs, L, g, dg, 3).float().numpy(), dy=dy.float().numpy(),
        wf=wf.detach().float().numpy(), w=w.detach().float().numpy(), decay=decay.float().numpy(),
        h=h.detach().float().numpy(), hl=np.array(hl), y=y.detach().numpy(),
        draw=raw.grad.reshape(bs, L, g, dg, 3).numpy(), dwf=wf.grad.numpy(), dw=w.grad.numpy(),
        dtype=np.array(str(dtype)),
    )
    print("mixer_mr_bf16_small written")


def main():
    featurizer_case()
    mixer_se_case()
    mixer_mr_case()
    for name, (bs, L, g, dg, hl, dtype) in CASES.items():
        gen = torch.Generator().manual_seed(0)
        x, B, C, dy = (torch.randn(bs, L, g, dg, generator=gen).to(dtype).double() for _ in range(4))
        if name == "arange_filter":
            h = torch.arange(g * hl, dtype=torch.float64).reshape(g, 1, hl)
        else:
            h = (torch.randn(g, 1, hl, generator=gen) / hl ** 0.5).to(dtype).double()
        bx, y2, y = oracle.gcg_fwd_ref_torch(x, B, C, h, return_intermediates=True)
        dx, dB, dC, dh = oracle.gcg_bwd_ref_torch(dy, x, B, C, h)
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            x=x.float().numpy(), B=B.float().numpy(), C=C.float().numpy(), h=h.float().numpy(),
            dy=dy.float().numpy(), bx=bx.numpy(), y2=y2.numpy(), y=y.numpy(),
            dx=dx.numpy(), dB=dB.numpy(), dC=dC.numpy(), dh=dh.numpy(),
            dtype=np.array(str(dtype)),
        )
        print(name, "written")


if __name__ == "__main__":
    main()
