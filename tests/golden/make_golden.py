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


def main():
    featurizer_case()
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
