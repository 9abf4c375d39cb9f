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


def main():
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
