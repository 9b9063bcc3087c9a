"""Writes the small known-answer fixtures in this directory.

The reference's own tests hold no stored vectors (they compare against stock
torch on random data), so these come from the fp64 CPU oracle of this
repository, which tests/test_oracle.py pins against stock torch convolutions
and autograd.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

CASES = {
    # name: (B, C_in, C_out, spatial, dilation)
    "strip_1x5_d1": (1, 1, 1, (1, 5), 1),
    "img_7x13_d3": (2, 3, 2, (7, 13), 3),
    "img_3x3_d3": (1, 2, 2, (3, 3), 3),
    "vol_5x7x11_d2": (1, 3, 2, (5, 7, 11), 2),
    "vol_2x2x2_d2": (1, 2, 1, (2, 2, 2), 2),
}


def main():
    for name, (B, C, Wd, size, d) in CASES.items():
        gen = torch.Generator().manual_seed(1234)
        ndim = len(size)
        x = torch.randn(B, C, *size, dtype=torch.float64, generator=gen)
        k = torch.randn(Wd, C, *([3] * ndim), dtype=torch.float64, generator=gen) * 0.4
        bias = torch.randn(Wd, dtype=torch.float64, generator=gen) * 0.2
        gy = torch.randn(B, Wd, *size, dtype=torch.float64, generator=gen)
        y = torch.empty(B, Wd, *size, dtype=torch.float64)
        oracle.conv_relu_forward(x, k, bias, y, d)
        gx = torch.zeros_like(x)
        gk = torch.zeros_like(k)
        gb = torch.zeros_like(bias)
        oracle.conv_relu_backward_x(y, gy, k, gx, d)
        oracle.conv_relu_backward_k(y, gy, x, gk, d)
        oracle.conv_relu_backward_bias(y, gy, gb)
        np.savez(os.path.join(HERE, name + ".npz"), dilation=np.int64(d), x=x.numpy(), k=k.numpy(),
                 bias=bias.numpy(), gy=gy.numpy(), y=y.numpy(), gx=gx.numpy(), gk=gk.numpy(), gb=gb.numpy())
        print("wrote", name)


if __name__ == "__main__":
    main()
