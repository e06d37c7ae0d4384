"""Writes the golden vectors of the windowed pyramid lookup: python tests/golden/lookup/make_lookup_fixtures.py

Inputs are seeded fp32 values; expected outputs and gradients come from the fp64 oracle (stored-volume lookup of
oracle/oracle.py, autograd for the gradients) and are stored rounded once to fp32.  The reference holds no vectors for
this function (its tests never call the lookup), so these files pin the oracle against drift and give the HIP path a
fixed target; what pins the oracle itself is in tests/test_lookup_oracle.py.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.abspath(os.path.join(HERE, "..", "..", "..")))
from oracle import oracle as O  # noqa: E402


def case(B, C, H, W, levels, r, spread, seed):
    g = torch.Generator().manual_seed(seed)
    fmap1 = torch.randn(B, C, H, W, generator=g)
    fmap2 = torch.randn(B, C, H, W, generator=g)
    yy, xx = torch.meshgrid(torch.arange(H), torch.arange(W), indexing="ij")
    coords = torch.stack([xx, yy]).float()[None].repeat(B, 1, 1, 1) + torch.randn(B, 2, H, W, generator=g) * spread
    up = torch.randn(B, levels * (2 * r + 1) ** 2, H, W, generator=g)
    a = fmap1.double().requires_grad_()
    b = fmap2.double().requires_grad_()
    out = O.CorrBlock4D(a, b, num_levels=levels).lookup(coords.double(), radius=r)
    (out * up.double()).sum().backward()
    return dict(in_fmap1=fmap1, in_fmap2=fmap2, in_coords=coords, in_up=up, in_levels=torch.tensor(levels),
                in_radius=torch.tensor(r), out_lookup=out.detach().float(), out_d_fmap1=a.grad.float(),
                out_d_fmap2=b.grad.float())


def main():
    for name, args in (("lookup_seeded_c32", (1, 32, 10, 16, 3, 4, 3.0, 201)),
                       ("lookup_seeded_oddC_far", (1, 37, 9, 14, 2, 2, 12.0, 202))):
        arrays = {k: v.numpy() for k, v in case(*args).items()}
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
        print(name, arrays["out_lookup"].shape)


if __name__ == "__main__":
    main()
