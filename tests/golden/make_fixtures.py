"""Writes the golden vectors of tests/golden/*.npz.

The reference keeps no stored vectors for this path (its scripts print differences of random inputs), so the
vectors here come from this repository's fp64 oracle, whose functions are pinned independently in
tests/test_oracle.py (closed forms, brute force, invariants).  They serve two purposes: the oracle cannot drift
unnoticed (tests/test_golden.py recomputes them on the CPU), and the GPU path is checked against files rather than
against code that runs in the same process.  Two of the cases are the structured inputs of the reference's own
scripts, whose expected outputs are known in closed form:
  ones_c10   scripts/test_compression_cuda.py:210-242  f1 = f2 = 1, C = 10, H = 4, W = 8, weights = 1 -> 80 and 40
  debug_bwd  scripts/test_maxavg_autograd.py:539-563   f = 1, argmax = 1, grads = arange

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
D = torch.float64


def seeded(B, H1, W1, H2, W2, C, K, seed):
    # inputs are fp32 values (what the operator takes), held in fp64 for the oracle
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    f1 = (r(B, H1, W1, C) / C ** 0.5).to(D)
    f2 = r(B, H2, W2, C).to(D)
    a_u = r(B, H1, W1, K, W2).softmax(-1).to(D)
    a_v = r(B, H1, W1, K, H2).softmax(-1).to(D)
    g_u, g_v = r(B, H1, W1, 2, H2).to(D), r(B, H1, W1, 2, W2).to(D)
    g_cu, g_cv = r(B, H1, W1, K, H2).to(D), r(B, H1, W1, K, W2).to(D)
    return dict(f1=f1, f2=f2, a_u=a_u, a_v=a_v, g_u=g_u, g_v=g_v, g_cu=g_cu, g_cv=g_cv)


def evaluate(x):
    out_u, out_v, am_u, am_v = O.max_argmax_avg_forward(x["f1"], x["f2"])
    cu, cv = O.compression_forward(x["f1"], x["f2"], x["a_u"], x["a_v"])
    am_u_in = x.get("am_u", am_u)
    am_v_in = x.get("am_v", am_v)
    m1, m2 = O.max_argmax_avg_backward(x["f1"], x["f2"], am_u_in, am_v_in, x["g_u"], x["g_v"])
    c1, c2, da_u, da_v = O.compression_backward(x["f1"], x["f2"], x["a_u"], x["a_v"], x["g_cu"], x["g_cv"])
    return dict(out_u=out_u, out_v=out_v, am_u=am_u, am_v=am_v, comp_u=cu, comp_v=cv,
                m_df1=m1, m_df2=m2, c_df1=c1, c_df2=c2, da_u=da_u, da_v=da_v)


def cases():
    yield "seeded_small", seeded(2, 5, 7, 5, 7, 16, 2, seed=101)
    yield "seeded_pooled_oddC", seeded(1, 5, 9, 2, 4, 37, 3, seed=102)
    yield "seeded_c256", seeded(1, 2, 32, 2, 32, 256, 4, seed=103)
    B, H, W, C, K = 1, 4, 8, 10, 2
    one = lambda *s: torch.ones(*s, dtype=D)
    yield "ones_c10", dict(f1=one(B, H, W, C), f2=one(B, H, W, C), a_u=one(B, H, W, K, W), a_v=one(B, H, W, K, H),
                           g_u=one(B, H, W, 2, H), g_v=one(B, H, W, 2, W), g_cu=one(B, H, W, K, H), g_cv=one(B, H, W, K, W))
    B, H, W, C, K = 1, 15, 15, 3, 1
    ar = lambda n, *s: torch.arange(n, dtype=D).expand(*s).contiguous()
    yield "debug_bwd", dict(f1=one(B, H, W, C), f2=one(B, H, W, C), a_u=one(B, H, W, K, W) / W, a_v=one(B, H, W, K, H) / H,
                            g_u=ar(H, B, H, W, 2, H), g_v=ar(W, B, H, W, 2, W), g_cu=one(B, H, W, K, H), g_cv=one(B, H, W, K, W),
                            am_u=torch.ones(B, H, W, 1, H, dtype=torch.int32), am_v=torch.ones(B, H, W, 1, W, dtype=torch.int32))


def main():
    for name, x in cases():
        y = evaluate(x)
        # stored as fp32 (inputs are fp32 values: exact; expected outputs rounded once, 6e-8 relative) and int32
        to32 = lambda v: v.numpy() if v.dtype == torch.int32 else v.to(torch.float32).numpy()
        arrays = {"in_" + k: to32(v) for k, v in x.items()}
        arrays.update({"out_" + k: to32(v) for k, v in y.items()})
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
        print(name, {k: tuple(v.shape) for k, v in y.items() if k in ("out_u", "comp_v")})


if __name__ == "__main__":
    main()
