"""GPU parity at the headline configuration (B=2, C=256, 55x128, K'=4) through the caller's interface.

* AlternateCorrBlockSepflow.separate() over the 4 pyramid levels (the fused path: one autograd node per level,
  attention producer, combined feature-gradient contraction, volume assembly) against the full-4D oracle in
  fp64: both volumes, the gradients of both feature maps and of the Conv3d attention parameters.
* sepcorr_fused_backward at the same size against the sum of the oracle's two backward functions.
* The gradient tolerance is shown, not assumed: the same tensors are computed by the fp32 CPU run of the 4D
  path, and the GPU's error against fp64 must stay within twice that run's error.
Mirrors scripts/test_maxavg_autograd.py:478-502 and scripts/test_compression_autograd.py:442-484 (comparison of
the operator's gradients with autograd through the 4D volume) at the size the benchmark is quoted on.
"""
import copy

import pytest
import torch

from oracle import oracle as O
from tests._util import assert_close, chain_ratio, check_argmax_levels, error_report, native_argmax_levels

pytestmark = pytest.mark.gpu

B, C, H, W, K = 2, 256, 55, 128, 4


def _attention(seed):
    torch.manual_seed(seed)
    return torch.nn.Conv3d(2, K, 3, padding=1), torch.nn.Conv3d(2, K, 3, padding=1)


def _oracle_separate(fmap1, fmap2, att, w1, w2, dtype, argmax):
    """CorrBlock4D.separate + loss backward in `dtype`, one batch element at a time (the Conv3d parameter
    gradients are sums over the batch).  Maxima are read where `argmax` (the native block's, verified against the
    fp64 volume to differ from the true argmax at near-ties only) points, so that the gradient of a maximum is
    routed alike on both sides.  Returns corr1, corr2, d_fmap1, d_fmap2, parameter gradients, near-tie count."""
    matt = tuple(copy.deepcopy(m).to(dtype) for m in att)
    c1s, c2s, g1s, g2s = [], [], [], []
    near_ties = 0
    for b in range(fmap1.shape[0]):
        x1 = fmap1[b:b + 1].to(dtype).requires_grad_()
        x2 = fmap2[b:b + 1].to(dtype).requires_grad_()
        blk = O.CorrBlock4D(x1, x2, num_levels=4)
        am = [(u[b:b + 1], v[b:b + 1]) for u, v in argmax]
        if dtype == torch.float64:
            near_ties += check_argmax_levels(am, blk, f"batch {b}")
        c1, c2 = blk.separate(matt, argmax=am)
        ((c1 * w1[b:b + 1].to(dtype)).sum() + (c2 * w2[b:b + 1].to(dtype)).sum()).backward()
        c1s.append(c1.detach()); c2s.append(c2.detach()); g1s.append(x1.grad); g2s.append(x2.grad)
    pg = [p.grad for m in matt for p in (m.weight, m.bias)]
    return torch.cat(c1s), torch.cat(c2s), torch.cat(g1s), torch.cat(g2s), pg, near_ties


def test_separate_at_headline_size_matches_the_4d_oracle(device):
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    fmap1, fmap2, _, _ = O.make_inputs(B, H, W, C, seed=1234)
    att = _attention(1234)
    gen = torch.Generator().manual_seed(3)
    nch = (2 + K) * 4
    w1 = torch.randn(B, nch, W, H, W, generator=gen) / 64
    w2 = torch.randn(B, nch, H, H, W, generator=gen) / 64

    g1 = fmap1.to(device).requires_grad_()
    g2 = fmap2.to(device).requires_grad_()
    gatt = tuple(copy.deepcopy(m).to(device) for m in att)
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    blk = AlternateCorrBlockSepflow(g1, g2, None, num_levels=4, support_backward=True)
    c1, c2 = blk(None, sep=True, attention_weights=gatt)
    assert c1.shape == (B, nch, W, H, W) and c2.shape == (B, nch, H, H, W)
    w1d, w2d = w1.to(device), w2.to(device)
    ((c1 * w1d).sum() + (c2 * w2d).sum()).backward()
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    print(f"peak allocated by separate() forward+backward: {peak / 2**20:.0f} MiB "
          f"(stored 4D pyramid: {B * (H * W) ** 2 * 4 * (1 + 1 / 4 + 1 / 16 + 1 / 64) / 2**20:.0f} MiB)", flush=True)

    argmax = native_argmax_levels(fmap1, fmap2, device)
    r64 = _oracle_separate(fmap1, fmap2, att, w1, w2, torch.float64, argmax)
    r32 = _oracle_separate(fmap1, fmap2, att, w1, w2, torch.float32, argmax)
    print(f"argmax near-tie mismatches over 4 levels: {r64[5]}", flush=True)
    assert_close(c1, r64[0], "corr1")
    assert_close(c2, r64[1], "corr2")
    error_report(g1.grad, r64[2], r32[2], "d_fmap1")
    error_report(g2.grad, r64[3], r32[3], "d_fmap2")
    got_pg = [p.grad for m in gatt for p in (m.weight, m.bias)]
    names = ("attention1.weight", "attention1.bias", "attention2.weight", "attention2.bias")
    for g, a, b32, n in zip(got_pg, r64[4], r32[4], names):
        error_report(g, a, b32, n + ".grad")


def test_fused_backward_at_headline_size_matches_the_oracle(device):
    from separableflowthesis_amd import MemorySaver as ms
    _, _, f1, f2 = O.make_inputs(B, H, W, C, seed=1234)
    d = lambda t: t.to(device)
    ou, ov, au, av = ms.max_argmax_avg_forward(d(f1), d(f2))
    g = torch.Generator().manual_seed(99)
    a_u = torch.randn(B, H, W, K, W, generator=g).softmax(-1).contiguous()
    a_v = torch.randn(B, H, W, K, H, generator=g).softmax(-1).contiguous()
    g_cu, g_cv = torch.randn(B, H, W, K, H, generator=g), torch.randn(B, H, W, K, W, generator=g)
    g_u, g_v = torch.randn(ou.shape, generator=g), torch.randn(ov.shape, generator=g)
    d1, d2 = ms.fused_backward(d(f1), d(f2), au, av, d(g_u), d(g_v), d(a_u), d(a_v), d(g_cu), d(g_cv))
    # the two reference entry points at the same inputs, for the same comparison
    c1, c2, _, _ = ms.compression_backward(d(f1), d(f2), d(a_u), d(a_v), d(g_cu), d(g_cv))
    m1, m2 = ms.max_argmax_avg_backward(d(f1), d(f2), au, av, d(g_u), d(g_v))
    # the same call through the two dense contractions (at this size the library takes the gather form by itself)
    ms.set_max_avg_backward(ms.MAXAVG_DENSE)
    try:
        n1, n2 = ms.max_argmax_avg_backward(d(f1), d(f2), au, av, d(g_u), d(g_v))
    finally:
        ms.set_max_avg_backward(ms.MAXAVG_AUTO)
    for b in range(B):
        sl = slice(b, b + 1)
        ref = {}
        for dt in (torch.float64, torch.float32):
            x1, x2 = f1[sl].to(dt), f2[sl].to(dt)
            rc = O.compression_backward(x1, x2, a_u[sl].to(dt), a_v[sl].to(dt), g_cu[sl].to(dt), g_cv[sl].to(dt))
            rm = O.max_argmax_avg_backward(x1, x2, au[sl].cpu(), av[sl].cpu(), g_u[sl].to(dt), g_v[sl].to(dt))
            ref[dt] = (rc[0] + rm[0], rc[1] + rm[1], rc[0], rc[1], rm[0], rm[1])
        r64, r32 = ref[torch.float64], ref[torch.float32]
        # d_f1: a wave's register accumulator takes the products of 4 rows (128), then
        # joins a running sum: the GPU's error has to stay within twice the fp32 CPU path's, and for the reference's two
        # entry points no more elements may fall outside the plain rtol 1e-4 / atol 1e-5 than the CPU path leaves outside.
        # d_f2: the pixel range is cut into few long splits to keep the scratch small; a split adds up to 49 tiles
        # of 32 pixels in one accumulator (chain_ratio turns that length into the expected ratio); the max/avg
        # call gathers rows instead: sums of a few hundred.
        rep = error_report(d1[sl], r64[0], r32[0], f"fused d_f1 [b={b}]")
        assert rep["gpu_outside_plain_tol"] <= rep["cpu32_outside_plain_tol"], rep
        error_report(d2[sl], r64[1], r32[1], f"fused d_f2 [b={b}]", max_ratio=chain_ratio(49 * 32))
        rep = error_report(c1[sl], r64[2], r32[2], f"compression d_f1 [b={b}]")
        assert rep["gpu_outside_plain_tol"] <= rep["cpu32_outside_plain_tol"], rep
        error_report(c2[sl], r64[3], r32[3], f"compression d_f2 [b={b}]", max_ratio=chain_ratio(49 * 32))
        rep = error_report(m1[sl], r64[4], r32[4], f"max/avg d_f1 [b={b}]")
        assert rep["gpu_outside_plain_tol"] <= rep["cpu32_outside_plain_tol"], rep
        error_report(m2[sl], r64[5], r32[5], f"max/avg d_f2 [b={b}]")
        rep = error_report(n1[sl], r64[4], r32[4], f"max/avg d_f1, dense [b={b}]")
        assert rep["gpu_outside_plain_tol"] <= rep["cpu32_outside_plain_tol"], rep
        error_report(n2[sl], r64[5], r32[5], f"max/avg d_f2, dense [b={b}]", max_ratio=chain_ratio(49 * 32))
