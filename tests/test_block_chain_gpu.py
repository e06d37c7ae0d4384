"""End-to-end parity of the in-scope part of the model's correlation chain, forward and gradients.

The model runs (core/sepflow.py:128-204): corr_fn = AlternateCorrBlockSepflow(fmap1, fmap2) ->
corr1, corr2 = corr_fn(None, sep=True, attention_weights) -> cost aggregation (GANet, not part of this build:
a seeded pointwise channel mix stands in for it, the same torch module on both sides) -> CorrBlock1D(corr1, corr2)
-> per flow iteration corr1d_fn(coords) and, without --no_4d_corr, corr_fn(coords).

Here that chain runs through the native block and lookups on the GPU and through the stored-4D-volume oracle
(CorrBlock4D.separate / .lookup, oracle.CorrBlock1D) in fp64 on the CPU; compared are all lookup outputs and the
gradients of a loss on them with respect to fmap1, fmap2, the attention parameters and the stand-in's parameters:
the gradient comparison of scripts/test_model.py:273-318 for the part of the model this build covers.  Peak
memory of both chains is printed (scripts/test_model.py:320-382 measures the same on the whole model).
"""
import copy

import pytest
import torch

from oracle import oracle as O
from tests._util import assert_close, check_argmax_levels, error_report, native_argmax_levels

pytestmark = pytest.mark.gpu


def _coords(B, H, W, gen, iters):
    yy, xx = torch.meshgrid(torch.arange(H), torch.arange(W), indexing="ij")
    base = torch.stack([xx, yy]).float()[None].expand(B, 2, H, W)
    out = []
    for it in range(iters):
        flow = torch.randn(B, 2, 1, 1, generator=gen) * 3 + torch.randn(B, 2, H, W, generator=gen) * (0.5 + it)
        out.append((base + flow).contiguous())
    return out


def _chain(fmap1, fmap2, att, agg, coords_list, weights, use_4d_lookup, native, dtype, device, argmax=None):
    """Runs the chain and the backward pass; returns (outputs, gradients) as CPU tensors."""
    cast = (lambda t: t.to(device)) if native else (lambda t: t.to(dtype))
    x1, x2 = cast(fmap1).requires_grad_(), cast(fmap2).requires_grad_()
    matt = tuple(copy.deepcopy(m) for m in att)
    magg = tuple(copy.deepcopy(m) for m in agg)
    for m in matt + magg:
        m.to(device) if native else m.to(dtype)
    if native:
        from separableflowthesis_amd import AlternateCorrBlockSepflow, CorrBlock1D
        corr_fn = AlternateCorrBlockSepflow(x1, x2, None, num_levels=4, radius=4, support_backward=True)
        corr1, corr2 = corr_fn(None, sep=True, attention_weights=matt)
    else:
        corr_fn = O.CorrBlock4D(x1, x2, num_levels=4)
        if dtype == torch.float64:
            print(f"argmax near-tie mismatches: {check_argmax_levels(argmax, corr_fn, 'chain')}", flush=True)
        corr1, corr2 = corr_fn.separate(matt, argmax=argmax)   # maxima read where the native block found them
    corr1, corr2 = magg[0](corr1), magg[1](corr2)          # stand-in for cost_agg1 / cost_agg2: (B,1,L,H,W)
    one_d = CorrBlock1D(corr1, corr2, num_levels=4, radius=4) if native else O.CorrBlock1D(corr1, corr2, 4, 4)
    outs, loss = [], 0
    for it, coords in enumerate(coords_list):
        c = cast(coords)
        o1, o2 = one_d(c)
        group = [o1, o2]
        if use_4d_lookup:
            group.append(corr_fn(c) if native else corr_fn.lookup(c, radius=4))
        for o, w in zip(group, weights[it]):
            loss = loss + (o * cast(w)).sum()
        outs += group
    loss.backward()
    grads = [x1.grad, x2.grad] + [p.grad for m in matt + magg for p in m.parameters()]
    return [o.detach().cpu() for o in outs], [g.detach().cpu() for g in grads]


@pytest.mark.parametrize("B,C,H,W,K,use_4d", [(2, 128, 24, 40, 2, True), (1, 256, 40, 64, 4, True), (2, 64, 16, 16, 4, False)])
def test_separate_then_lookups_forward_and_gradients(device, B, C, H, W, K, use_4d):
    fmap1, fmap2, _, _ = O.make_inputs(B, H, W, C, seed=21)
    torch.manual_seed(17)
    att = (torch.nn.Conv3d(2, K, 3, padding=1), torch.nn.Conv3d(2, K, 3, padding=1))
    nch = (2 + K) * 4
    agg = (torch.nn.Conv3d(nch, 1, 1), torch.nn.Conv3d(nch, 1, 1))
    gen = torch.Generator().manual_seed(5)
    iters = 3
    coords = _coords(B, H, W, gen, iters)
    n1, n4 = 4 * 9, 4 * 81
    weights = [[torch.randn(B, n1, H, W, generator=gen), torch.randn(B, n1, H, W, generator=gen),
                torch.randn(B, n4, H, W, generator=gen) / 8] for _ in range(iters)]

    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    got_o, got_g = _chain(fmap1, fmap2, att, agg, coords, weights, use_4d, True, None, device)
    torch.cuda.synchronize()
    peak_native = torch.cuda.max_memory_allocated() - base
    argmax = native_argmax_levels(fmap1, fmap2, device)
    ref_o, ref_g = _chain(fmap1, fmap2, att, agg, coords, weights, use_4d, False, torch.float64, device, argmax)
    c32_o, c32_g = _chain(fmap1, fmap2, att, agg, coords, weights, use_4d, False, torch.float32, device, argmax)
    pyramid_4d = B * (H * W) ** 2 * 4 * (1 + 1 / 4 + 1 / 16 + 1 / 64)
    print(f"chain B={B} C={C} {H}x{W} K'={K}: native peak {peak_native / 2**20:.1f} MiB, "
          f"stored 4D pyramid alone {pyramid_4d / 2**20:.1f} MiB", flush=True)

    per_it = 3 if use_4d else 2
    names = ("corr1d out1", "corr1d out2", "corr_fn(coords)")
    for i, (g, r) in enumerate(zip(got_o, ref_o)):
        assert_close(g, r, f"iteration {i // per_it}: {names[i % per_it]}", scale_atol=True)
    gnames = ["d_fmap1", "d_fmap2", "attention1.weight.grad", "attention1.bias.grad", "attention2.weight.grad",
              "attention2.bias.grad", "agg1.weight.grad", "agg1.bias.grad", "agg2.weight.grad", "agg2.bias.grad"]
    for g, r, c, n in zip(got_g, ref_g, c32_g, gnames):
        if n.startswith("agg"):   # torch's own Conv3d gradient on the GPU: not this library's arithmetic
            assert_close(g, r, n, scale_atol=True)
        else:
            error_report(g, r, c, n, max_ratio=3.0)
