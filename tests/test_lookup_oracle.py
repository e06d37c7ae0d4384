"""Pins the oracle of the windowed pyramid lookup (CorrBlock.__call__, core/corr.py:193-248) on the CPU.

The reference holds no vectors for this function (its tests never call the lookup), so the restatement is pinned by
what the definition fixes: direct indexing of the stored volume at integer targets, an affine volume that bilinear
sampling reproduces exactly, zero padding outside the level, the pyramid's coordinate scaling, and an independent
gather formulation that uses neither the 4D volume nor grid_sample.
"""
import pytest
import torch

from oracle import oracle as O


def _sqrt32(c):
    """sqrt(C) as the reference takes it: in fp32 (core/corr.py:282)."""
    return float(torch.sqrt(torch.tensor(c).float()))


def _grid(B, H, W, dtype=torch.float64):
    yy, xx = torch.meshgrid(torch.arange(H), torch.arange(W), indexing='ij')
    return torch.stack([xx, yy]).to(dtype)[None].repeat(B, 1, 1, 1)


def test_integer_targets_read_the_stored_volume_with_x_on_the_first_window_index():
    B, C, H, W, r = 2, 8, 9, 12, 2
    g = torch.Generator().manual_seed(3)
    fmap1 = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
    fmap2 = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
    flow = torch.randint(-3, 4, (B, 2, H, W), generator=g).double()
    coords = _grid(B, H, W) + flow
    out = O.CorrBlock4D(fmap1, fmap2, num_levels=1).lookup(coords, radius=r)
    S = torch.einsum('bcij,bcuv->bijuv', fmap1, fmap2) / _sqrt32(C)
    n = 2 * r + 1
    for b in range(B):
        for i in range(0, H, 2):
            for j in range(0, W, 3):
                x, y = int(coords[b, 0, i, j]), int(coords[b, 1, i, j])
                for a in range(n):
                    for c in range(n):
                        u, v = y + c - r, x + a - r          # x moves with a, y with c
                        want = S[b, i, j, u, v] if 0 <= u < H and 0 <= v < W else 0.0
                        assert abs(float(out[b, a * n + c, i, j]) - float(want)) < 1e-12


@pytest.mark.parametrize("levels", [1, 3])
def test_affine_volume_is_sampled_exactly_and_levels_halve_the_coordinates(levels):
    # fmap2[:,u,v] = (1,u,v) and fmap1[:,i,j] = (al,be,ga): S = al + be*u + ga*v; 2x2 pooling keeps it affine with
    # (u,v) -> (2u'+1/2, 2v'+1/2), so level l reads al + be*(2^l*(y_l+1/2)-1/2) + ga*(...) at interior targets
    B, H, W, r = 1, 16, 24, 1
    u = torch.arange(H, dtype=torch.float64).view(H, 1).expand(H, W)
    v = torch.arange(W, dtype=torch.float64).view(1, W).expand(H, W)
    fmap2 = torch.stack([torch.ones_like(u), u, v])[None]
    g = torch.Generator().manual_seed(5)
    fmap1 = torch.randn(B, 3, H, W, generator=g, dtype=torch.float64)
    coords = _grid(B, H, W) + torch.rand(B, 2, H, W, generator=g, dtype=torch.float64) * 3 - 1.5
    out = O.CorrBlock4D(fmap1, fmap2, num_levels=levels).lookup(coords, radius=r)
    n = 2 * r + 1
    checked = 0
    for lvl in range(levels):
        Hl, Wl = H >> lvl, W >> lvl
        for a in range(n):
            for c in range(n):
                xs = coords[:, 0] / 2 ** lvl + a - r
                ys = coords[:, 1] / 2 ** lvl + c - r
                inside = (xs >= 0) & (xs <= Wl - 1) & (ys >= 0) & (ys <= Hl - 1)
                uu = 2 ** lvl * (ys + 0.5) - 0.5
                vv = 2 ** lvl * (xs + 0.5) - 0.5
                want = (fmap1[:, 0] + fmap1[:, 1] * uu + fmap1[:, 2] * vv) / _sqrt32(3)
                got = out[:, lvl * n * n + a * n + c]
                assert float((got - want)[inside].abs().max()) < 1e-10
                checked += int(inside.sum())
    assert checked > 1000


def test_targets_outside_the_image_fade_to_zero():
    B, C, H, W, r = 1, 4, 6, 7, 1
    fmap1 = torch.ones(B, C, H, W, dtype=torch.float64)
    fmap2 = torch.ones(B, C, H, W, dtype=torch.float64)          # S = sqrt(C)... /sqrt(C): every sample is C/sqrt(C)
    coords = _grid(B, H, W)
    coords[:, 0] -= 0.25                                          # quarter pixel to the left
    out = O.CorrBlock4D(fmap1, fmap2, num_levels=1).lookup(coords, radius=r)
    s = C / _sqrt32(C)
    n = 2 * r + 1
    # pixel (i,0): x = -0.25; window a=0 -> x=-1.25 (fully outside), a=1 -> -0.25 (weight 0.75 on column 0)
    assert abs(float(out[0, 0 * n + 1, 2, 0])) < 1e-12
    assert abs(float(out[0, 1 * n + 1, 2, 0]) - 0.75 * s) < 1e-12
    assert abs(float(out[0, 2 * n + 1, 2, 0]) - s) < 1e-12
    # far away: nothing
    far = coords + 100.0
    assert float(O.CorrBlock4D(fmap1, fmap2, num_levels=1).lookup(far, radius=r).abs().max()) == 0.0


@pytest.mark.parametrize("B,C,H,W,levels,r", [(2, 16, 16, 24, 3, 3), (1, 5, 11, 13, 2, 4), (1, 32, 16, 40, 4, 4)])
def test_gather_formulation_equals_the_stored_volume_lookup(B, C, H, W, levels, r):
    g = torch.Generator().manual_seed(11)
    fmap1 = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
    fmap2 = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
    coords = _grid(B, H, W) + torch.randn(B, 2, H, W, generator=g, dtype=torch.float64) * 6
    a = O.CorrBlock4D(fmap1, fmap2, num_levels=levels).lookup(coords, radius=r)
    b = O.lookup_direct(fmap1, fmap2, coords, levels, r)
    assert a.shape == (B, levels * (2 * r + 1) ** 2, H, W)
    assert float((a - b).abs().max()) < 1e-11


def test_a_level_of_size_one_is_undefined_in_the_stored_volume_path_only():
    # the reference normalises by (H-1), (W-1) (core/utils/utils.py:114-115): a level with one row or column gives
    # NaN there; the gather formulation (and the native kernel) keep the definition's value instead
    g = torch.Generator().manual_seed(4)
    fmap1 = torch.randn(1, 4, 2, 6, generator=g, dtype=torch.float64)
    fmap2 = torch.randn(1, 4, 2, 6, generator=g, dtype=torch.float64)
    coords = _grid(1, 2, 6)
    a = O.CorrBlock4D(fmap1, fmap2, num_levels=2).lookup(coords, radius=1)
    b = O.lookup_direct(fmap1, fmap2, coords, 2, 1)
    assert bool(torch.isnan(a[:, 9:]).any()) and bool(torch.isfinite(b).all())
    assert float((a[:, :9] - b[:, :9]).abs().max()) < 1e-12


def test_gradients_of_both_formulations_agree():
    # autograd through grid_sample on the stored pyramid against autograd through the gather formulation
    B, C, H, W, levels, r = 1, 6, 8, 12, 2, 2
    g = torch.Generator().manual_seed(21)
    fmap1 = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
    fmap2 = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
    coords = _grid(B, H, W) + torch.randn(B, 2, H, W, generator=g, dtype=torch.float64) * 2
    up = torch.randn(B, levels * (2 * r + 1) ** 2, H, W, generator=g, dtype=torch.float64)
    grads = []
    for fn in (lambda a, b: O.CorrBlock4D(a, b, num_levels=levels).lookup(coords, radius=r),
               lambda a, b: O.lookup_direct(a, b, coords, levels, r)):
        a = fmap1.clone().requires_grad_()
        b = fmap2.clone().requires_grad_()
        (fn(a, b) * up).sum().backward()
        grads.append((a.grad, b.grad))
    assert float((grads[0][0] - grads[1][0]).abs().max()) < 1e-11
    assert float((grads[0][1] - grads[1][1]).abs().max()) < 1e-11
    # the lookup is bilinear in (fmap1, fmap2): <up, out> = <d_fmap1, fmap1> = <d_fmap2, fmap2>
    val = float((O.lookup_direct(fmap1, fmap2, coords, levels, r) * up).sum())
    assert abs(float((grads[1][0] * fmap1).sum()) - val) < 1e-9 * max(1.0, abs(val))
    assert abs(float((grads[1][1] * fmap2).sum()) - val) < 1e-9 * max(1.0, abs(val))


def _golden():
    import glob
    import os
    import numpy as np
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lookup")
    for f in sorted(glob.glob(os.path.join(here, "*.npz"))):
        z = np.load(f, allow_pickle=False)
        yield os.path.basename(f), {k: torch.from_numpy(z[k]) for k in z.files}


def test_oracle_reproduces_the_lookup_golden_vectors():
    names = []
    for name, z in _golden():
        names.append(name)
        levels, r = int(z["in_levels"]), int(z["in_radius"])
        a = z["in_fmap1"].double().requires_grad_()
        b = z["in_fmap2"].double().requires_grad_()
        out = O.lookup_direct(a, b, z["in_coords"].double(), levels, r)      # the formulation the files were not made with
        (out * z["in_up"].double()).sum().backward()
        assert torch.allclose(out.detach().float(), z["out_lookup"], rtol=1e-6, atol=1e-6), name
        assert torch.allclose(a.grad.float(), z["out_d_fmap1"], rtol=1e-6, atol=1e-5), name
        assert torch.allclose(b.grad.float(), z["out_d_fmap2"], rtol=1e-6, atol=1e-5), name
    assert len(names) == 2
