"""Pins the oracle of the 3D-volume lookup (CorrBlock1D, core/corr.py:513-624) on the CPU.

The reference holds no vectors for it.  Pinned by: integer targets read pyramid entries that are explicit means of the
stored volume; an affine profile along the displacement axis is reproduced exactly at every level; zero padding at the
ends; the [-1, 1] clamp of the first volume; and an independent formulation without avg_pool2d and grid_sample.
"""
import pytest
import torch

from oracle import oracle as O


def _grid(B, H, W, dtype=torch.float64):
    yy, xx = torch.meshgrid(torch.arange(H), torch.arange(W), indexing='ij')
    return torch.stack([xx, yy]).to(dtype)[None].repeat(B, 1, 1, 1)


def _volumes(B, dim, H, W, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, dim, W, H, W, generator=g, dtype=torch.float64),
            torch.randn(B, dim, H, H, W, generator=g, dtype=torch.float64), g)


def test_integer_targets_read_means_of_the_stored_second_volume():
    B, dim, H, W, r, L = 1, 2, 16, 12, 2, 3
    c1, c2, g = _volumes(B, dim, H, W, 1)
    coords = _grid(B, H, W)
    coords[:, 1] = (coords[:, 1] // 4) * 4 + 4.0            # y a multiple of 4: integer at levels 0..2
    _, out2 = O.CorrBlock1D(c1, c2, num_levels=L, radius=r)(coords)
    n = 2 * r + 1
    for l in range(L):
        for d in range(dim):
            for k in range(n):
                for (i, j) in ((0, 0), (5, 7), (15, 11)):
                    m = int(coords[0, 1, i, j]) // 2 ** l + k - r
                    want = c2[0, d, m * 2 ** l:(m + 1) * 2 ** l, i, j].mean() if 0 <= m < H >> l else 0.0
                    got = out2[0, l * dim * n + d * n + k, i, j]
                    assert abs(float(got) - float(want)) < 1e-12


def test_affine_profile_is_reproduced_at_every_level_inside_the_volume():
    B, dim, H, W, r, L = 1, 1, 32, 8, 1, 3
    w = torch.arange(H, dtype=torch.float64).view(1, 1, H, 1, 1)
    g = torch.Generator().manual_seed(2)
    al = torch.randn(B, 1, 1, H, W, generator=g, dtype=torch.float64)
    be = torch.randn(B, 1, 1, H, W, generator=g, dtype=torch.float64)
    c2 = al + be * w                                          # affine along the displacement axis, per pixel
    c1 = torch.zeros(B, dim, W, H, W, dtype=torch.float64)
    coords = _grid(B, H, W) + torch.rand(B, 2, H, W, generator=g, dtype=torch.float64) * 2 - 1
    _, out2 = O.CorrBlock1D(c1, c2, num_levels=L, radius=r)(coords)
    checked = 0
    for l in range(L):
        for k in range(3):
            pos = coords[:, 1] / 2 ** l + k - r
            inside = (pos >= 0) & (pos <= (H >> l) - 1)
            want = al[:, 0, 0] + be[:, 0, 0] * (2 ** l * (pos + 0.5) - 0.5)     # pooling maps entry m to 2^l (m + 1/2) - 1/2
            got = out2[:, l * 3 + k]
            assert float((got - want)[inside].abs().max()) < 1e-10
            checked += int(inside.sum())
    assert checked > 1000


def test_first_volume_positions_are_clamped_to_the_unit_interval():
    # core/corr.py:593: every sampling position of corr1 ends up in [-1, 1], wherever the flow points
    B, dim, H, W, r = 1, 1, 6, 8, 2
    c1, c2, g = _volumes(B, dim, H, W, 3)
    coords = _grid(B, H, W) + 3.0
    out1, _ = O.CorrBlock1D(c1, c2, num_levels=1, radius=r)(coords)
    # x >= 3: x + k - r >= 1 for all k, clamped to 1: every window entry reads column 1 of the volume
    for k in range(2 * r + 1):
        assert float((out1[0, k] - c1[0, 0, 1]).abs().max()) < 1e-12
    far = coords - 100.0                                      # clamped to -1: outside, zero
    out1, _ = O.CorrBlock1D(c1, c2, num_levels=1, radius=r)(far)
    assert float(out1.abs().max()) < 1e-12   # position -1 exactly: full weight on entry -1, none on entry 0


@pytest.mark.parametrize("B,dim,H,W,L,r", [(2, 3, 10, 24, 3, 2), (1, 1, 16, 16, 4, 4), (1, 6, 9, 11, 2, 3)])
def test_direct_formulation_equals_the_pooled_grid_sample_path(B, dim, H, W, L, r):
    c1, c2, g = _volumes(B, dim, H, W, 4)
    coords = _grid(B, H, W) + torch.randn(B, 2, H, W, generator=g, dtype=torch.float64) * 4
    o1, o2 = O.CorrBlock1D(c1, c2, num_levels=L, radius=r)(coords)
    d1 = O.lookup1d_direct(c1, coords[:, 0], L, r, True)
    d2 = O.lookup1d_direct(c2, coords[:, 1], L, r, False)
    assert o1.shape == (B, L * dim * (2 * r + 1), H, W)
    assert float((o1 - d1).abs().max()) < 1e-12 and float((o2 - d2).abs().max()) < 1e-12
