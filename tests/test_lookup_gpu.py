"""GPU parity of the windowed pyramid lookup (sepcorr_lookup_forward through the C ABI) against the fp64 oracle.

Tolerance: rtol 1e-4 / atol 1e-5 against the oracle's stored-volume lookup in fp64 (`CorrBlock4D.lookup`), or its
gather formulation where the volume would be too large to hold.
"""
import pytest
import torch

from oracle import oracle as O
from tests._util import assert_close

pytestmark = pytest.mark.gpu


def _coords(B, H, W, g, spread):
    yy, xx = torch.meshgrid(torch.arange(H), torch.arange(W), indexing='ij')
    base = torch.stack([xx, yy]).float()[None].repeat(B, 1, 1, 1)
    return (base + torch.randn(B, 2, H, W, generator=g) * spread).contiguous()


def _native(fmap1, fmap2, coords, levels, r, device):
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    blk = AlternateCorrBlockSepflow(fmap1.to(device), fmap2.to(device), None, num_levels=levels, radius=r)
    return blk(coords.to(device))


@pytest.mark.parametrize("B,C,H,W,levels,r,spread", [
    (2, 256, 16, 24, 3, 4, 4.0),      # the model's radius and feature size
    (1, 256, 55, 128, 4, 4, 8.0),     # one image of the benchmark shape, 4 levels
    (1, 64, 11, 37, 2, 4, 3.0),       # ragged row tiles, one float4 per lane
    (1, 128, 9, 33, 2, 2, 30.0),      # most targets outside the image
    (1, 100, 8, 20, 2, 3, 2.0),       # C not a multiple of 64
    (1, 37, 8, 20, 2, 1, 2.0),        # C not a multiple of 4: scalar loads
    (1, 512, 8, 16, 1, 4, 2.0),
    (1, 1024, 4, 8, 1, 8, 2.0),       # limits: C = 1024, radius 8
])
def test_lookup_matches_stored_volume_oracle(device, B, C, H, W, levels, r, spread):
    g = torch.Generator().manual_seed(1234 + C + W)
    fmap1 = torch.randn(B, C, H, W, generator=g)
    fmap2 = torch.randn(B, C, H, W, generator=g)
    coords = _coords(B, H, W, g, spread)
    got = _native(fmap1, fmap2, coords, levels, r, device)
    if B * H * W * H * W <= 16 * 2 ** 20:
        ref = O.CorrBlock4D(fmap1.double(), fmap2.double(), num_levels=levels).lookup(coords.double(), radius=r)
    else:
        ref = O.lookup_direct(fmap1.double(), fmap2.double(), coords.double(), levels, r)
    assert got.shape == ref.shape and got.dtype == torch.float32
    assert_close(got, ref, "lookup")


def test_lookup_integer_targets_equal_the_separated_maximum(device):
    # with a window that covers the whole level, max over the window = the max channel of separate()'s inputs;
    # ties the lookup to the operators of this library through the volume itself
    from separableflowthesis_amd import MemorySaver
    B, C, H, W, r = 1, 64, 7, 7, 8
    g = torch.Generator().manual_seed(9)
    fmap1 = torch.randn(B, C, H, W, generator=g)
    fmap2 = torch.randn(B, C, H, W, generator=g)
    coords = torch.full((B, 2, H, W), 3.0)                       # window [-5, 11] covers 0..6 in both axes
    got = _native(fmap1, fmap2, coords, 1, r, device)
    f1 = (fmap1.permute(0, 2, 3, 1).contiguous() / 8.0).to(device)
    f2 = fmap2.permute(0, 2, 3, 1).contiguous().to(device)
    out_u, out_v = MemorySaver.max_avg_forward(f1, f2)
    assert_close(got.max(dim=1)[0], out_u[:, :, :, 0].max(dim=-1)[0], "window max")


def test_lookup_special_coordinates_and_errors(device):
    from separableflowthesis_amd import MemorySaver
    B, C, H, W = 1, 64, 6, 10
    g = torch.Generator().manual_seed(2)
    f1 = torch.randn(B, H, W, C, generator=g).to(device)
    f2 = torch.randn(B, H, W, C, generator=g).to(device)
    coords = torch.zeros(B, 2, H, W)
    coords[0, 0, 0, 0] = 1e30
    coords[0, 1, 0, 1] = -1e30
    coords[0, 0, 0, 2] = float('inf')
    out = MemorySaver.lookup_forward(f1, [f2], coords.to(device), 4, 0.125).cpu()
    assert float(out[0, :, 0, 0].abs().max()) == 0.0 and float(out[0, :, 0, 1].abs().max()) == 0.0
    assert bool(torch.isfinite(out[0, :, 1:, :]).all())
    with pytest.raises(RuntimeError):
        MemorySaver.lookup_forward(f1, [f2], coords.to(device), 9, 1.0)
    with pytest.raises(RuntimeError):
        MemorySaver.lookup_forward(f1, [f2], coords[:, :1].contiguous().to(device), 4, 1.0)
    with pytest.raises(RuntimeError):
        MemorySaver.lookup_forward(f1, [f2[..., :32].contiguous()], coords.to(device), 4, 1.0)
    with pytest.raises(RuntimeError):
        MemorySaver.lookup_forward(f1.cpu(), [f2], coords.to(device), 4, 1.0)
