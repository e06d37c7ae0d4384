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


@pytest.mark.parametrize("B,C,H,W,levels,r,spread", [
    (2, 256, 16, 24, 3, 4, 3.0),
    (1, 256, 28, 64, 4, 4, 6.0),      # half the benchmark shape: sliced pixel ranges on the coarse levels
    (1, 64, 11, 37, 2, 4, 3.0),       # ragged tiles of fmap2 positions
    (1, 100, 9, 20, 2, 3, 25.0),      # most windows outside, C not a multiple of 64
    (1, 37, 8, 20, 2, 1, 2.0),
    (1, 300, 8, 16, 2, 2, 2.0),       # two channel blocks in the d_f2 kernel
    (1, 64, 10, 12, 1, 2, 2.0),       # a single level
    (3, 32, 6, 70, 2, 4, 1.0),        # batch of three, long rows, one float4 per lane
])
def test_lookup_gradients_match_autograd_through_the_oracle(device, B, C, H, W, levels, r, spread):
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    g = torch.Generator().manual_seed(4321 + C + W)
    fmap1 = torch.randn(B, C, H, W, generator=g)
    fmap2 = torch.randn(B, C, H, W, generator=g)
    coords = _coords(B, H, W, g, spread)
    up = torch.randn(B, levels * (2 * r + 1) ** 2, H, W, generator=g)
    r1 = fmap1.double().requires_grad_()
    r2 = fmap2.double().requires_grad_()
    (O.lookup_direct(r1, r2, coords.double(), levels, r) * up.double()).sum().backward()
    g1 = fmap1.to(device).requires_grad_()
    g2 = fmap2.to(device).requires_grad_()
    blk = AlternateCorrBlockSepflow(g1, g2, None, num_levels=levels, radius=r)
    out = blk(coords.to(device))
    out.backward(up.to(device), retain_graph=True)       # the block's NHWC copies are shared by later calls
    assert_close(g1.grad, r1.grad, "d_fmap1", scale_atol=True)
    assert_close(g2.grad, r2.grad, "d_fmap2", scale_atol=True)
    # a second call on the same block (next flow iteration) accumulates into the same leaves
    blk(coords.to(device)).backward(up.to(device))
    assert_close(g1.grad, 2 * r1.grad, "d_fmap1 accumulated", scale_atol=True)


def test_lookup_backward_is_deterministic_and_checks_its_workspace(device):
    import ctypes
    from separableflowthesis_amd import MemorySaver, _lib
    B, C, H, W, r = 1, 64, 12, 20, 4
    g = torch.Generator().manual_seed(8)
    f1 = torch.randn(B, H, W, C, generator=g).to(device)
    f2s = [torch.randn(B, H >> l, W >> l, C, generator=g).to(device) for l in range(3)]
    coords = _coords(B, H, W, g, 3.0).to(device)
    up = torch.randn(B, 3 * 81, H, W, generator=g).to(device)
    a = MemorySaver.lookup_backward(f1, f2s, coords, up, r, 0.125)
    b = MemorySaver.lookup_backward(f1, f2s, coords, up, r, 0.125)
    assert torch.equal(a[0], b[0]) and all(torch.equal(x, y) for x, y in zip(a[1], b[1]))
    lib = _lib.load()
    ptrs = (ctypes.c_void_p * 3)(*[t.data_ptr() for t in f2s])
    h2 = (ctypes.c_int * 3)(*[t.shape[1] for t in f2s])
    w2 = (ctypes.c_int * 3)(*[t.shape[2] for t in f2s])
    need = lib.sepcorr_lookup_backward_workspace_bytes(h2, w2, B, H, W, C, 3, r)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    rc = lib.sepcorr_lookup_backward(f1.data_ptr(), ptrs, h2, w2, coords.data_ptr(), up.data_ptr(), a[0].data_ptr(),
                                     ptrs, B, H, W, C, 3, r, 0.125, ws.data_ptr(), need - 1, None)
    assert rc == -3 and b"workspace" in lib.sepcorr_last_error()


def test_lookup_matches_the_golden_vectors(device):
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    from tests.test_lookup_oracle import _golden
    n = 0
    for name, z in _golden():
        n += 1
        g1 = z["in_fmap1"].to(device).requires_grad_()
        g2 = z["in_fmap2"].to(device).requires_grad_()
        blk = AlternateCorrBlockSepflow(g1, g2, None, num_levels=int(z["in_levels"]), radius=int(z["in_radius"]))
        out = blk(z["in_coords"].to(device))
        out.backward(z["in_up"].to(device))
        assert_close(out, z["out_lookup"], name + " lookup")
        assert_close(g1.grad, z["out_d_fmap1"], name + " d_fmap1", scale_atol=True)
        assert_close(g2.grad, z["out_d_fmap2"], name + " d_fmap2", scale_atol=True)
    assert n == 2


def _lookup_tensors(device, seed, B=1, C=64, H=12, W=20, L=3, r=4):
    g = torch.Generator().manual_seed(seed)
    t = dict(f1=torch.randn(B, H, W, C, generator=g), coords=_coords(B, H, W, g, 3.0),
             up=torch.randn(B, L * (2 * r + 1) ** 2, H, W, generator=g))
    for l in range(L):
        t[f"f2_{l}"] = torch.randn(B, H >> l, W >> l, C, generator=g)
    return {k: v.to(device) for k, v in t.items()}


def _lookup_ops(t, L=3, r=4):
    from separableflowthesis_amd import MemorySaver
    f2s = [t[f"f2_{l}"] for l in range(L)]
    out = MemorySaver.lookup_forward(t["f1"], f2s, t["coords"], r, 0.125)
    d_f1, d_f2 = MemorySaver.lookup_backward(t["f1"], f2s, t["coords"], t["up"], r, 0.125)
    return [out, d_f1] + d_f2


def test_lookup_follows_the_callers_stream_and_replays_from_a_captured_graph(device):
    ref = _lookup_ops(_lookup_tensors(device, 91))
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        t = {k: v * 1.0 for k, v in _lookup_tensors(device, 91).items()}    # produced on s: the kernels must wait for it
        got = _lookup_ops(t)
    s.synchronize()
    assert all(torch.equal(x, y) for x, y in zip(got, ref))
    static = _lookup_tensors(device, 92)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _lookup_ops(static)
    for seed in (93, 94, 95):
        fresh = _lookup_tensors(device, seed)
        ref = _lookup_ops(fresh)                  # eager work between the replays
        torch.cuda.synchronize()
        for k in static:
            static[k].copy_(fresh[k])
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(x, y) for x, y in zip(outs, ref)), f"replay with seed {seed} differs from eager"


def test_lookup_at_the_high_resolution_size_on_row_bands(device):
    # B=1, C=256, 136x240 (the largest benchmark shape; its 4D volume would be 4.3 GB).  Image-1 pixels are independent
    # units of the lookup, so the oracle evaluates three bands of rows and those rows of the full GPU result are compared,
    # values and d_fmap1; d_fmap2 is checked through the bilinear identity <up, out> = <d_fmap2, fmap2>.
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    B, C, H, W, L, r = 1, 256, 136, 240, 4, 4
    g = torch.Generator().manual_seed(2024)
    fmap1 = torch.randn(B, C, H, W, generator=g)
    fmap2 = torch.randn(B, C, H, W, generator=g)
    coords = _coords(B, H, W, g, 5.0)
    up = torch.randn(B, L * 81, H, W, generator=g)
    g1 = fmap1.to(device).requires_grad_()
    g2 = fmap2.to(device).requires_grad_()
    out = AlternateCorrBlockSepflow(g1, g2, None, num_levels=L, radius=r)(coords.to(device))
    out.backward(up.to(device))
    for i0 in (0, 67, 134):
        rows = slice(i0, i0 + 2)
        a = fmap1[:, :, rows].double().requires_grad_()
        ref = O.lookup_direct(a, fmap2.double(), coords[:, :, rows].double(), L, r)
        (ref * up[:, :, rows].double()).sum().backward()
        assert_close(out[:, :, rows], ref, f"lookup rows {i0}..")
        assert_close(g1.grad[:, :, rows], a.grad, f"d_fmap1 rows {i0}..", scale_atol=True)
    lhs = float((out.detach().double().cpu() * up.double()).sum())
    rhs = float((g2.grad.double().cpu() * fmap2.double()).sum())
    assert abs(lhs - rhs) <= 1e-4 * abs(lhs) + 1e-2
