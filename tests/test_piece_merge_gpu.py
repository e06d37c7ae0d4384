"""Sweeps dealt out in pieces of tiles against the same sweeps run tile by tile, under memory traffic from a second stream.

With a workspace the forward-type sweeps (and d_f1) cut a pixel tile's rows into pieces that different workgroups take;
a piece leaves its column state in a slot in device memory, counts itself in, and whichever piece of a tile arrives last
adds up all pieces in row order.  Without a workspace every workgroup sweeps whole tiles and nothing is handed over.
Maxima and argmax must come out bit-equal either way (the merge keeps the lower row on ties, as the unsplit sweep does);
sums differ by the rounding of a different association only.  The hand-over relies on stores and loads that go through
to device memory and on a device-scope atomic counter; the launches below run it 200 times per size while another
stream of the same GPU streams a buffer through the memory system, and stop at the first difference.
Called through the C ABI.
"""
import pytest
import torch

from separableflowthesis_amd import _lib
from tests._util import op_inputs

pytestmark = pytest.mark.gpu

LAUNCHES = 200


@pytest.mark.parametrize("dims", [(1, 48, 64, 48, 64, 256), (2, 55, 128, 55, 128, 256)], ids=["cfg1", "cfg4"])
def test_split_and_unsplit_sweeps_agree_under_memory_traffic(device, dims):
    lib = _lib.load()
    B, H1, W1, H2, W2, C = dims
    f1, f2, g = op_inputs(*dims, seed=31)
    f1, f2 = f1.to(device), f2.to(device)
    K = 4
    a_u = torch.randn(B, H1, W1, K, W2, generator=g).softmax(-1).to(device)
    a_v = torch.randn(B, H1, W1, K, H2, generator=g).softmax(-1).to(device)
    P = lambda t: t.data_ptr()
    E = lambda *s, dt=torch.float32: torch.empty(*s, dtype=dt, device=device)
    nws = lib.sepcorr_forward_workspace_bytes(*dims, K)
    assert nws > 0, "these sizes are dealt out in pieces when a workspace is given"
    ws = torch.empty(nws, dtype=torch.uint8, device=device)
    main = torch.cuda.current_stream()

    def maxavg(wptr, n):
        ou, ov = E(B, H1, W1, 2, H2), E(B, H1, W1, 2, W2)
        au, av = E(B, H1, W1, 1, H2, dt=torch.int32), E(B, H1, W1, 1, W2, dt=torch.int32)
        _lib.check(lib.sepcorr_max_argmax_avg_forward(P(f1), P(f2), P(ou), P(ov), P(au), P(av), *dims, wptr, n, main.cuda_stream))
        return ou, ov, au, av

    def weighted(wptr, n):
        cu, cv = E(B, H1, W1, K, H2), E(B, H1, W1, K, W2)
        _lib.check(lib.sepcorr_compression_forward(P(f1), P(f2), P(a_u), P(a_v), P(cu), P(cv), *dims, K, wptr, n, main.cuda_stream))
        return cu, cv

    # the reference results: whole tiles, no hand-over, idle chip
    rou, rov, rau, rav = maxavg(None, 0)
    rcu, rcv = weighted(None, 0)
    torch.cuda.synchronize()

    # memory traffic beside the sweeps: copies of 256 MiB back and forth on a second stream
    side = torch.cuda.Stream()
    src = torch.empty(64 << 20, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    for n in range(LAUNCHES):
        with torch.cuda.stream(side):
            for _ in range(2):
                dst.copy_(src, non_blocking=True)
                src.copy_(dst, non_blocking=True)
        ou, ov, au, av = maxavg(P(ws), nws)
        cu, cv = weighted(P(ws), nws)
        torch.cuda.synchronize()
        assert torch.equal(ou[:, :, :, 0], rou[:, :, :, 0]), f"launch {n}: max over columns differs"
        assert torch.equal(ov[:, :, :, 0], rov[:, :, :, 0]), f"launch {n}: max over rows differs (merged pieces)"
        assert torch.equal(au, rau), f"launch {n}: argmax_u differs"
        assert torch.equal(av, rav), f"launch {n}: argmax_v differs (merged pieces)"
        for got, ref, name in ((ou[:, :, :, 1], rou[:, :, :, 1], "avg_u"), (ov[:, :, :, 1], rov[:, :, :, 1], "avg_v"),
                               (cu, rcu, "comp_u"), (cv, rcv, "comp_v")):
            err = float((got - ref).abs().max())
            assert err <= 2e-6 * max(1.0, float(ref.abs().max())), f"launch {n}: {name} differs by {err}"
    side.synchronize()


def test_split_d_f1_agrees_with_itself_under_memory_traffic(device):
    """d_f1 of the compression backward is dealt out in pieces as well (partial [32 pixels][channels] sums in slots):
    run to run identical, also beside another stream's traffic."""
    lib = _lib.load()
    dims = (2, 55, 128, 55, 128, 256)
    B, H1, W1, H2, W2, C = dims
    K = 4
    f1, f2, g = op_inputs(*dims, seed=32)
    f1, f2 = f1.to(device), f2.to(device)
    a_u = torch.randn(B, H1, W1, K, W2, generator=g).softmax(-1).to(device)
    a_v = torch.randn(B, H1, W1, K, H2, generator=g).softmax(-1).to(device)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g).to(device)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g).to(device)
    P = lambda t: t.data_ptr()
    nws = lib.sepcorr_backward_workspace_bytes(*dims)
    ws = torch.empty(nws, dtype=torch.uint8, device=device)
    main = torch.cuda.current_stream()

    def call():
        d1, d2 = torch.empty_like(f1), torch.empty_like(f2)
        da_u, da_v = torch.empty_like(a_u), torch.empty_like(a_v)
        _lib.check(lib.sepcorr_compression_backward(P(f1), P(f2), P(a_u), P(a_v), P(g_cu), P(g_cv), P(d1), P(d2), P(da_u), P(da_v),
                                                    *dims, K, P(ws), nws, main.cuda_stream))
        return d1, d2, da_u, da_v

    ref = call()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    src = torch.empty(64 << 20, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    for n in range(50):
        with torch.cuda.stream(side):
            dst.copy_(src, non_blocking=True)
            src.copy_(dst, non_blocking=True)
        got = call()
        torch.cuda.synchronize()
        for x, y, name in zip(got, ref, ("d_f1", "d_f2", "d_a_u", "d_a_v")):
            assert torch.equal(x, y), f"launch {n}: {name} differs from the first call's"
    side.synchronize()


@pytest.mark.parametrize("dims", [(1, 55, 128, 55, 128, 256), (1, 48, 64, 48, 64, 256)], ids=["cfg3", "cfg1"])
def test_sweep_with_and_without_scratch(device, dims):
    """The shape of the workgroups depends on whether the steps are dealt out (scratch given: two 4-wave workgroups per
    CU) or whole tiles are swept (no scratch: 8 waves): same maxima and argmax, sums to rounding.  A buffer smaller
    than sepcorr_forward_workspace_bytes() is refused, not silently ignored."""
    lib = _lib.load()
    B, H1, W1, H2, W2, C = dims
    f1, f2, g = op_inputs(*dims, seed=33)
    f1, f2 = f1.to(device), f2.to(device)
    P = lambda t: t.data_ptr()
    E = lambda *s, dt=torch.float32: torch.empty(*s, dtype=dt, device=device)
    nws = lib.sepcorr_forward_workspace_bytes(*dims, 2)
    assert nws > 0
    ws = torch.empty(nws, dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream().cuda_stream

    def run(n):
        ou, ov = E(B, H1, W1, 2, H2), E(B, H1, W1, 2, W2)
        au, av = E(B, H1, W1, 1, H2, dt=torch.int32), E(B, H1, W1, 1, W2, dt=torch.int32)
        rc = lib.sepcorr_max_argmax_avg_forward(P(f1), P(f2), P(ou), P(ov), P(au), P(av), *dims, P(ws) if n else None, n, stream)
        torch.cuda.synchronize()
        return rc, (ou, ov, au, av)

    rc, ref = run(nws)
    assert rc == 0
    rc, got = run(0)
    assert rc == 0
    assert torch.equal(got[0][:, :, :, 0], ref[0][:, :, :, 0]) and torch.equal(got[1][:, :, :, 0], ref[1][:, :, :, 0]), "maxima differ"
    assert torch.equal(got[2], ref[2]) and torch.equal(got[3], ref[3]), "argmax differs"
    for x, y in ((got[0][:, :, :, 1], ref[0][:, :, :, 1]), (got[1][:, :, :, 1], ref[1][:, :, :, 1])):
        assert float((x - y).abs().max()) <= 2e-6 * max(1.0, float(y.abs().max())), "averages differ"
    rc, _ = run((nws // 2) & ~255)
    assert rc != 0 and b"workspace" in lib.sepcorr_last_error()
