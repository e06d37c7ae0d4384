"""Tensors that are only 4-byte aligned: the attention and assemble kernels that move 8 or 16 bytes per lane must stand
back for the ones that do not, with the same results.

The Python mirror allocates every output itself (256-byte aligned), so these calls go through the C ABI with tensors
placed one float into larger buffers."""
import ctypes

import pytest
import torch

from separableflowthesis_amd import _lib

pytestmark = pytest.mark.gpu


def _shifted(t, device):
    """A contiguous copy of t whose first element lies 4 bytes past a 256-byte boundary."""
    buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=device)
    view = buf[1:].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 8 == 4
    return view


@pytest.mark.parametrize("B,H1,W1,L,K", [(1, 5, 9, 128, 4), (2, 4, 6, 64, 4), (1, 3, 7, 240, 2), (1, 4, 5, 27, 3)])
def test_attention_kernels_on_unaligned_tensors(device, B, H1, W1, L, K):
    lib = _lib.load()
    g = torch.Generator().manual_seed(21)
    sep = torch.randn(B, H1, W1, 2, L, generator=g).to(device)
    w = (torch.randn(K, 2, 3, 3, 3, generator=g) * 0.3).to(device)
    bias = torch.randn(K, generator=g).to(device)
    dz = torch.randn(B, H1, W1, K, L, generator=g).to(device)
    init = torch.randn(B, H1, W1, 2, L, generator=g).to(device)
    P = lambda t: t.data_ptr()
    s = torch.cuda.current_stream().cuda_stream
    nws = lib.sepcorr_attention_logits_levels_workspace_bytes((ctypes.c_int * 1)(L), 1, B, H1, W1, K)
    ws = torch.empty(max(nws, 1), dtype=torch.uint8, device=device)
    arr = lambda ts: (ctypes.c_void_p * len(ts))(*[P(t) for t in ts])

    def run(sep_, dz_, init_, shift_out):
        mk = (lambda t: _shifted(torch.zeros_like(t), device)) if shift_out else torch.zeros_like
        z, st, d_sep = mk(dz), torch.zeros(B, H1, W1, K, 2, device=device), mk(sep)
        d_w, d_b = torch.zeros_like(w), torch.zeros_like(bias)
        _lib.check(lib.sepcorr_attention_logits_forward(P(sep_), P(w), P(bias), P(z), P(st), B, H1, W1, L, K, s))
        _lib.check(lib.sepcorr_attention_logits_backward_levels(arr([sep_]), P(w), arr([dz_]), arr([init_]), arr([d_sep]), P(d_w), P(d_b),
                                                               (ctypes.c_int * 1)(L), 1, B, H1, W1, K, P(ws), nws, s))
        torch.cuda.synchronize()
        return z, st, d_sep, d_w, d_b

    ref = run(sep, dz, init, False)
    for which in range(4):   # one tensor off at a time, then all of them
        args = [sep, dz, init]
        if which < 3:
            args[which] = _shifted(args[which], device)
        else:
            args = [_shifted(t, device) for t in args]
        got = run(*args, shift_out=which == 3)
        for x, y, name in zip(got, ref, ("logits", "row statistics", "d_sep", "d_weight", "d_bias")):
            tol = 1e-5 * float(y.abs().max()) + 1e-6
            err = float((x - y).abs().max())
            assert err <= tol, f"case {which}: {name} differs by {err} (allowed {tol})"


@pytest.mark.parametrize("B,H1,W1,L0,specs", [(2, 5, 40, 64, [(2, 64), (4, 64), (2, 32), (4, 16)]),
                                              (1, 3, 12, 27, [(2, 27), (4, 13)])])
def test_assemble_on_unaligned_tensors(device, B, H1, W1, L0, specs):
    lib = _lib.load()
    g = torch.Generator().manual_seed(22)
    srcs = [torch.randn(B, H1, W1, ch, Li, generator=g).to(device) for ch, Li in specs]
    CT = sum(ch for ch, _ in specs)
    grad = torch.randn(B, CT, L0, H1, W1, generator=g).to(device)
    n = len(specs)
    ch = (ctypes.c_int * n)(*[c for c, _ in specs])
    li = (ctypes.c_int * n)(*[l for _, l in specs])
    arr = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    s = torch.cuda.current_stream().cuda_stream

    def run(shift):
        mk = (lambda t: _shifted(t, device)) if shift else (lambda t: t)
        ins = [mk(t) for t in srcs]
        dst = mk(torch.zeros(B, CT, L0, H1, W1, device=device))
        _lib.check(lib.sepcorr_assemble_forward_multi(arr(ins), ch, li, n, dst.data_ptr(), B, H1, W1, CT, L0, s))
        gin = mk(grad)
        gs = [mk(torch.zeros_like(t)) for t in srcs]
        _lib.check(lib.sepcorr_assemble_backward_multi(gin.data_ptr(), arr(gs), ch, li, n, B, H1, W1, CT, L0, s))
        torch.cuda.synchronize()
        return [dst] + gs

    for x, y in zip(run(True), run(False)):
        assert torch.equal(x, y), "16-byte and 4-byte accesses of the assemble kernels disagree"
