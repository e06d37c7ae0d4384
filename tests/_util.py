"""Helpers shared by the parity tests."""
import torch

from oracle import oracle as O

RTOL = 1e-4   # tolerance stated for this path: rtol 1e-4 / atol 1e-5 in fp32
ATOL = 1e-5


def assert_close(got, ref, name, scale_atol=False):
    """|got-ref| <= atol + rtol*|ref| element-wise, ref computed in fp64.

    For forward outputs (O(1) values) atol is the plain 1e-5.  Gradients of N(0,1) upstream grads
    are sums of thousands of O(1) products: their magnitude is O(100) and the fp32 rounding of
    any summation order, the reference's CPU path included, is O(1e-5) absolute, so for those
    tensors (scale_atol=True) atol is taken relative to the tensor's RMS: 1e-5*max(1, rms(ref)).
    """
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    atol = ATOL
    if scale_atol:
        atol = ATOL * max(1.0, float(ref.pow(2).mean().sqrt()))
    err = (got - ref).abs()
    bound = atol + RTOL * ref.abs()
    bad = err > bound
    assert not bool(bad.any()), (
        f"{name}: {int(bad.sum())} of {bad.numel()} elements outside rtol={RTOL} atol={atol:.3g}; "
        f"max abs err {float(err.max()):.3g}, max err/bound {float((err / bound).max()):.3g}")


def check_argmax(am_gpu, am_ref, s64, axis, name, eps=2e-6):
    """Indices must be equal except where the two candidates are tied to within fp32 rounding.

    s64 is the fp64 volume (B,H1,W1,H2,W2); axis=4 for argmax_u (index into v), 3 for argmax_v.
    Returns the number of near-tie mismatches (reported, not hidden).
    """
    a = am_gpu[:, :, :, 0].long().cpu()
    r = am_ref[:, :, :, 0].long().cpu()
    L = s64.shape[axis]
    assert int(a.min()) >= 0 and int(a.max()) < L, f"{name}: index out of range"
    mism = a != r
    n = int(mism.sum())
    if n:
        va = torch.gather(s64, axis, a.unsqueeze(axis)).squeeze(axis)
        vr = torch.gather(s64, axis, r.unsqueeze(axis)).squeeze(axis)
        gap = (va - vr).abs()[mism]
        tol = eps * torch.maximum(vr.abs()[mism], torch.ones_like(gap))
        assert bool((gap <= tol).all()), (
            f"{name}: {int((gap > tol).sum())} argmax mismatches are not near-ties (max gap {float(gap.max()):.3g})")
    return n


def op_inputs(B, H1, W1, H2, W2, C, seed, scale=True):
    g = torch.Generator().manual_seed(seed)
    f1 = torch.randn(B, H1, W1, C, generator=g)
    f2 = torch.randn(B, H2, W2, C, generator=g)
    if scale:
        f1 = f1 / torch.sqrt(torch.tensor(float(C)))
    return f1.contiguous(), f2.contiguous(), g


def softmax_weights(B, H1, W1, K, L, g):
    return torch.randn(B, H1, W1, K, L, generator=g).softmax(dim=-1).contiguous()
