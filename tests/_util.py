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


def chain_ratio(chain):
    """Bound for error_report's ratio where the GPU adds `chain` products one after the other in one fp32 MFMA
    accumulator while the CPU's sgemm adds blocks of a few hundred (taken as 256) and then the block sums: rounding
    error grows with the square root of the length of a sequential sum, so the ratio of the two errors is expected
    near sqrt(chain / 256); 25 % on top, and never below the default 2."""
    return max(2.0, 1.25 * (chain / 256.0) ** 0.5)


def error_report(got, ref64, cpu32, name, max_ratio=2.0):
    """Gradient parity made explicit: the error of the GPU result against fp64 next to the error the fp32 CPU
    run of the same full-4D path makes against fp64.

    Asserts the usual bound (assert_close with the RMS-scaled absolute term) and, so that this bound is not
    just asserted to be fair, that the GPU's RMS error is at most `max_ratio` times the fp32 CPU path's.
    Prints both errors and how many elements fall outside the plain rtol 1e-4 / atol 1e-5.
    """
    g = got.detach().double().cpu()
    r = ref64.detach().double().cpu()
    c = cpu32.detach().double().cpu()
    eg, ec = (g - r).abs(), (c - r).abs()
    plain = ATOL + RTOL * r.abs()
    rms = lambda e: float(e.pow(2).mean().sqrt())
    rep = {"name": name, "rms_ref": rms(r), "gpu_rms_err": rms(eg), "cpu32_rms_err": rms(ec),
           "gpu_max_err": float(eg.max()), "cpu32_max_err": float(ec.max()),
           "gpu_outside_plain_tol": int((eg > plain).sum()), "cpu32_outside_plain_tol": int((ec > plain).sum()),
           "numel": r.numel()}
    print("parity " + " ".join(f"{k}={v:.4g}" if isinstance(v, float) else f"{k}={v}" for k, v in rep.items()), flush=True)
    assert_close(got, ref64, name, scale_atol=True)
    floor = 1e-7 * max(1.0, rep["rms_ref"])   # both exact to the last bit or so: nothing to compare
    assert rep["gpu_rms_err"] <= max_ratio * max(rep["cpu32_rms_err"], floor), (
        f"{name}: GPU rms error {rep['gpu_rms_err']:.3g} exceeds {max_ratio} x the fp32 CPU path's {rep['cpu32_rms_err']:.3g}")
    return rep


def native_argmax_levels(fmap1, fmap2, device, num_levels=4):
    """The argmax tensors the native block's forward pass produces at every pyramid level, for NCHW fmaps as the
    caller holds them: same inputs, same kernels as AlternateCorrBlockSepflow.separate (core/corr.py:416-425).
    Returns [(argmax_u, argmax_v)] on the CPU."""
    import torch.nn.functional as F
    from separableflowthesis_amd import MemorySaver
    x1, x2 = fmap1.to(device), fmap2.to(device)
    f1 = x1.permute(0, 2, 3, 1).contiguous() / torch.sqrt(torch.tensor(x1.shape[1]).float())
    out = []
    for _ in range(num_levels):
        _, _, am_u, am_v = MemorySaver.max_argmax_avg_forward(f1, x2.permute(0, 2, 3, 1).contiguous())
        out.append((am_u.cpu(), am_v.cpu()))
        x2 = F.avg_pool2d(x2, 2, stride=2)
    return out


def check_argmax_levels(argmax, block64, name):
    """Every index of `argmax` (from native_argmax_levels) against the fp64 pyramid of an oracle CorrBlock4D: equal to
    the oracle's argmax except at near-ties.  Returns the number of near-tie mismatches over all levels."""
    B, h1, w1, _, _ = block64.shape
    n = 0
    for lvl, (corr, (am_u, am_v)) in enumerate(zip(block64.pyramid, argmax)):
        s64 = corr.detach().reshape(B, h1, w1, corr.shape[2], corr.shape[3])
        _, _, rau, rav = O.max_argmax_avg_from_volume(s64)
        n += check_argmax(am_u, rau, s64, 4, f"{name}: level {lvl} argmax_u")
        n += check_argmax(am_v, rav, s64, 3, f"{name}: level {lvl} argmax_v")
    return n
