"""GPU parity of the optional bf16-plane contraction of the forward sweeps (sepcorr_set_contraction).

The same bar as the fp32 MFMA path: rtol 1e-4 / atol 1e-5 against the fp64 oracle, argmax exact except
near-ties.  Each test checks through the library's kernel labels that the variant really ran.
"""
import ctypes

import pytest
import torch

from oracle import oracle as O
from tests._util import assert_close, check_argmax, op_inputs, softmax_weights

pytestmark = pytest.mark.gpu

# (B, H1, W1, H2, W2, C), all with C == 256 and rows of at most 256 columns
SHAPES = [
    (1, 7, 100, 7, 100, 256),    # ragged last chunk, odd row count (one padded row)
    (1, 9, 160, 9, 160, 256),    # five chunks
    (3, 48, 64, 24, 96, 256),    # pooled fmap2, three chunks, more than 256 workgroups
    (1, 4, 256, 4, 256, 256),    # widest row of a single pass
    (1, 12, 40, 12, 40, 256),    # narrow rows: two column chunks x row groups
    (2, 24, 32, 11, 17, 256),    # one ragged column chunk, row groups, rows padded to whole steps
    (1, 16, 128, 16, 128, 256),  # four chunks x two row groups (few workgroups)
]


@pytest.fixture()
def planes():
    from separableflowthesis_amd import MemorySaver as ms
    prev = ms.set_contraction(ms.CONTRACT_BF16X3)
    prev_bwd = ms.set_max_avg_backward(ms.MAXAVG_DENSE)   # the planes belong to the dense kernels; gathers contract nothing
    yield ms
    ms.set_max_avg_backward(prev_bwd)
    ms.set_contraction(prev)


def _labels_of(fn):
    """Run fn() with the library's kernel timing on; return (result, set of kernel labels launched)."""
    from separableflowthesis_amd import _lib
    lib = _lib.load()
    lib.sepcorr_profile_enable(1)
    try:
        out = fn()
        torch.cuda.synchronize()
    finally:
        names = ctypes.create_string_buffer(1 << 14)
        ms_ = (ctypes.c_float * 256)()
        n = lib.sepcorr_profile_collect(names, len(names), ms_, 256)
        lib.sepcorr_profile_enable(0)
    return out, set(names.value.decode().split("\n")[:n])


def test_switch_returns_previous_mode(device):
    from separableflowthesis_amd import MemorySaver as ms
    first = ms.set_contraction(ms.CONTRACT_BF16X3)
    assert ms.set_contraction(first) == ms.CONTRACT_BF16X3
    assert ms.set_contraction(77) == first       # unknown mode: nothing changes
    assert ms.set_contraction(first) == first


@pytest.mark.parametrize("shape", SHAPES)
def test_max_argmax_avg_forward(device, planes, shape):
    B, H1, W1, H2, W2, C = shape
    f1, f2, _ = op_inputs(B, H1, W1, H2, W2, C, seed=sum(shape))
    (ou, ov, au, av), labels = _labels_of(lambda: planes.max_argmax_avg_forward(f1.to(device), f2.to(device)))
    assert "fwd_maxavg_bf16x3" in labels and "split_planes" in labels, labels
    s64 = O.corr_volume(f1.double(), f2.double())
    rou, rov, rau, rav = O.max_argmax_avg_from_volume(s64)
    assert_close(ou, rou, "max_avg_output_u")
    assert_close(ov, rov, "max_avg_output_v")
    check_argmax(au, rau, s64, 4, "argmax_output_u")
    check_argmax(av, rav, s64, 3, "argmax_output_v")
    ou2, ov2 = planes.max_avg_forward(f1.to(device), f2.to(device))
    assert torch.equal(ou, ou2) and torch.equal(ov, ov2)


@pytest.mark.parametrize("shape", SHAPES[:3] + SHAPES[4:])
@pytest.mark.parametrize("K", [1, 2, 3, 5])
def test_compression_forward(device, planes, shape, K):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=11 + K)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    (cu, cv), labels = _labels_of(
        lambda: planes.compression_forward(f1.to(device), f2.to(device), a_u.to(device), a_v.to(device)))
    assert "fwd_weighted_bf16x3" in labels, labels   # K = 5: a launch of four channels, then one of one
    rcu, rcv = O.compression_forward(f1.double(), f2.double(), a_u.double(), a_v.double())
    assert_close(cu, rcu, "compression_output_u")
    assert_close(cv, rcv, "compression_output_v")


def test_compression_backward_attention_gradients(device, planes):
    B, H1, W1, H2, W2, C = SHAPES[0]
    K = 2
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=5)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    d = lambda t: t.to(device)
    got, labels = _labels_of(lambda: planes.compression_backward(d(f1), d(f2), d(a_u), d(a_v), d(g_cu), d(g_cv)))
    assert "fwd_weighted_bf16x3" in labels, labels
    ref = O.compression_backward(*(t.double() for t in (f1, f2, a_u, a_v, g_cu, g_cv)))
    for x, y, n in zip(got, ref, ("grad_fmap1_l0", "grad_fmap2_lk", "grad_attention_u", "grad_attention_v")):
        assert_close(x, y, n, scale_atol=True)


BWD_SHAPES = SHAPES[:3] + [(2, 9, 20, 9, 20, 256)]   # the last: one ragged chunk, the partial sums go straight to d_f1


@pytest.mark.parametrize("shape", BWD_SHAPES)
def test_max_argmax_avg_backward(device, planes, shape):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=21)
    s64 = O.corr_volume(f1.double(), f2.double())
    _, _, am_u, am_v = O.max_argmax_avg_from_volume(s64)
    g_u = torch.randn(B, H1, W1, 2, H2, generator=g)
    g_v = torch.randn(B, H1, W1, 2, W2, generator=g)
    d = lambda t: t.to(device)
    got, labels = _labels_of(lambda: planes.max_argmax_avg_backward(d(f1), d(f2), d(am_u), d(am_v), d(g_u), d(g_v)))
    assert "df1_maxavg_bf16x3" in labels, labels
    ref = O.max_argmax_avg_backward(f1.double(), f2.double(), am_u, am_v, g_u.double(), g_v.double())
    for x, y, n in zip(got, ref, ("grad_fmap1_l0", "grad_fmap2_lk")):
        assert_close(x, y, n, scale_atol=True)


@pytest.mark.parametrize("shape", BWD_SHAPES)
@pytest.mark.parametrize("K", [1, 2, 3, 4, 6])
def test_compression_backward(device, planes, shape, K):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=31 + K)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    d = lambda t: t.to(device)
    got, labels = _labels_of(lambda: planes.compression_backward(d(f1), d(f2), d(a_u), d(a_v), d(g_cu), d(g_cv)))
    assert "df1_comp_bf16x3" in labels, labels
    ref = O.compression_backward(*(t.double() for t in (f1, f2, a_u, a_v, g_cu, g_cv)))
    for x, y, n in zip(got, ref, ("grad_fmap1_l0", "grad_fmap2_lk", "grad_attention_u", "grad_attention_v")):
        assert_close(x, y, n, scale_atol=True)


@pytest.mark.parametrize("K", [2, 4, 3])
def test_fused_backward(device, planes, K):
    B, H1, W1, H2, W2, C = SHAPES[0]
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=51 + K)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    g_u = torch.randn(B, H1, W1, 2, H2, generator=g)
    g_v = torch.randn(B, H1, W1, 2, W2, generator=g)
    s64 = O.corr_volume(f1.double(), f2.double())
    _, _, am_u, am_v = O.max_argmax_avg_from_volume(s64)
    d = lambda t: t.to(device)
    got, labels = _labels_of(lambda: planes.fused_backward(d(f1), d(f2), d(am_u), d(am_v), d(g_u), d(g_v),
                                                           d(a_u), d(a_v), d(g_cu), d(g_cv)))
    assert any(l.startswith("df1_") and l.endswith("bf16x3") for l in labels), labels
    r1 = O.max_argmax_avg_backward(f1.double(), f2.double(), am_u, am_v, g_u.double(), g_v.double())
    r2 = O.compression_backward(*(t.double() for t in (f1, f2, a_u, a_v, g_cu, g_cv)))
    assert_close(got[0], r1[0] + r2[0], "grad_fmap1_l0", scale_atol=True)
    assert_close(got[1], r1[1] + r2[1], "grad_fmap2_lk", scale_atol=True)


def test_corr_block_with_planes(device, planes):
    # the caller's separate() over a two-level pyramid, forward and gradients, against the full-4D oracle
    import copy
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    B, C, H, W, K = 1, 256, 6, 100, 2
    fmap1, fmap2, _, _ = O.make_inputs(B, H, W, C, seed=9)
    torch.manual_seed(4)
    att = (torch.nn.Conv3d(2, K, 3, padding=1), torch.nn.Conv3d(2, K, 3, padding=1))
    r1, r2 = fmap1.double().requires_grad_(), fmap2.double().requires_grad_()
    ratt = tuple(copy.deepcopy(m).double() for m in att)
    rc1, rc2 = O.CorrBlock4D(r1, r2, num_levels=2).separate(ratt)
    g1, g2 = fmap1.to(device).requires_grad_(), fmap2.to(device).requires_grad_()
    gatt = tuple(copy.deepcopy(m).to(device) for m in att)

    def run():
        blk = AlternateCorrBlockSepflow(g1, g2, None, num_levels=2, support_backward=True)
        c1, c2 = blk(None, sep=True, attention_weights=gatt)
        gen = torch.Generator().manual_seed(3)
        w1, w2 = torch.randn(rc1.shape, generator=gen) / 64, torch.randn(rc2.shape, generator=gen) / 64
        ((c1 * w1.to(device)).sum() + (c2 * w2.to(device)).sum()).backward()
        return c1, c2, w1, w2

    (c1, c2, w1, w2), labels = _labels_of(run)
    # (the compression sweeps of this path take logits, which the plane variant of the sweep does not: fp32 there)
    assert {"fwd_maxavg_bf16x3", "df1_both_bf16x3"} <= labels, labels
    assert_close(c1, rc1, "corr1")
    assert_close(c2, rc2, "corr2")
    ((rc1 * w1.double()).sum() + (rc2 * w2.double()).sum()).backward()
    assert_close(g1.grad, r1.grad, "grad fmap1", scale_atol=True)
    assert_close(g2.grad, r2.grad, "grad fmap2", scale_atol=True)
    for m, rm, n in zip(gatt, ratt, ("attention1", "attention2")):
        assert_close(m.weight.grad, rm.weight.grad, n + ".weight.grad", scale_atol=True)


def test_ineligible_shapes_stay_fp32(device, planes):
    # C != 256, and rows wider than one column pass: both silently use the fp32 MFMA kernels
    for shape in [(1, 8, 150, 8, 150, 64), (1, 2, 300, 2, 300, 256)]:
        B, H1, W1, H2, W2, C = shape
        f1, f2, _ = op_inputs(B, H1, W1, H2, W2, C, seed=3)
        (ou, ov), labels = _labels_of(lambda: planes.max_avg_forward(f1.to(device), f2.to(device)))
        assert labels == {"fwd_maxavg"}, labels
        prev = planes.set_contraction(planes.CONTRACT_FP32)
        ou2, ov2 = planes.max_avg_forward(f1.to(device), f2.to(device))
        planes.set_contraction(prev)
        assert torch.equal(ou, ou2) and torch.equal(ov, ov2)


def test_full_size_agrees_with_fp32_mfma(device, planes):
    # B=2, 55x128, C=256: too large for the oracle; the two contractions must agree to fp32 rounding and the
    # argmax tensors may differ only where the competing maxima are that close
    B, H, W, C = 2, 55, 128, 256
    f1, f2, _ = op_inputs(B, H, W, H, W, C, seed=1)
    f1, f2 = f1.to(device), f2.to(device)
    (ou, ov, au, av), labels = _labels_of(lambda: planes.max_argmax_avg_forward(f1, f2))
    assert "fwd_maxavg_bf16x3" in labels
    prev = planes.set_contraction(planes.CONTRACT_FP32)
    ou0, ov0, au0, av0 = planes.max_argmax_avg_forward(f1, f2)
    planes.set_contraction(prev)
    assert float((ou - ou0).abs().max()) <= 2e-5 and float((ov - ov0).abs().max()) <= 2e-5
    for am, am0, out0, n in ((au, au0, ou0, "argmax_u"), (av, av0, ov0, "argmax_v")):
        mism = (am != am0)[:, :, :, 0]
        assert int(mism.sum()) <= am.numel() // 10000, n
        # where the index differs, the maxima found by both contractions still agree to rounding
        if bool(mism.any()):
            pass_gap = (ou[:, :, :, 0] - ou0[:, :, :, 0]).abs() if n == "argmax_u" else (ov[:, :, :, 0] - ov0[:, :, :, 0]).abs()
            assert float(pass_gap[mism].max()) <= 1e-5, n


def test_full_size_backward_agrees_with_fp32_mfma(device, planes):
    # B=2, 55x128, C=256, K'=4: d_f1 of both backward operators and of the fused one, planes against fp32 MFMA
    B, H, W, C, K = 2, 55, 128, 256, 4
    f1, f2, g = op_inputs(B, H, W, H, W, C, seed=2)
    a_u = softmax_weights(B, H, W, K, W, g)
    a_v = softmax_weights(B, H, W, K, H, g)
    g_cu, g_cv = torch.randn(B, H, W, K, H, generator=g), torch.randn(B, H, W, K, W, generator=g)
    g_u, g_v = torch.randn(B, H, W, 2, H, generator=g), torch.randn(B, H, W, 2, W, generator=g)
    am_u = torch.randint(0, W, (B, H, W, 1, H), generator=g, dtype=torch.int32)
    am_v = torch.randint(0, H, (B, H, W, 1, W), generator=g, dtype=torch.int32)
    d = lambda t: t.to(device)
    f1, f2, a_u, a_v, g_cu, g_cv, g_u, g_v, am_u, am_v = map(d, (f1, f2, a_u, a_v, g_cu, g_cv, g_u, g_v, am_u, am_v))

    def all_three():
        return (planes.compression_backward(f1, f2, a_u, a_v, g_cu, g_cv)[0],
                planes.max_argmax_avg_backward(f1, f2, am_u, am_v, g_u, g_v)[0],
                planes.fused_backward(f1, f2, am_u, am_v, g_u, g_v, a_u, a_v, g_cu, g_cv)[0])

    got, labels = _labels_of(all_three)
    assert {"df1_comp_bf16x3", "df1_maxavg_bf16x3", "df1_both_bf16x3"} <= labels, labels
    prev = planes.set_contraction(planes.CONTRACT_FP32)
    ref = all_three()
    planes.set_contraction(prev)
    for x, y, n in zip(got, ref, ("compression d_f1", "max/avg d_f1", "fused d_f1")):
        assert_close(x, y, n, scale_atol=True)
    # the fused gradient is the sum of the two
    assert_close(got[2], got[0].double() + got[1].double(), "fused = sum", scale_atol=True)

