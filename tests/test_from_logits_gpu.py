"""GPU parity of the attention compression taken straight from the logits (softmax inside the operator), through the
C ABI: values, saved row statistics, gradients of features and logits, against the oracle's softmax + compression
with torch autograd (core/corr.py:441-448, libs/MemorySaver/functions/MemorySaver.py:107-177)."""
import pytest
import torch

from oracle import oracle as O
from tests._util import assert_close, op_inputs

pytestmark = pytest.mark.gpu

SHAPES = [
    (1, 1, 1, 1, 1, 1),
    (2, 5, 7, 5, 7, 16),
    (1, 9, 13, 4, 6, 117),
    (1, 12, 40, 12, 40, 256),
    (1, 8, 150, 8, 150, 64),
    (2, 24, 32, 24, 32, 256),
    (1, 16, 48, 16, 48, 300),
    (8, 32, 48, 16, 24, 32),
    (1, 4, 40, 3, 300, 32),       # two column passes
    (1, 3, 11, 2, 301, 7),
    (1, 20, 36, 140, 36, 64),     # rows of out_u too long to be collected in LDS
]


def _ms():
    from separableflowthesis_amd import MemorySaver
    return MemorySaver


def _logits(B, H1, W1, H2, W2, K, g, scale=2.0):
    return (torch.randn(B, H1, W1, K, W2, generator=g) * scale).contiguous(), (torch.randn(B, H1, W1, K, H2, generator=g) * scale).contiguous()


@pytest.mark.parametrize("K", [1, 2, 4, 5])
@pytest.mark.parametrize("shape", SHAPES)
def test_forward_backward_from_logits(device, shape, K):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(*shape, seed=51)
    z_u, z_v = _logits(B, H1, W1, H2, W2, K, g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    ref_in = [t.double().requires_grad_() for t in (f1, f2, z_u, z_v)]
    rcu, rcv = O.compression_from_logits(*ref_in)
    ((rcu * g_cu.double()).sum() + (rcv * g_cv.double()).sum()).backward()
    d = lambda t: t.to(device)
    ms = _ms()
    cu, cv, st_u, st_v = ms.compression_forward_from_logits(d(f1), d(f2), d(z_u), d(z_v))
    assert_close(cu, rcu, "compression_output_u")
    assert_close(cv, rcv, "compression_output_v")
    for st, z in ((st_u, z_u), (st_v, z_v)):
        m = z.double().max(-1)[0]
        assert_close(st[..., 0], m, "row max")
        assert_close(st[..., 1], (z.double() - m.unsqueeze(-1)).exp().sum(-1), "row sum of exp")
    d1, d2, dz_u, dz_v = ms.compression_backward_from_logits(d(f1), d(f2), d(z_u), d(z_v), st_u, st_v, cu, cv, d(g_cu), d(g_cv))
    for got, r, n in zip((d1, d2, dz_u, dz_v), ref_in, ("d_f1", "d_f2", "d_logits_u", "d_logits_v")):
        assert_close(got, r.grad, n, scale_atol=True)
    # without the feature gradients: the same logit gradients, bit for bit
    n1, n2, ez_u, ez_v = ms.compression_backward_from_logits(d(f1), d(f2), d(z_u), d(z_v), st_u, st_v, cu, cv, d(g_cu), d(g_cv),
                                                             need_features=False)
    assert n1 is None and n2 is None and torch.equal(ez_u, dz_u) and torch.equal(ez_v, dz_v)
    # statistics handed in (as the attention producer does) give the same outputs
    cu2, cv2, _, _ = ms.compression_forward_from_logits(d(f1), d(f2), d(z_u), d(z_v), st_u, st_v)
    assert torch.equal(cu2, cu) and torch.equal(cv2, cv)


def test_extreme_logits_stay_finite(device):
    B, H1, W1, H2, W2, C, K = 1, 6, 10, 6, 40, 32, 2
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=3)
    z_u, z_v = _logits(B, H1, W1, H2, W2, K, g, scale=60.0)   # exp of the raw logits would overflow fp32
    z_u[0, 0, 0, 0] = 0.0                                      # and one constant row
    d = lambda t: t.to(device)
    cu, cv, st_u, st_v = _ms().compression_forward_from_logits(d(f1), d(f2), d(z_u), d(z_v))
    rcu, rcv = O.compression_from_logits(f1.double(), f2.double(), z_u.double(), z_v.double())
    assert torch.isfinite(cu).all() and torch.isfinite(cv).all()
    assert_close(cu, rcu, "compression_output_u")
    assert_close(cv, rcv, "compression_output_v")


def test_autograd_function_and_attention_logits(device):
    """ComputeSelfCompressionFromLogitsFunction and AttentionLogitsFunction through torch autograd against the chain
    Conv3d -> softmax -> compression on the 4D volume, with gradients down to the Conv3d parameters."""
    from separableflowthesis_amd.functions import AttentionLogitsFunction, ComputeSelfCompressionFromLogitsFunction
    B, H1, W1, H2, W2, C, K = 2, 10, 14, 10, 14, 64, 3
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=77)
    sep_v = torch.randn(B, H1, W1, 2, W2, generator=g)
    sep_u = torch.randn(B, H1, W1, 2, H2, generator=g)
    w1, w2 = torch.randn(K, 2, 3, 3, 3, generator=g) * 0.3, torch.randn(K, 2, 3, 3, 3, generator=g) * 0.3
    b1, b2 = torch.randn(K, generator=g), torch.randn(K, generator=g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    leaves = (f1, f2, sep_v, sep_u, w1, b1, w2, b2)
    r = [t.double().requires_grad_() for t in leaves]
    rcu, rcv = O.compression_from_logits(r[0], r[1], O.attention_logits(r[2], r[4], r[5]), O.attention_logits(r[3], r[6], r[7]))
    ((rcu * g_cu.double()).sum() + (rcv * g_cv.double()).sum()).backward()
    x = [t.to(device).requires_grad_() for t in leaves]
    z_u, st_u = AttentionLogitsFunction.apply(x[2], x[4], x[5])
    z_v, _ = AttentionLogitsFunction.apply(x[3], x[6], x[7])
    assert_close(z_u, O.attention_logits(r[2], r[4], r[5]), "logits_u")
    assert not st_u.requires_grad
    # statistics from the producer for one volume, computed by the operator for the other: same thing
    cu, cv = ComputeSelfCompressionFromLogitsFunction.apply(x[0], x[1], z_u, z_v)
    cu2, cv2 = ComputeSelfCompressionFromLogitsFunction.apply(x[0], x[1], z_u, z_v, st_u, None)
    assert torch.equal(cu, cu2) and torch.equal(cv, cv2)
    assert_close(cu, rcu, "compression_output_u")
    assert_close(cv, rcv, "compression_output_v")
    ((cu * g_cu.to(device)).sum() + (cv * g_cv.to(device)).sum()).backward()
    for got, ref, n in zip(x, r, ("d_f1", "d_f2", "d_sep_v", "d_sep_u", "d_w1", "d_b1", "d_w2", "d_b2")):
        assert_close(got.grad, ref.grad, n, scale_atol=True)
    # the producer's statistics are those of its logits
    from separableflowthesis_amd import MemorySaver
    z, st = MemorySaver.attention_logits_forward(x[2].detach(), x[4].detach(), x[5].detach())
    m = z.double().max(-1)[0]
    assert_close(st[..., 0], m, "producer row max")
    assert_close(st[..., 1], (z.double() - m.unsqueeze(-1)).exp().sum(-1), "producer row sum of exp")
    assert_close(MemorySaver.softmax_from_stats(z, st), z.double().softmax(-1), "softmax from statistics")


@pytest.mark.parametrize("B", [1, 2], ids=["cfg3", "cfg4"])
def test_from_logits_at_benchmark_sizes(device, B):
    C, H, W, K = 256, 55, 128, 4
    _, _, f1, f2 = O.make_inputs(B, H, W, C, seed=1234)
    g = torch.Generator().manual_seed(99)
    z_u, z_v = _logits(B, H, W, H, W, K, g)
    g_cu, g_cv = torch.randn(B, H, W, K, H, generator=g), torch.randn(B, H, W, K, W, generator=g)
    d = lambda t: t.to(device)
    ms = _ms()
    cu, cv, st_u, st_v = ms.compression_forward_from_logits(d(f1), d(f2), d(z_u), d(z_v))
    d1, d2, dz_u, dz_v = ms.compression_backward_from_logits(d(f1), d(f2), d(z_u), d(z_v), st_u, st_v, cu, cv, d(g_cu), d(g_cv))
    for b in range(B):
        sl = slice(b, b + 1)
        r = [t[sl].double().requires_grad_() for t in (f1, f2, z_u, z_v)]
        rcu, rcv = O.compression_from_logits(*r)
        ((rcu * g_cu[sl].double()).sum() + (rcv * g_cv[sl].double()).sum()).backward()
        assert_close(cu[sl], rcu, "compression_output_u")
        assert_close(cv[sl], rcv, "compression_output_v")
        for got, ref, n in zip((d1, d2, dz_u, dz_v), r, ("d_f1", "d_f2", "d_logits_u", "d_logits_v")):
            assert_close(got[sl], ref.grad, n, scale_atol=True)
