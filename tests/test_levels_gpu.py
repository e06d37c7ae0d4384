"""GPU parity of the entry points that take several pyramid levels per call (one launch for all levels where the shapes
allow, level by level inside the call otherwise): values against the fp64 oracle per level, argmax exact up to near-ties,
logit gradients against autograd through softmax + compression."""
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O
from tests._util import assert_close, check_argmax

pytestmark = pytest.mark.gpu

# (B, H, W, C, levels): one-launch shapes (rows of 1, 2 or 4 chunks of 32 columns) and shapes that fall back
CASES = [
    (2, 24, 64, 64, 4),      # 64, 32, 16, 8 columns
    (1, 55, 128, 256, 4),    # the benchmark image: 128, 64, 32, 16
    (2, 16, 32, 32, 3),
    (1, 20, 40, 32, 3),      # 40 columns = 2 chunks, 20 = 1, 10 = 1
    (1, 12, 96, 32, 2),      # 96 columns = 3 chunks: level by level
    (1, 8, 150, 36, 2),      # C not a multiple of 32, wide rows: level by level
    (3, 9, 16, 64, 1),       # a single level
]


def _levels(B, H, W, C, nlev, seed):
    g = torch.Generator().manual_seed(seed)
    f1 = torch.randn(B, H, W, C, generator=g) / C ** 0.5
    fmap2 = torch.randn(B, C, H, W, generator=g)
    lv = []
    for _ in range(nlev):
        lv.append(fmap2.permute(0, 2, 3, 1).contiguous())
        fmap2 = F.avg_pool2d(fmap2, 2, stride=2)
    return f1, lv, g


@pytest.mark.parametrize("case", CASES)
def test_max_argmax_avg_forward_levels(device, case):
    from separableflowthesis_amd import MemorySaver as ms
    B, H, W, C, nlev = case
    f1, lv, _ = _levels(*case, seed=5)
    got = ms.max_argmax_avg_forward_levels(f1.to(device), [t.to(device) for t in lv])
    assert len(got) == nlev
    for l, (f2, (ou, ov, au, av)) in enumerate(zip(lv, got)):
        s64 = O.corr_volume(f1.double(), f2.double())
        rou, rov, rau, rav = O.max_argmax_avg_from_volume(s64)
        assert_close(ou, rou, f"level {l} max_avg_output_u")
        assert_close(ov, rov, f"level {l} max_avg_output_v")
        check_argmax(au, rau, s64, 4, f"level {l} argmax_output_u")
        check_argmax(av, rav, s64, 3, f"level {l} argmax_output_v")


@pytest.mark.parametrize("K", [2, 4, 5])
@pytest.mark.parametrize("case", CASES)
def test_compression_from_logits_levels(device, case, K):
    from separableflowthesis_amd import MemorySaver as ms
    B, H, W, C, nlev = case
    f1, lv, g = _levels(*case, seed=6)
    z_u = [(torch.randn(B, H, W, K, t.shape[2], generator=g) * 2).contiguous() for t in lv]
    z_v = [(torch.randn(B, H, W, K, t.shape[1], generator=g) * 2).contiguous() for t in lv]
    g_cu = [torch.randn(B, H, W, K, t.shape[1], generator=g) for t in lv]
    g_cv = [torch.randn(B, H, W, K, t.shape[2], generator=g) for t in lv]
    d = lambda ts: [t.to(device) for t in ts]
    dz_u, dz_v = d(z_u), d(z_v)
    st_u = [torch.empty(B, H, W, K, 2, device=device) for _ in lv]
    st_v = [torch.empty(B, H, W, K, 2, device=device) for _ in lv]
    for l in range(nlev):   # row statistics as the attention producer would hand them over
        ms.softmax_from_stats  # (the helper below computes the statistics; the weights are not needed)
        from separableflowthesis_amd import _lib
        lib = _lib.load()
        for z, st in ((dz_u[l], st_u[l]), (dz_v[l], st_v[l])):
            _lib.check(lib.sepcorr_softmax_rows(z.data_ptr(), st.data_ptr(), 0, None, z.numel() // z.shape[-1], z.shape[-1],
                                                torch.cuda.current_stream().cuda_stream))
    comp = ms.compression_forward_from_logits_levels(f1.to(device), d(lv), dz_u, dz_v, st_u, st_v)
    grads = ms.compression_logit_gradients_levels(f1.to(device), d(lv), dz_u, dz_v, st_u, st_v, [c[0] for c in comp],
                                                  [c[1] for c in comp], d(g_cu), d(g_cv))
    for l in range(nlev):
        r = [t.double().requires_grad_() for t in (z_u[l], z_v[l])]
        rcu, rcv = O.compression_from_logits(f1.double(), lv[l].double(), *r)
        ((rcu * g_cu[l].double()).sum() + (rcv * g_cv[l].double()).sum()).backward()
        assert_close(comp[l][0], rcu, f"level {l} compression_output_u")
        assert_close(comp[l][1], rcv, f"level {l} compression_output_v")
        assert_close(grads[l][0], r[0].grad, f"level {l} d_logits_u", scale_atol=True)
        assert_close(grads[l][1], r[1].grad, f"level {l} d_logits_v", scale_atol=True)


@pytest.mark.parametrize("B,H1,W1,K,Ls", [
    (2, 55, 128, 4, (128, 64, 32, 16)),     # attention1 over the four levels of the headline size
    (2, 55, 128, 4, (55, 27, 13, 6)),       # attention2
    (1, 9, 21, 2, (70, 7)),                 # rows of more than 64 and of fewer than 16 entries in one call
    (1, 6, 10, 5, (300, 20, 5)),            # the long-row kernel beside the short ones, K = 5
])
def test_attention_modules_over_several_levels(device, B, H1, W1, K, Ls):
    """One attention module on the max/avg volumes of several levels in shared launches = the single-level calls:
    logits, statistics and input gradients bit for bit (same kernels, same order of operations), weight and bias
    gradients as the sum over the levels; the upstream gradient of the volumes is added in the same pass."""
    from separableflowthesis_amd import MemorySaver as ms
    g = torch.Generator().manual_seed(sum(Ls) + K)
    seps = [torch.randn(B, H1, W1, 2, L, generator=g).to(device) for L in Ls]
    w = (torch.randn(K, 2, 3, 3, 3, generator=g) / 4).to(device)
    b = torch.randn(K, generator=g).to(device)
    dzs = [torch.randn(B, H1, W1, K, L, generator=g).to(device) for L in Ls]
    inits = [torch.randn(B, H1, W1, 2, L, generator=g).to(device) for L in Ls]

    zs, sts = ms.attention_logits_forward_levels(seps, w, b)
    d_seps, d_w, d_b = ms.attention_logits_backward_levels(seps, w, dzs, inits)
    d_seps0, d_w0, none_b = ms.attention_logits_backward_levels(seps, w, dzs, None, need_bias=False)
    assert none_b is None
    sum_w, sum_b = torch.zeros_like(w, dtype=torch.float64), torch.zeros_like(b, dtype=torch.float64)
    for l, L in enumerate(Ls):
        z1, st1 = ms.attention_logits_forward(seps[l], w, b)
        assert torch.equal(zs[l], z1) and torch.equal(sts[l], st1)
        ds1, dw1, db1 = ms.attention_logits_backward(seps[l], w, dzs[l])
        assert torch.equal(d_seps0[l], ds1)
        assert torch.equal(d_seps[l], ds1 + inits[l])
        sum_w += dw1.double()
        sum_b += db1.double()
    torch.testing.assert_close(d_w.double(), sum_w, rtol=1e-5, atol=1e-5 * float(sum_w.abs().max()))
    torch.testing.assert_close(d_w0.double(), sum_w, rtol=1e-5, atol=1e-5 * float(sum_w.abs().max()))
    torch.testing.assert_close(d_b.double(), sum_b, rtol=1e-5, atol=1e-5 * float(sum_b.abs().max()))


def test_attention_levels_argument_errors(device):
    from separableflowthesis_amd import MemorySaver as ms
    w = torch.randn(2, 2, 3, 3, 3, device=device)
    seps = [torch.randn(1, 4, 4, 2, 8, device=device) for _ in range(5)]
    with pytest.raises(RuntimeError):
        ms.attention_logits_forward_levels(seps, w, None)                      # more than 4 levels
    with pytest.raises(RuntimeError):
        ms.attention_logits_forward_levels([seps[0], torch.randn(1, 4, 5, 2, 8, device=device)], w, None)
    with pytest.raises(RuntimeError):
        ms.attention_logits_backward_levels(seps[:2], w, [torch.randn(1, 4, 4, 2, 8, device=device)] * 2,
                                            [torch.randn(1, 4, 4, 2, 9, device=device)] * 2)
