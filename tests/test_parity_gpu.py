"""GPU parity: every C-ABI entry point (through the ctypes mirror of the native module) against
the CPU oracle on the same seeded inputs.  Tolerances: rtol 1e-4 / atol 1e-5 (see _util.assert_close),
argmax exact except fp32 near-ties adjudicated with the fp64 volume."""
import pytest
import torch

from oracle import oracle as O
from tests._util import assert_close, check_argmax, op_inputs, softmax_weights

pytestmark = pytest.mark.gpu

# (B, H1, W1, H2, W2, C): ragged tiles, pooled fmap2, C not a multiple of 4/8, >4 waves, tiny
SHAPES = [
    (1, 1, 1, 1, 1, 1),
    (2, 5, 7, 5, 7, 16),
    (1, 9, 13, 4, 6, 117),      # pyramid-level fmap2, odd C (scalar load path)
    (3, 17, 31, 17, 31, 100),   # the reference's uniform tests use C=100 (scripts/test_maxavg_cuda.py:321-325)
    (1, 12, 40, 12, 40, 256),
    (1, 8, 150, 8, 150, 64),    # 5 waves per workgroup
    (1, 6, 250, 3, 125, 36),    # 8-wave f1 side irrelevant; W2=125 -> 4 waves, ragged
    (1, 4, 256, 4, 256, 32),    # widest supported row: 8 waves
    (2, 24, 32, 24, 32, 256),
    (2, 9, 20, 9, 20, 64),      # W2 % 4 == 0 and C % 4 == 0: tiled d_f2 path, row count not a multiple of 4
    (1, 30, 36, 15, 20, 100),   # tiled d_f2 with a ragged 128-channel block and pooled fmap2
    (1, 16, 48, 16, 48, 300),   # two channel blocks, the second ragged
    (8, 32, 48, 16, 24, 32),    # narrow rows, many workgroups: 1 column chunk x 4 row groups
    (1, 4, 40, 3, 300, 32),     # rows wider than 256 columns: two column passes
    (1, 5, 24, 2, 520, 20),     # three column passes, last one ragged
    (1, 3, 11, 2, 301, 7),      # wide rows on the generic load paths
    (1, 2, 3, 1, 2048, 8),      # the widest supported row: 8 column passes
    (1, 2, 5, 2, 8, 1024),      # the most channels supported: 4 channel blocks in the backward kernels
]


def _native():
    from separableflowthesis_amd import MemorySaver
    return MemorySaver


@pytest.mark.parametrize("shape", SHAPES)
def test_max_argmax_avg_forward(device, shape):
    B, H1, W1, H2, W2, C = shape
    f1, f2, _ = op_inputs(B, H1, W1, H2, W2, C, seed=hash(shape) % 1000)
    ms = _native()
    ou, ov, au, av = ms.max_argmax_avg_forward(f1.to(device), f2.to(device))
    s64 = O.corr_volume(f1.double(), f2.double())
    rou, rov, rau, rav = O.max_argmax_avg_from_volume(s64)
    assert ou.shape == rou.shape and ov.shape == rov.shape and au.shape == rau.shape and av.shape == rav.shape
    assert au.dtype == torch.int32 and av.dtype == torch.int32
    assert_close(ou, rou, "max_avg_output_u")
    assert_close(ov, rov, "max_avg_output_v")
    check_argmax(au, rau, s64, 4, "argmax_output_u")
    check_argmax(av, rav, s64, 3, "argmax_output_v")
    # the variant without argmax returns the same numbers bit for bit
    ou2, ov2 = ms.max_avg_forward(f1.to(device), f2.to(device))
    assert torch.equal(ou, ou2) and torch.equal(ov, ov2)


@pytest.mark.parametrize("shape", SHAPES[1:7] + SHAPES[12:])
@pytest.mark.parametrize("K", [1, 2, 4, 5])
def test_compression_forward(device, shape, K):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=7 + K)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    cu, cv = _native().compression_forward(f1.to(device), f2.to(device), a_u.to(device), a_v.to(device))
    rcu, rcv = O.compression_forward(f1.double(), f2.double(), a_u.double(), a_v.double())
    assert_close(cu, rcu, "compression_output_u")
    assert_close(cv, rcv, "compression_output_v")


def test_compression_forward_structured_ones(device):
    # scripts/test_compression_cuda.py:210-242
    f = torch.ones(1, 4, 8, 10, device=device)
    a_u = torch.ones(1, 4, 8, 2, 8, device=device)
    a_v = torch.ones(1, 4, 8, 2, 4, device=device)
    cu, cv = _native().compression_forward(f, f, a_u, a_v)
    assert torch.all(cu == 80) and torch.all(cv == 40)


def test_forward_ties_lowest_index(device):
    f1 = torch.ones(1, 1, 1, 2)
    f2 = torch.zeros(1, 3, 4, 2)
    f2[0, 1, 2] = 1; f2[0, 1, 3] = 1; f2[0, 2, 2] = 1
    _, _, au, av = _native().max_argmax_avg_forward(f1.to(device), f2.to(device))
    assert au[0, 0, 0, 0].tolist() == [0, 2, 2] and av[0, 0, 0, 0].tolist() == [0, 0, 1, 1]
    # all-equal volume across several waves: every argmax is 0
    f1 = torch.ones(1, 2, 3, 4); f2 = torch.ones(1, 5, 100, 4)
    ou, ov, au, av = _native().max_argmax_avg_forward(f1.to(device), f2.to(device))
    assert torch.all(au == 0) and torch.all(av == 0) and torch.all(ou == 4) and torch.all(ov == 4)
    # the same where a row is swept in several passes of 256 columns and the last chunk is ragged
    f1 = torch.ones(1, 2, 3, 8); f2 = torch.ones(1, 3, 300, 8)
    ou, ov, au, av = _native().max_argmax_avg_forward(f1.to(device), f2.to(device))
    assert torch.all(au == 0) and torch.all(av == 0) and torch.all(ou == 8) and torch.all(ov == 8)
    # two equal maxima in different column passes: the lower column wins
    f2 = torch.zeros(1, 2, 300, 8); f2[0, 0, 290] = 1; f2[0, 0, 17] = 1; f2[0, 1, 299] = 1; f2[0, 1, 256] = 1
    _, _, au, av = _native().max_argmax_avg_forward(f1.to(device), f2.to(device))
    assert torch.all(au[..., 0] == 17) and torch.all(au[..., 1] == 256)


@pytest.mark.parametrize("shape", [(1, 2, 5, 3, 40, 16), (1, 3, 7, 9, 300, 32), (2, 4, 4, 20, 70, 256)])
def test_argmax_stays_in_range_without_finite_values(device, shape):
    """Rows/columns holding only NaN or -inf: the reference's kernel leaves its pre-zeroed argmax at 0
    (MemorySaver_kernel_forward.cu:990-992 zero-fill, :498-507 strict '>' update); every index must stay a valid
    index of its axis, so that a consumer may gather with it."""
    B, H1, W1, H2, W2, C = shape
    g = torch.Generator().manual_seed(8)
    f1 = torch.randn(B, H1, W1, C, generator=g)
    f2 = torch.randn(B, H2, W2, C, generator=g)
    f1n = f1.clone(); f1n[0, 0, 0] = float("nan")            # pixel (0,0): the whole slice S[0,0,0,:,:] is NaN
    f2n = f2.clone(); f2n[0, H2 - 1] = float("nan")          # last fmap2 row: NaN for every pixel
    for a, b in ((f1n, f2), (f1, f2n), (f1n, f2n)):
        _, _, au, av = _native().max_argmax_avg_forward(a.to(device), b.to(device))
        assert int(au.min()) >= 0 and int(au.max()) < W2
        assert int(av.min()) >= 0 and int(av.max()) < H2
    _, _, au, av = _native().max_argmax_avg_forward(f1n.to(device), f2.to(device))
    assert torch.all(au[0, 0, 0] == 0) and torch.all(av[0, 0, 0] == 0)
    # -inf everywhere for one pixel (inf * positive features of one sign)
    f1i = f1.abs(); f1i[0, 0, 0] = float("-inf")
    _, _, au, av = _native().max_argmax_avg_forward(f1i.to(device), f2.abs().to(device))
    assert torch.all(au[0, 0, 0] == 0) and torch.all(av[0, 0, 0] == 0)


@pytest.mark.parametrize("shape", SHAPES)
def test_max_argmax_avg_backward(device, shape):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=21)
    ms = _native()
    d = lambda t: t.to(device)
    ou, ov, au, av = ms.max_argmax_avg_forward(d(f1), d(f2))
    g_u = torch.randn(ou.shape, generator=g)
    g_v = torch.randn(ov.shape, generator=g)
    d1, d2 = ms.max_argmax_avg_backward(d(f1), d(f2), au, av, d(g_u), d(g_v))
    # same argmax on both sides: the backward formula is then a plain linear map
    r1, r2 = O.max_argmax_avg_backward(f1.double(), f2.double(), au.cpu(), av.cpu(), g_u.double(), g_v.double())
    assert_close(d1, r1, "grad_fmap1_l0", scale_atol=True)
    assert_close(d2, r2, "grad_fmap2_lk", scale_atol=True)
    # run-to-run identical: no atomics anywhere
    e1, e2 = ms.max_argmax_avg_backward(d(f1), d(f2), au, av, d(g_u), d(g_v))
    assert torch.equal(d1, e1) and torch.equal(d2, e2)


def test_backward_debug_case_of_the_reference(device):
    # scripts/test_maxavg_autograd.py:539-563
    B, H, W, C = 1, 15, 15, 3
    f = torch.ones(B, H, W, C, device=device)
    au = torch.ones(B, H, W, 1, H, dtype=torch.int32, device=device)
    av = torch.ones(B, H, W, 1, W, dtype=torch.int32, device=device)
    g_u = torch.arange(H, dtype=torch.float32, device=device).expand(B, H, W, 2, H).contiguous()
    g_v = torch.arange(W, dtype=torch.float32, device=device).expand(B, H, W, 2, W).contiguous()
    d1, d2 = _native().max_argmax_avg_backward(f, f, au, av, g_u, g_v)
    r1, r2 = O.max_argmax_avg_backward(f.cpu().double(), f.cpu().double(), au.cpu(), av.cpu(), g_u.cpu().double(), g_v.cpu().double())
    assert_close(d1, r1, "grad_fmap1_l0", scale_atol=True)
    assert_close(d2, r2, "grad_fmap2_lk", scale_atol=True)


def test_backward_out_of_range_argmax_is_harmless(device):
    f1, f2, g = op_inputs(1, 4, 5, 4, 5, 8, seed=3)
    au = torch.full((1, 4, 5, 1, 4), 1000, dtype=torch.int32, device=device)
    av = torch.full((1, 4, 5, 1, 5), -7, dtype=torch.int32, device=device)
    g_u = torch.zeros(1, 4, 5, 2, 4, device=device); g_u[:, :, :, 0] = 1
    g_v = torch.zeros(1, 4, 5, 2, 5, device=device); g_v[:, :, :, 0] = 1
    d1, d2 = _native().max_argmax_avg_backward(f1.to(device), f2.to(device), au, av, g_u, g_v)
    assert torch.all(d1 == 0) and torch.all(d2 == 0)


@pytest.mark.parametrize("shape", SHAPES[1:7] + SHAPES[9:])
@pytest.mark.parametrize("K", [1, 2, 4, 5])
def test_compression_backward(device, shape, K):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=31 + K)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    d = lambda t: t.to(device)
    got = _native().compression_backward(d(f1), d(f2), d(a_u), d(a_v), d(g_cu), d(g_cv))
    ref = O.compression_backward(*(t.double() for t in (f1, f2, a_u, a_v, g_cu, g_cv)))
    for x, y, n in zip(got, ref, ("grad_fmap1_l0", "grad_fmap2_lk", "grad_attention_u", "grad_attention_v")):
        assert_close(x, y, n, scale_atol=True)
    again = _native().compression_backward(d(f1), d(f2), d(a_u), d(a_v), d(g_cu), d(g_cv))
    assert all(torch.equal(x, y) for x, y in zip(got, again))


@pytest.mark.parametrize("shape", SHAPES[1:7] + SHAPES[9:])
@pytest.mark.parametrize("K", [1, 2, 3, 4, 6])
def test_fused_backward_is_the_sum_of_both_backwards(device, shape, K):
    # G of the two operators added before the contraction: the oracle is the sum of its two backward functions
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=51 + K)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    g_u = torch.randn(B, H1, W1, 2, H2, generator=g)
    g_v = torch.randn(B, H1, W1, 2, W2, generator=g)
    d = lambda t: t.to(device)
    ms = _native()
    _, _, au, av = ms.max_argmax_avg_forward(d(f1), d(f2))
    d1, d2 = ms.fused_backward(d(f1), d(f2), au, av, d(g_u), d(g_v), d(a_u), d(a_v), d(g_cu), d(g_cv))
    m1, m2 = O.max_argmax_avg_backward(f1.double(), f2.double(), au.cpu(), av.cpu(), g_u.double(), g_v.double())
    c1, c2, ra_u, ra_v = O.compression_backward(*(t.double() for t in (f1, f2, a_u, a_v, g_cu, g_cv)))
    assert_close(d1, m1 + c1, "grad_fmap1_l0", scale_atol=True)
    assert_close(d2, m2 + c2, "grad_fmap2_lk", scale_atol=True)
    e1, e2 = ms.fused_backward(d(f1), d(f2), au, av, d(g_u), d(g_v), d(a_u), d(a_v), d(g_cu), d(g_cv))
    assert torch.equal(d1, e1) and torch.equal(d2, e2)
    # added to a gradient of fmap1 that other pyramid levels left (sepcorr_fused_backward_add): same d_f2, d_f1 on top
    other = torch.randn(f1.shape, generator=g).to(device)
    s1, s2 = ms.fused_backward(d(f1), d(f2), au, av, d(g_u), d(g_v), d(a_u), d(a_v), d(g_cu), d(g_cv), add_to_grad_fmap1=other.clone())
    assert torch.equal(s2, d2)
    err = float((s1 - (other + d1)).abs().max())   # one fp32 addition apart
    assert err <= 1e-6 * max(1.0, float(d1.abs().max())), f"grad_fmap1_l0 added to another level's: differs by {err}"
    # the weight gradients alone (compression backward without feature gradients)
    da_u, da_v = ms.compression_weight_gradients(d(f1), d(f2), d(a_u), d(a_v), d(g_cu), d(g_cv))
    assert_close(da_u, ra_u, "grad_attention_u", scale_atol=True)
    assert_close(da_v, ra_v, "grad_attention_v", scale_atol=True)


# From 2^25 (pixel, position) pairs on the library takes the combined d_f2 with 8-row workgroups, whose average term
# of g_v comes from a table; sizes above that limit with one and two channel blocks, two and four weight channels,
# rows that are no multiple of 32 columns and row counts that are no multiple of 8.
@pytest.mark.parametrize("shape,K", [((2, 56, 100, 56, 100, 64), 2), ((1, 72, 120, 72, 120, 128), 4),
                                     ((1, 78, 112, 78, 112, 128), 2), ((1, 64, 96, 64, 96, 256), 2)])
def test_fused_backward_above_the_8_row_limit(device, shape, K):
    B, H1, W1, H2, W2, C = shape
    assert B * H1 * W1 * H2 * W2 >= 2 ** 25
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=151 + K)
    a_u = softmax_weights(B, H1, W1, K, W2, g)
    a_v = softmax_weights(B, H1, W1, K, H2, g)
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g)
    g_u = torch.randn(B, H1, W1, 2, H2, generator=g)
    g_v = torch.randn(B, H1, W1, 2, W2, generator=g)
    d = lambda t: t.to(device)
    ms = _native()
    _, _, au, av = ms.max_argmax_avg_forward(d(f1), d(f2))
    d1, d2 = ms.fused_backward(d(f1), d(f2), au, av, d(g_u), d(g_v), d(a_u), d(a_v), d(g_cu), d(g_cv))
    # the library's two separate backward calls
    x1, x2, _, _ = ms.compression_backward(d(f1), d(f2), d(a_u), d(a_v), d(g_cu), d(g_cv))
    y1, y2 = ms.max_argmax_avg_backward(d(f1), d(f2), au, av, d(g_u), d(g_v))
    assert_close(d1, (x1 + y1).double(), "grad_fmap1_l0 against the two calls", scale_atol=True)
    assert_close(d2, (x2 + y2).double(), "grad_fmap2_lk against the two calls", scale_atol=True)
    # the fp64 oracle, one batch entry at a time (the 4D volume of these sizes is 0.3-0.6 GB in fp64)
    for b in range(B):
        sl = slice(b, b + 1)
        m1, m2 = O.max_argmax_avg_backward(f1[sl].double(), f2[sl].double(), au[sl].cpu(), av[sl].cpu(),
                                           g_u[sl].double(), g_v[sl].double())
        c1, c2, _, _ = O.compression_backward(*(t[sl].double() for t in (f1, f2, a_u, a_v, g_cu, g_cv)))
        assert_close(d1[sl], m1 + c1, "grad_fmap1_l0", scale_atol=True)
        assert_close(d2[sl], m2 + c2, "grad_fmap2_lk", scale_atol=True)
    e1, e2 = ms.fused_backward(d(f1), d(f2), au, av, d(g_u), d(g_v), d(a_u), d(a_v), d(g_cu), d(g_cv))
    assert torch.equal(d1, e1) and torch.equal(d2, e2)


def test_autograd_functions_match_autograd_through_4d(device):
    # mirrors overall_grad_test (scripts/test_maxavg_autograd.py:478-502, test_compression_autograd.py:442-484):
    # loss = sum of MSE(channel, 0) over all output channels, at a pooled level
    from separableflowthesis_amd import ComputeMaxArgmaxAvgFunction, ComputeSelfCompressionFunction
    B, H, W, C, K, level = 2, 16, 24, 37, 2, 1
    f1, f2l0, g = op_inputs(B, H, W, H, W, C, seed=5, scale=False)
    f1 = f1 / 8
    a_u = softmax_weights(B, H, W, K, W >> level, g)
    a_v = softmax_weights(B, H, W, K, H >> level, g)

    def loss_of(outs):
        return sum((o ** 2).mean() for t in outs for o in t.unbind(dim=3))

    # 4D autograd on the CPU in fp64
    c = [t.double().clone().requires_grad_() for t in (f1, f2l0, a_u, a_v)]
    s = O.pool_volume(O.corr_volume(c[0], c[1]), level)
    mu, mv = s.max(dim=4)[0], s.max(dim=3)[0]
    outs = (torch.stack((mu, s.mean(dim=4)), 3), torch.stack((mv, s.mean(dim=3)), 3)) + O.compression_from_volume(s, c[2], c[3])
    loss_of(outs).backward()
    # the operator on the GPU, fmap2 pooled outside as AlternateCorrBlockSepflow does
    x = [t.to(device).clone().requires_grad_() for t in (f1, f2l0, a_u, a_v)]
    f2lk = O.pool_fmap2(x[1], level)
    o1 = ComputeMaxArgmaxAvgFunction.apply(x[0], f2lk)
    o2 = ComputeSelfCompressionFunction.apply(x[0], f2lk, x[2], x[3])
    loss_of(o1 + o2).backward()
    for got, ref, n in zip(x, c, ("fmap1", "fmap2", "a_u", "a_v")):
        assert_close(got.grad, ref.grad, "grad " + n, scale_atol=True)


def test_max_avg_function_has_no_backward(device):
    from separableflowthesis_amd import ComputeMaxAvgFunction, ComputeMaxAvgModule
    f1 = torch.randn(1, 4, 4, 8, device=device, requires_grad=True)
    f2 = torch.randn(1, 4, 4, 8, device=device)
    ou, ov = ComputeMaxAvgModule()(f1, f2)
    with pytest.raises(NotImplementedError):
        (ou.sum() + ov.sum()).backward()


def test_error_conventions_on_device(device):
    ms = _native()
    f = torch.randn(1, 4, 4, 8, device=device)
    with pytest.raises(RuntimeError, match="contiguous"):
        ms.max_avg_forward(f.permute(0, 2, 1, 3), f)
    with pytest.raises(RuntimeError, match="dtype"):
        ms.max_avg_forward(f.double(), f.double())
    with pytest.raises(RuntimeError, match="differ"):
        ms.max_avg_forward(f, torch.randn(1, 4, 4, 9, device=device))
    with pytest.raises(RuntimeError, match="exceeds"):
        ms.max_avg_forward(torch.randn(1, 1, 2, 4, device=device), torch.randn(1, 1, 2100, 4, device=device))
    with pytest.raises(RuntimeError, match="shape"):
        ms.compression_forward(f, f, torch.randn(1, 4, 4, 2, 4, device=device), torch.randn(1, 4, 4, 2, 5, device=device))


def _all_ops(ms, t):
    ou, ov, au, av = ms.max_argmax_avg_forward(t["f1"], t["f2"])
    cu, cv = ms.compression_forward(t["f1"], t["f2"], t["a_u"], t["a_v"])
    c1, c2, da_u, da_v = ms.compression_backward(t["f1"], t["f2"], t["a_u"], t["a_v"], t["g_cu"], t["g_cv"])
    m1, m2 = ms.max_argmax_avg_backward(t["f1"], t["f2"], au, av, t["g_u"], t["g_v"])
    f1, f2 = ms.fused_backward(t["f1"], t["f2"], au, av, t["g_u"], t["g_v"], t["a_u"], t["a_v"], t["g_cu"], t["g_cv"])
    return [ou, ov, au, av, cu, cv, c1, c2, da_u, da_v, m1, m2, f1, f2]


def _op_tensors(device, seed, B=2, H1=9, W1=20, H2=9, W2=20, C=64, K=4):
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=seed)
    t = dict(f1=f1, f2=f2, a_u=softmax_weights(B, H1, W1, K, W2, g), a_v=softmax_weights(B, H1, W1, K, H2, g),
             g_u=torch.randn(B, H1, W1, 2, H2, generator=g), g_v=torch.randn(B, H1, W1, 2, W2, generator=g),
             g_cu=torch.randn(B, H1, W1, K, H2, generator=g), g_cv=torch.randn(B, H1, W1, K, W2, generator=g))
    return {k: v.to(device) for k, v in t.items()}


def test_ops_follow_the_callers_stream(device):
    # work queued on a side stream right after the inputs were produced there; the library's own side streams
    # fork from and join back into that stream
    ms = _native()
    ref = _all_ops(ms, _op_tensors(device, seed=71))
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        t = _op_tensors(device, seed=71)
        t = {k: v * 1.0 for k, v in t.items()}   # produced on s: the ops must wait for it
        got = _all_ops(ms, t)
    s.synchronize()
    assert all(torch.equal(x, y) for x, y in zip(got, ref))


def test_ops_replay_correctly_from_a_captured_graph(device):
    # all five reference functions and the fused backward in one captured graph (outputs and scratch come from
    # the graph's pool); every replay is checked against the eager result for the inputs of that replay
    ms = _native()
    static = _op_tensors(device, seed=81)
    _all_ops(ms, static)                      # warm-up outside the capture (lazy initialisations)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _all_ops(ms, static)
    for seed in (82, 83, 84):
        fresh = _op_tensors(device, seed=seed)
        ref = _all_ops(ms, fresh)             # eager work between the replays
        torch.cuda.synchronize()
        for k in static:
            static[k].copy_(fresh[k])
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(x, y) for x, y in zip(outs, ref)), f"replay with seed {seed} differs from eager"
