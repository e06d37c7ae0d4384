"""GPU parity of the two ways sepcorr_max_argmax_avg_backward computes its gradients (sepcorr_set_max_avg_backward).

The gather path (feature rows chosen by the maxima + two small products for the averages) and the dense path
(recomputed correlation tiles) are each checked against the fp64 oracle on the same argmax, against each other, and
for run-to-run identity.  Cases the scan of the gather path has to get right: more hits in one column than its queue
holds, pixels that all choose the same position, argmax entries outside their range, pixel counts that are not a
multiple of the scan step, and channel counts below a full wave.
"""
import pytest
import torch

from oracle import oracle as O
from separableflowthesis_amd import MemorySaver as ms
from tests._util import assert_close, op_inputs

pytestmark = pytest.mark.gpu

SHAPES = [
    (1, 1, 1, 1, 1, 4),
    (2, 5, 7, 5, 7, 16),
    (1, 12, 40, 12, 40, 256),
    (1, 8, 150, 8, 150, 64),
    (1, 6, 250, 3, 125, 36),
    (2, 24, 32, 24, 32, 256),
    (1, 30, 36, 15, 20, 100),
    (8, 32, 48, 16, 24, 32),
    (1, 4, 40, 3, 300, 32),
    (1, 2, 3, 1, 2048, 8),
    (1, 33, 31, 33, 31, 252),    # 1023 pixels: one short of four scan steps; 63 lanes of channels
    (3, 16, 16, 40, 7, 128),     # more lines than a 32-line tile holds, three batches
    (1, 20, 52, 9, 300, 12),     # 309 lines: two chunks of the gradient tile
]


@pytest.fixture
def modes():
    prev = ms.set_max_avg_backward(ms.MAXAVG_AUTO)
    yield
    ms.set_max_avg_backward(prev)


def _run(mode, *args):
    ms.set_max_avg_backward(mode)
    return ms.max_argmax_avg_backward(*args)


@pytest.mark.parametrize("shape", SHAPES)
def test_gather_and_dense_against_the_oracle(device, modes, shape):
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=77)
    d = lambda t: t.to(device)
    ou, ov, au, av = ms.max_argmax_avg_forward(d(f1), d(f2))
    g_u = torch.randn(ou.shape, generator=g)
    g_v = torch.randn(ov.shape, generator=g)
    args = (d(f1), d(f2), au, av, d(g_u), d(g_v))
    r1, r2 = O.max_argmax_avg_backward(f1.double(), f2.double(), au.cpu(), av.cpu(), g_u.double(), g_v.double())
    for mode, name in ((ms.MAXAVG_GATHER, "gather"), (ms.MAXAVG_DENSE, "dense"), (ms.MAXAVG_AUTO, "auto")):
        d1, d2 = _run(mode, *args)
        assert_close(d1, r1, f"grad_fmap1_l0 ({name})", scale_atol=True)
        assert_close(d2, r2, f"grad_fmap2_lk ({name})", scale_atol=True)
        e1, e2 = _run(mode, *args)
        assert torch.equal(d1, e1) and torch.equal(d2, e2), f"{name}: results change from run to run"


def test_sizes_the_gather_path_does_not_take_fall_back_to_dense(device, modes):
    for shape in [(1, 9, 13, 4, 6, 117), (1, 2, 5, 2, 8, 1024), (1, 16, 48, 16, 48, 300)]:   # C % 4 != 0, C > 256
        B, H1, W1, H2, W2, C = shape
        f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=5)
        d = lambda t: t.to(device)
        ou, ov, au, av = ms.max_argmax_avg_forward(d(f1), d(f2))
        args = (d(f1), d(f2), au, av, d(torch.randn(ou.shape, generator=g)), d(torch.randn(ov.shape, generator=g)))
        a = _run(ms.MAXAVG_GATHER, *args)
        b = _run(ms.MAXAVG_DENSE, *args)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_mode_setter(modes):
    first = ms.set_max_avg_backward(ms.MAXAVG_GATHER)
    assert first == ms.MAXAVG_AUTO
    assert ms.set_max_avg_backward(99) == ms.MAXAVG_GATHER      # unknown mode: nothing changes
    assert ms.set_max_avg_backward(ms.MAXAVG_DENSE) == ms.MAXAVG_GATHER
    assert ms.set_max_avg_backward(first) == ms.MAXAVG_DENSE


@pytest.mark.parametrize("shape", [(1, 40, 50, 6, 9, 64), (2, 24, 60, 5, 8, 256)])
def test_every_pixel_chooses_the_same_position(device, modes, shape):
    """One position of fmap2 collects every pixel (2000 and 1440 hits in one column: several queue loads in a single
    scan step), all others none."""
    B, H1, W1, H2, W2, C = shape
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=9)
    au = torch.full((B, H1, W1, 1, H2), W2 - 2, dtype=torch.int32)
    av = torch.full((B, H1, W1, 1, W2), 1, dtype=torch.int32)
    g_u = torch.randn(B, H1, W1, 2, H2, generator=g)
    g_v = torch.randn(B, H1, W1, 2, W2, generator=g)
    d = lambda t: t.to(device)
    r1, r2 = O.max_argmax_avg_backward(f1.double(), f2.double(), au, av, g_u.double(), g_v.double())
    d1, d2 = _run(ms.MAXAVG_GATHER, d(f1), d(f2), d(au), d(av), d(g_u), d(g_v))
    assert_close(d1, r1, "grad_fmap1_l0", scale_atol=True)
    assert_close(d2, r2, "grad_fmap2_lk", scale_atol=True)


def test_random_argmax_and_entries_outside_the_range(device, modes):
    """Any index is accepted: entries outside [0, W2) or [0, H2) contribute nothing on either path (the dense kernels
    compare positions with the index; the gather path must not fetch through it)."""
    B, H1, W1, H2, W2, C = 2, 13, 21, 7, 12, 48
    f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=13)
    au = torch.randint(-3, W2 + 3, (B, H1, W1, 1, H2), generator=g, dtype=torch.int32)
    av = torch.randint(-3, H2 + 3, (B, H1, W1, 1, W2), generator=g, dtype=torch.int32)
    au[0, 0, 0, 0, 0] = 2 ** 31 - 1
    av[0, 0, 0, 0, 0] = -2 ** 31
    g_u = torch.randn(B, H1, W1, 2, H2, generator=g)
    g_v = torch.randn(B, H1, W1, 2, W2, generator=g)
    d = lambda t: t.to(device)
    args = (d(f1), d(f2), d(au), d(av), d(g_u), d(g_v))
    # oracle on the valid entries: an invalid index is a gradient of zero at a valid position
    ok_u = (au >= 0) & (au < W2)
    ok_v = (av >= 0) & (av < H2)
    gu0 = g_u.clone(); gu0[:, :, :, 0:1] *= ok_u
    gv0 = g_v.clone(); gv0[:, :, :, 0:1] *= ok_v
    r1, r2 = O.max_argmax_avg_backward(f1.double(), f2.double(), au.clamp(0, W2 - 1) * ok_u, av.clamp(0, H2 - 1) * ok_v,
                                       gu0.double(), gv0.double())
    for mode, name in ((ms.MAXAVG_GATHER, "gather"), (ms.MAXAVG_DENSE, "dense")):
        d1, d2 = _run(mode, *args)
        assert_close(d1, r1, f"grad_fmap1_l0 ({name})", scale_atol=True)
        assert_close(d2, r2, f"grad_fmap2_lk ({name})", scale_atol=True)


@pytest.mark.parametrize("size", [(2, 55, 128), (1, 136, 240)], ids=["cfg4", "cfg5"])
def test_gather_at_the_reference_resolution(device, modes, size):
    """C=256 at the sizes of benchmark configurations 4 and 5 on both paths: the gradients agree to fp32 rounding of
    sums of 183 / 376 rows per pixel (and about twice as many per position)."""
    (B, H, W), C = size, 256
    f1, f2, g = op_inputs(B, H, W, H, W, C, seed=31)
    d = lambda t: t.to(device)
    ou, ov, au, av = ms.max_argmax_avg_forward(d(f1), d(f2))
    args = (d(f1), d(f2), au, av, d(torch.randn(ou.shape, generator=g)), d(torch.randn(ov.shape, generator=g)))
    a1, a2 = _run(ms.MAXAVG_GATHER, *args)
    b1, b2 = _run(ms.MAXAVG_DENSE, *args)
    for x, y, n in ((a1, b1, "grad_fmap1_l0"), (a2, b2, "grad_fmap2_lk")):
        err = float((x - y).abs().max()) / float(y.abs().max())
        assert err < 2e-5, f"{n}: gather and dense differ by {err:.2e} of the largest entry"


def _inputs(device, seed, B=2, H=32, W=64, C=64):
    """A size whose three chains of kernels run on three streams (>= 300 000 rows, fmap2 below 4 MB per batch entry)."""
    f1, f2, g = op_inputs(B, H, W, H, W, C, seed=seed)
    t = dict(f1=f1, f2=f2,
             am_u=torch.randint(0, W, (B, H, W, 1, H), generator=g, dtype=torch.int32),
             am_v=torch.randint(0, H, (B, H, W, 1, W), generator=g, dtype=torch.int32),
             g_u=torch.randn(B, H, W, 2, H, generator=g), g_v=torch.randn(B, H, W, 2, W, generator=g))
    return {k: v.to(device) for k, v in t.items()}


def _bwd(t):
    return ms.max_argmax_avg_backward(t["f1"], t["f2"], t["am_u"], t["am_v"], t["g_u"], t["g_v"])


def test_gather_follows_the_callers_stream_and_replays_from_a_captured_graph(device, modes):
    """The gather path forks onto the library's two side streams and orders its last scan slice behind the table of
    average gradients with an event: under capture these become graph dependencies.  Every replay is checked against
    the eager result for the inputs of that replay, with eager work between the replays."""
    ms.set_max_avg_backward(ms.MAXAVG_GATHER)
    ref = _bwd(_inputs(device, seed=91))
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        t = {k: v.clone() for k, v in _inputs(device, seed=91).items()}   # produced on s: the op must wait for it
        got = _bwd(t)
    s.synchronize()
    assert all(torch.equal(x, y) for x, y in zip(got, ref))

    static = _inputs(device, seed=92)
    _bwd(static)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _bwd(static)
    for seed in (93, 94, 95):
        fresh = _inputs(device, seed=seed)
        ref = _bwd(fresh)
        torch.cuda.synchronize()
        for k in static:
            static[k].copy_(fresh[k])
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(x, y) for x, y in zip(outs, ref)), f"replay with seed {seed} differs from eager"


def test_gather_equals_dense_on_seeded_random_shapes(device, modes):
    """60 seeded shapes (all sizes 1..40, C a multiple of 4 up to 256, random argmax with a few entries outside the
    range): the two paths agree to fp32 rounding everywhere."""
    rng = torch.Generator().manual_seed(2024)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=rng))
    for n in range(60):
        B, H1, W1, H2, W2, C = r(1, 3), r(1, 40), r(1, 40), r(1, 40), r(1, 40), 4 * r(1, 64)
        f1, f2, g = op_inputs(B, H1, W1, H2, W2, C, seed=300 + n)
        au = torch.randint(-1, W2 + 1, (B, H1, W1, 1, H2), generator=g, dtype=torch.int32)
        av = torch.randint(-1, H2 + 1, (B, H1, W1, 1, W2), generator=g, dtype=torch.int32)
        g_u = torch.randn(B, H1, W1, 2, H2, generator=g)
        g_v = torch.randn(B, H1, W1, 2, W2, generator=g)
        args = tuple(t.to(device) for t in (f1, f2, au, av, g_u, g_v))
        a1, a2 = _run(ms.MAXAVG_GATHER, *args)
        b1, b2 = _run(ms.MAXAVG_DENSE, *args)
        for x, y, name in ((a1, b1, "grad_fmap1_l0"), (a2, b2, "grad_fmap2_lk")):
            scale = max(float(y.abs().max()), 1e-6)
            err = float((x - y).abs().max()) / scale
            assert err < 2e-5, f"shape {(B, H1, W1, H2, W2, C)} {name}: gather and dense differ by {err:.2e} of the largest entry"
