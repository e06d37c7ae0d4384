"""Pins the CPU oracle (oracle/oracle.py and the C loop restatement) without the reference.

The reference stores no golden vectors for this path (its tests print differences of random
inputs), so each oracle function is pinned by checks chosen so that a plausible mistake fails:
closed forms, brute-force loops, invariants of the mathematics, fp64 gradcheck, and agreement
of two independently written restatements (library routines vs straight C loops).
"""
import math

import numpy as np
import pytest
import torch

from oracle import loops as L
from oracle import oracle as O

torch.manual_seed(0)
D = torch.float64


def rnd(*shape, g=None):
    return torch.randn(*shape, dtype=D, generator=g)


def gen(seed):
    return torch.Generator().manual_seed(seed)


# ---- forward max / avg / argmax -------------------------------------------------------------

def test_all_ones_closed_form():
    # f1=f2=1 with C=c: S == c everywhere; max=avg=c; argmax is the lowest index (0)
    f1 = torch.ones(1, 3, 5, 7, dtype=D)
    f2 = torch.ones(1, 2, 4, 7, dtype=D)
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    assert torch.all(ou == 7) and torch.all(ov == 7)
    assert torch.all(au == 0) and torch.all(av == 0)
    assert ou.shape == (1, 3, 5, 2, 2) and ov.shape == (1, 3, 5, 2, 4)
    assert au.shape == (1, 3, 5, 1, 2) and av.shape == (1, 3, 5, 1, 4) and au.dtype == torch.int32


def test_one_hot_features_give_indicator_volume():
    # f2[u,v] = e_{u*W2+v}, f1[i,j] = e_{t(i,j)}: S[i,j,u,v] = [u*W2+v == t]
    H1, W1, H2, W2 = 2, 3, 3, 4
    C = H2 * W2
    f2 = torch.eye(C, dtype=D).reshape(1, H2, W2, C)
    t = torch.tensor([[0, 5, 11], [7, 2, 9]])
    f1 = torch.eye(C, dtype=D)[t].reshape(1, H1, W1, C)
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    for i in range(H1):
        for j in range(W1):
            tu, tv = divmod(int(t[i, j]), W2)
            exp_mu = torch.zeros(H2, dtype=D); exp_mu[tu] = 1
            exp_mv = torch.zeros(W2, dtype=D); exp_mv[tv] = 1
            assert torch.equal(ou[0, i, j, 0], exp_mu) and torch.equal(ov[0, i, j, 0], exp_mv)
            assert torch.allclose(ou[0, i, j, 1], exp_mu / W2) and torch.allclose(ov[0, i, j, 1], exp_mv / H2)
            assert int(au[0, i, j, 0, tu]) == tv and int(av[0, i, j, 0, tv]) == tu
            # rows without the hit are all-zero ties: lowest index
            assert all(int(au[0, i, j, 0, u]) == 0 for u in range(H2) if u != tu)
            assert all(int(av[0, i, j, 0, v]) == 0 for v in range(W2) if v != tv)


@pytest.mark.parametrize("shape", [(2, 3, 4, 5, 2, 3), (1, 4, 2, 3, 3, 1)])
def test_forward_matches_python_loops(shape):
    B, H1, W1, C, H2, W2 = shape
    f1, f2 = rnd(B, H1, W1, C), rnd(B, H2, W2, C)
    a_u, a_v = rnd(B, H1, W1, 3, W2), rnd(B, H1, W1, 3, H2)
    ref = O.loops_forward(f1, f2, a_u, a_v)
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    cu, cv = O.compression_forward(f1, f2, a_u, a_v)
    assert torch.allclose(ou, ref["out_u"], atol=1e-12) and torch.allclose(ov, ref["out_v"], atol=1e-12)
    assert torch.equal(au, ref["am_u"]) and torch.equal(av, ref["am_v"])
    assert torch.allclose(cu, ref["cu"], atol=1e-12) and torch.allclose(cv, ref["cv"], atol=1e-12)


def test_mean_identity_rank_one():
    # avg_v[i,j,v] = <f1[i,j], mean_u f2[u,v]>  and  avg_u[i,j,u] = <f1[i,j], mean_v f2[u,v]>: needs no 4D
    f1, f2 = rnd(2, 5, 6, 9), rnd(2, 4, 7, 9)
    ou, ov = O.max_avg_forward(f1, f2)
    assert torch.allclose(ov[:, :, :, 1], torch.einsum('bijc,bvc->bijv', f1, f2.mean(dim=1)), atol=1e-12)
    assert torch.allclose(ou[:, :, :, 1], torch.einsum('bijc,buc->biju', f1, f2.mean(dim=2)), atol=1e-12)


def test_transposing_fmap2_swaps_u_and_v_outputs():
    f1, f2 = rnd(1, 4, 5, 6), rnd(1, 3, 7, 6)
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    ou_t, ov_t, au_t, av_t = O.max_argmax_avg_forward(f1, f2.transpose(1, 2).contiguous())
    assert torch.allclose(ou, ov_t) and torch.allclose(ov, ou_t)
    assert torch.equal(au, av_t) and torch.equal(av, au_t)


def test_permuting_fmap2_columns_permutes_v_outputs_and_remaps_argmax_u():
    f1, f2 = rnd(1, 3, 4, 5), rnd(1, 4, 6, 5)
    perm = torch.tensor([3, 0, 5, 1, 4, 2])
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    ou_p, ov_p, au_p, av_p = O.max_argmax_avg_forward(f1, f2[:, :, perm].contiguous())
    assert torch.allclose(ou, ou_p)                      # reductions over v do not care about the order
    assert torch.allclose(ov[..., perm], ov_p) and torch.equal(av[..., perm], av_p)
    assert torch.equal(perm[au_p.long()], au.long())     # new index j holds old column perm[j]


def test_ties_resolve_to_lowest_index():
    f1 = torch.ones(1, 1, 1, 2, dtype=D)
    f2 = torch.zeros(1, 3, 4, 2, dtype=D)
    f2[0, 1, 2] = 1; f2[0, 1, 3] = 1; f2[0, 2, 2] = 1    # S = 2 at (1,2),(1,3),(2,2)
    _, _, au, av = O.max_argmax_avg_forward(f1, f2)
    assert au[0, 0, 0, 0].tolist() == [0, 2, 2]
    assert av[0, 0, 0, 0].tolist() == [0, 0, 1, 1]
    lu, lv, lau, lav = L.max_argmax_avg_forward(f1.numpy(), f2.numpy())
    assert lau[0, 0, 0, 0].tolist() == [0, 2, 2] and lav[0, 0, 0, 0].tolist() == [0, 0, 1, 1]


@pytest.mark.parametrize("level", [1, 2, 3])
def test_pooling_commutes_with_correlation(level):
    # avg_pool2d of the 4D volume == correlation against avg_pool2d(fmap2) (core/corr.py:36-38 vs :380-382),
    # including odd sizes (both floor)
    f1, f2 = rnd(1, 3, 3, 6), rnd(1, 11, 13, 6)
    a = O.pool_volume(O.corr_volume(f1, f2), level)
    b = O.corr_volume(f1, O.pool_fmap2(f2, level))
    assert a.shape == b.shape == (1, 3, 3, 11 >> level, 13 >> level)
    assert torch.allclose(a, b, atol=1e-12)


# ---- compression ------------------------------------------------------------------------------

def test_compression_structured_all_ones():
    # the reference's structured case (scripts/test_compression_cuda.py:210-242): f=1, C=10, 4x8, a=1
    f = torch.ones(1, 4, 8, 10, dtype=D)
    a_u = torch.ones(1, 4, 8, 2, 8, dtype=D)
    a_v = torch.ones(1, 4, 8, 2, 4, dtype=D)
    cu, cv = O.compression_forward(f, f, a_u, a_v)
    assert cu.shape == (1, 4, 8, 2, 4) and cv.shape == (1, 4, 8, 2, 8)
    assert torch.all(cu == 80) and torch.all(cv == 40)
    lcu, lcv = L.compression_forward(f.numpy(), f.numpy(), a_u.numpy(), a_v.numpy())
    assert np.all(lcu == 80) and np.all(lcv == 40)


def test_compression_reduces_to_avg_and_max_channels():
    f1, f2 = rnd(1, 3, 4, 5), rnd(1, 4, 6, 5)
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    H2, W2 = 4, 6
    # uniform weights -> the avg channel
    cu, cv = O.compression_forward(f1, f2, torch.full((1, 3, 4, 1, W2), 1 / W2, dtype=D),
                                   torch.full((1, 3, 4, 1, H2), 1 / H2, dtype=D))
    assert torch.allclose(cu[:, :, :, 0], ou[:, :, :, 1]) and torch.allclose(cv[:, :, :, 0], ov[:, :, :, 1])
    # a single one-hot weight vector picks one column / row of S
    s = O.corr_volume(f1, f2)
    a_u = torch.zeros(1, 3, 4, 1, W2, dtype=D); a_u[..., 4] = 1
    a_v = torch.zeros(1, 3, 4, 1, H2, dtype=D); a_v[..., 2] = 1
    cu, cv = O.compression_forward(f1, f2, a_u, a_v)
    assert torch.allclose(cu[:, :, :, 0], s[..., 4]) and torch.allclose(cv[:, :, :, 0], s[:, :, :, 2])


def test_compression_is_linear_in_weights():
    f1, f2 = rnd(1, 2, 3, 4), rnd(1, 3, 5, 4)
    a1, a2 = rnd(1, 2, 3, 2, 5), rnd(1, 2, 3, 2, 5)
    b1, b2 = rnd(1, 2, 3, 2, 3), rnd(1, 2, 3, 2, 3)
    x = O.compression_forward(f1, f2, 2 * a1 - 3 * a2, 2 * b1 - 3 * b2)
    y1 = O.compression_forward(f1, f2, a1, b1)
    y2 = O.compression_forward(f1, f2, a2, b2)
    assert torch.allclose(x[0], 2 * y1[0] - 3 * y2[0]) and torch.allclose(x[1], 2 * y1[1] - 3 * y2[1])


# ---- backward -----------------------------------------------------------------------------------

def test_maxavg_backward_formula_equals_autograd_through_4d():
    g = gen(3)
    f1, f2 = rnd(2, 4, 5, 6, g=g), rnd(2, 3, 7, 6, g=g)
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    g_u, g_v = rnd(*ou.shape, g=g), rnd(*ov.shape, g=g)
    d1, d2 = O.max_argmax_avg_backward(f1, f2, au, av, g_u, g_v)
    a1, a2 = O.autograd_max_avg(f1, f2, g_u, g_v)
    assert torch.allclose(d1, a1, atol=1e-10) and torch.allclose(d2, a2, atol=1e-10)


def test_compression_backward_formula_equals_autograd_through_4d():
    g = gen(4)
    f1, f2 = rnd(1, 3, 4, 5, g=g), rnd(1, 4, 3, 5, g=g)
    a_u, a_v = rnd(1, 3, 4, 3, 3, g=g), rnd(1, 3, 4, 3, 4, g=g)
    g_cu, g_cv = rnd(1, 3, 4, 3, 4, g=g), rnd(1, 3, 4, 3, 3, g=g)
    got = O.compression_backward(f1, f2, a_u, a_v, g_cu, g_cv)
    ref = O.autograd_compression(f1, f2, a_u, a_v, g_cu, g_cv)
    for x, y in zip(got, ref):
        assert torch.allclose(x, y, atol=1e-10)


def test_gradcheck_fp64_of_the_4d_definition():
    g = gen(5)
    f1, f2 = rnd(1, 2, 2, 3, g=g).requires_grad_(), rnd(1, 2, 3, 3, g=g).requires_grad_()
    a_u, a_v = rnd(1, 2, 2, 2, 3, g=g).requires_grad_(), rnd(1, 2, 2, 2, 2, g=g).requires_grad_()

    def avg_and_compression(f1, f2, a_u, a_v):
        s = O.corr_volume(f1, f2)
        cu, cv = O.compression_from_volume(s, a_u, a_v)
        return s.mean(dim=4), s.mean(dim=3), s.max(dim=4)[0], s.max(dim=3)[0], cu, cv

    assert torch.autograd.gradcheck(avg_and_compression, (f1, f2, a_u, a_v), eps=1e-6, atol=1e-6)


def test_backward_debug_case_of_the_reference():
    # scripts/test_maxavg_autograd.py:539-563: ones features, argmax==1 everywhere, grads = arange
    B, H, W, C = 1, 5, 6, 3
    f1 = torch.ones(B, H, W, C, dtype=D); f2 = torch.ones(B, H, W, C, dtype=D)
    au = torch.ones(B, H, W, 1, H, dtype=torch.int32); av = torch.ones(B, H, W, 1, W, dtype=torch.int32)
    g_u = torch.arange(H, dtype=D).expand(B, H, W, 2, H).contiguous()
    g_v = torch.arange(W, dtype=D).expand(B, H, W, 2, W).contiguous()
    d1, d2 = O.max_argmax_avg_backward(f1, f2, au, av, g_u, g_v)
    # closed form: sum_{u,v} G = 2*sum(arange(H)) + 2*sum(arange(W)) for every pixel, every channel
    tot = 2 * sum(range(H)) + 2 * sum(range(W))
    assert torch.allclose(d1, torch.full_like(d1, tot))
    # dF2[u,v] = N1 * (u*[v==1] + u/W + v*[u==1] + v/H)
    uu = torch.arange(H, dtype=D).view(H, 1); vv = torch.arange(W, dtype=D).view(1, W)
    exp = H * W * (uu * (vv == 1) + uu / W + vv * (uu == 1) + vv / H)
    assert torch.allclose(d2[0, :, :, 0], exp)
    l1, l2 = L.max_argmax_avg_backward(f1.numpy(), f2.numpy(), au.numpy(), av.numpy(), g_u.numpy(), g_v.numpy())
    assert np.allclose(l1, d1.numpy()) and np.allclose(l2, d2.numpy())


def test_avg_only_grads_give_rank_one_df2():
    # with only avg grads: dF2[u,v,:] = sum_p (g_u[p,1,u]/W2 + g_v[p,1,v]/H2) f1[p,:]
    g = gen(6)
    f1, f2 = rnd(1, 3, 4, 5, g=g), rnd(1, 4, 6, 5, g=g)
    g_u = torch.zeros(1, 3, 4, 2, 4, dtype=D); g_u[:, :, :, 1] = rnd(1, 3, 4, 4, g=g)
    g_v = torch.zeros(1, 3, 4, 2, 6, dtype=D); g_v[:, :, :, 1] = rnd(1, 3, 4, 6, g=g)
    _, _, au, av = O.max_argmax_avg_forward(f1, f2)
    _, d2 = O.max_argmax_avg_backward(f1, f2, au, av, g_u, g_v)
    exp = torch.einsum('biju,bijc->buc', g_u[:, :, :, 1], f1).unsqueeze(2) / 6 \
        + torch.einsum('bijv,bijc->bvc', g_v[:, :, :, 1], f1).unsqueeze(1) / 4
    assert torch.allclose(d2, exp, atol=1e-10)


def test_attention_gradient_identity():
    # sum_v a_u[v] da_u[v] == sum_u g_cu[u] comp_u[u]  (both equal sum_{u,v} S a_u g_cu)
    g = gen(7)
    f1, f2 = rnd(1, 2, 3, 4, g=g), rnd(1, 3, 5, 4, g=g)
    a_u, a_v = rnd(1, 2, 3, 2, 5, g=g), rnd(1, 2, 3, 2, 3, g=g)
    g_cu, g_cv = rnd(1, 2, 3, 2, 3, g=g), rnd(1, 2, 3, 2, 5, g=g)
    cu, cv = O.compression_forward(f1, f2, a_u, a_v)
    _, _, da_u, da_v = O.compression_backward(f1, f2, a_u, a_v, g_cu, g_cv)
    assert torch.allclose((a_u * da_u).sum(-1), (g_cu * cu).sum(-1))
    assert torch.allclose((a_v * da_v).sum(-1), (g_cv * cv).sum(-1))


# ---- two independent restatements agree ---------------------------------------------------------

@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-11), (np.float32, 2e-4)])
def test_c_loops_agree_with_library_restatement(dtype, tol):
    g = gen(8)
    B, H1, W1, H2, W2, C, K = 2, 6, 7, 5, 9, 13, 3
    td = torch.float64 if dtype == np.float64 else torch.float32
    f1, f2 = rnd(B, H1, W1, C, g=g).to(td), rnd(B, H2, W2, C, g=g).to(td)
    a_u, a_v = rnd(B, H1, W1, K, W2, g=g).to(td), rnd(B, H1, W1, K, H2, g=g).to(td)
    ou, ov, au, av = O.max_argmax_avg_forward(f1, f2)
    lu, lv, lau, lav = L.max_argmax_avg_forward(f1.numpy(), f2.numpy())
    assert np.allclose(ou.numpy(), lu, atol=tol) and np.allclose(ov.numpy(), lv, atol=tol)
    if dtype == np.float64:
        assert np.array_equal(au.numpy(), lau) and np.array_equal(av.numpy(), lav)
    cu, cv = O.compression_forward(f1, f2, a_u, a_v)
    lcu, lcv = L.compression_forward(f1.numpy(), f2.numpy(), a_u.numpy(), a_v.numpy())
    assert np.allclose(cu.numpy(), lcu, atol=tol) and np.allclose(cv.numpy(), lcv, atol=tol)
    g_u, g_v = rnd(*ou.shape, g=g).to(td), rnd(*ov.shape, g=g).to(td)
    d = O.max_argmax_avg_backward(f1, f2, au, av, g_u, g_v)
    l = L.max_argmax_avg_backward(f1.numpy(), f2.numpy(), au.numpy(), av.numpy(), g_u.numpy(), g_v.numpy())
    assert all(np.allclose(x.numpy(), y, atol=tol * 10) for x, y in zip(d, l))
    g_cu, g_cv = rnd(*cu.shape, g=g).to(td), rnd(*cv.shape, g=g).to(td)
    d = O.compression_backward(f1, f2, a_u, a_v, g_cu, g_cv)
    l = L.compression_backward(*(x.numpy() for x in (f1, f2, a_u, a_v, g_cu, g_cv)))
    assert all(np.allclose(x.numpy(), y, atol=tol * 10) for x, y in zip(d, l))


def test_out_of_range_argmax_selects_nothing():
    f1, f2 = rnd(1, 2, 2, 3), rnd(1, 2, 3, 3)
    au = torch.full((1, 2, 2, 1, 2), 99, dtype=torch.int32)
    av = torch.full((1, 2, 2, 1, 3), -5, dtype=torch.int32)
    g_u = torch.zeros(1, 2, 2, 2, 2, dtype=D); g_u[:, :, :, 0] = 1
    g_v = torch.zeros(1, 2, 2, 2, 3, dtype=D); g_v[:, :, :, 0] = 1
    d1, d2 = O.max_argmax_avg_backward(f1, f2, au, av, g_u, g_v)
    assert torch.all(d1 == 0) and torch.all(d2 == 0)
    l1, l2 = L.max_argmax_avg_backward(f1.numpy(), f2.numpy(), au.numpy(), av.numpy(), g_u.numpy(), g_v.numpy())
    assert np.all(l1 == 0) and np.all(l2 == 0)


# ---- attention-weight producer ---------------------------------------------------------------------

def test_attention_weights_closed_forms():
    g = gen(21)
    B, H1, W1, L, K = 1, 3, 4, 6, 2
    sep = rnd(B, H1, W1, 2, L, g=g)
    w = torch.zeros(K, 2, 3, 3, 3, dtype=D)
    # zero weights: uniform softmax, whatever the bias
    a = O.attention_weights(sep, w, torch.tensor([0.3, -2.0], dtype=D))
    assert a.shape == (B, H1, W1, K, L) and torch.allclose(a, torch.full_like(a, 1 / L))
    # centre tap on channel c: softmax of the pixel's own row
    w[0, 1, 1, 1, 1] = 2.0
    a = O.attention_weights(sep, w, None)
    assert torch.allclose(a[:, :, :, 0], (2.0 * sep[:, :, :, 1]).softmax(-1))
    # tap dl=2 reads l+1 (cross-correlation, zero padded); tap di=0 reads row i-1; tap dj=2 reads column j+1
    w.zero_(); w[1, 0, 2, 1, 1] = 1.0
    shifted = torch.cat((sep[:, :, :, 0, 1:], torch.zeros(B, H1, W1, 1, dtype=D)), dim=-1)
    assert torch.allclose(O.attention_weights(sep, w, None)[:, :, :, 1], shifted.softmax(-1))
    w.zero_(); w[0, 0, 1, 0, 1] = 1.0
    up = torch.cat((torch.zeros(B, 1, W1, L, dtype=D), sep[:, :-1, :, 0]), dim=1)
    assert torch.allclose(O.attention_weights(sep, w, None)[:, :, :, 0], up.softmax(-1))
    w.zero_(); w[0, 1, 1, 1, 2] = 1.0
    right = torch.cat((sep[:, :, 1:, 1], torch.zeros(B, H1, 1, L, dtype=D)), dim=2)
    assert torch.allclose(O.attention_weights(sep, w, None)[:, :, :, 0], right.softmax(-1))
    # rows sum to one
    a = O.attention_weights(sep, rnd(K, 2, 3, 3, 3, g=g), rnd(K, g=g))
    assert torch.allclose(a.sum(-1), torch.ones(B, H1, W1, K, dtype=D))


def test_attention_weights_equal_the_module_path():
    # the same numbers as the caller's torch.nn.Conv3d module applied to the permuted volume
    torch.manual_seed(3)
    conv = torch.nn.Conv3d(2, 3, 3, padding=1).double()
    sep = rnd(2, 4, 5, 2, 7)
    ref = conv(sep.permute(0, 3, 4, 1, 2)).softmax(dim=2).permute(0, 3, 4, 1, 2)
    assert torch.allclose(O.attention_weights(sep, conv.weight, conv.bias), ref, atol=1e-14)


# ---- module level ---------------------------------------------------------------------------------

def test_corrblock4d_level0_equals_op_level_and_scaling():
    fmap1, fmap2, f1, f2 = O.make_inputs(1, 6, 8, 16, seed=11, dtype=D)
    blk = O.CorrBlock4D(fmap1, fmap2, num_levels=1)
    corr1, corr2 = blk.separate(None)
    ou, ov = O.max_avg_forward(f1, f2)
    # corr1 (B,2,W,H1,W1) keeps v; corr2 (B,2,H,H1,W1) keeps u
    assert torch.allclose(corr1, ov.permute(0, 3, 4, 1, 2), atol=1e-12)
    assert torch.allclose(corr2, ou.permute(0, 3, 4, 1, 2), atol=1e-12)
    # scaling is 1/sqrt(C)
    s = O.corr_volume(f1, f2)
    assert math.isclose(float(s[0, 1, 2, 3, 4]), float((fmap1[0, :, 1, 2] * fmap2[0, :, 3, 4]).sum() / 4.0), rel_tol=1e-12)


def test_corrblock4d_shapes_and_channel_order_with_attention():
    torch.manual_seed(1)
    fmap1, fmap2, f1, f2 = O.make_inputs(1, 8, 16, 8, seed=12)
    att = (torch.nn.Conv3d(2, 2, 3, padding=1), torch.nn.Conv3d(2, 2, 3, padding=1))
    with torch.no_grad():
        corr1, corr2 = O.CorrBlock4D(fmap1, fmap2, num_levels=4).separate(att)
    assert corr1.shape == (1, 16, 16, 8, 16) and corr2.shape == (1, 16, 8, 8, 16)
    # level 0, channels 0..1 are max/avg; channels 2..3 the attention sums with softmax weights:
    ou, ov = O.max_avg_forward(f1, f2)
    assert torch.allclose(corr1[:, 0:2], ov.permute(0, 3, 4, 1, 2), atol=1e-5)
    with torch.no_grad():
        a_u = att[0](ov.permute(0, 3, 4, 1, 2)).softmax(dim=2).permute(0, 3, 4, 1, 2)
        a_v = att[1](ou.permute(0, 3, 4, 1, 2)).softmax(dim=2).permute(0, 3, 4, 1, 2)
    cu, cv = O.compression_forward(f1, f2, a_u.contiguous(), a_v.contiguous())
    assert torch.allclose(corr2[:, 2:4], cu.permute(0, 3, 4, 1, 2), atol=1e-5)
    assert torch.allclose(corr1[:, 2:4], cv.permute(0, 3, 4, 1, 2), atol=1e-5)
    # a softmax-weighted sum lies between min and max of what it averages
    s = O.corr_volume(f1, f2)
    assert torch.all(cu <= s.max(dim=4)[0].unsqueeze(3) + 1e-5) and torch.all(cu >= s.min(dim=4)[0].unsqueeze(3) - 1e-5)


def test_compression_from_logits_closed_forms_and_gradient_structure():
    """Pins oracle.compression_from_logits (softmax over the kept axis + compression, core/corr.py:441-448):
    constant logits give uniform weights, i.e. the avg channel of the max/avg operator; a row with one dominant
    logit picks one slice of the volume; the gradient of the logits equals the explicit softmax-backward formula
    applied to the operator's weight gradients, each of its rows sums to zero, and the row sums of a * d_a equal
    the dot products of upstream gradient and output (the identity the fused backward uses)."""
    B, H1, W1, H2, W2, C, K = 1, 3, 4, 5, 6, 8, 2
    g = torch.Generator().manual_seed(31)
    f1 = torch.randn(B, H1, W1, C, generator=g, dtype=torch.float64)
    f2 = torch.randn(B, H2, W2, C, generator=g, dtype=torch.float64)
    s = O.corr_volume(f1, f2)
    # constant logits (any constant): comp_u = mean over v, comp_v = mean over u
    cu, cv = O.compression_from_logits(f1, f2, torch.full((B, H1, W1, K, W2), 3.7, dtype=torch.float64),
                                       torch.full((B, H1, W1, K, H2), -1.2, dtype=torch.float64))
    assert torch.allclose(cu, s.mean(dim=4).unsqueeze(3).expand(-1, -1, -1, K, -1), atol=1e-12)
    assert torch.allclose(cv, s.mean(dim=3).unsqueeze(3).expand(-1, -1, -1, K, -1), atol=1e-12)
    # one dominant logit at column 2 / row 4: the slices S[..., :, 2] and S[..., 4, :]
    z_u = torch.zeros(B, H1, W1, K, W2, dtype=torch.float64); z_u[..., 2] = 800.0
    z_v = torch.zeros(B, H1, W1, K, H2, dtype=torch.float64); z_v[..., 4] = 800.0
    cu, cv = O.compression_from_logits(f1, f2, z_u, z_v)
    assert torch.allclose(cu[:, :, :, 0], s[..., 2], atol=1e-12) and torch.allclose(cv[:, :, :, 1], s[:, :, :, 4], atol=1e-12)
    # gradients
    z_u = torch.randn(B, H1, W1, K, W2, generator=g, dtype=torch.float64).requires_grad_()
    z_v = torch.randn(B, H1, W1, K, H2, generator=g, dtype=torch.float64).requires_grad_()
    g_cu = torch.randn(B, H1, W1, K, H2, generator=g, dtype=torch.float64)
    g_cv = torch.randn(B, H1, W1, K, W2, generator=g, dtype=torch.float64)
    cu, cv = O.compression_from_logits(f1, f2, z_u, z_v)
    ((cu * g_cu).sum() + (cv * g_cv).sum()).backward()
    a_u, a_v = z_u.detach().softmax(-1), z_v.detach().softmax(-1)
    _, _, da_u, da_v = O.compression_backward(f1, f2, a_u, a_v, g_cu, g_cv)
    for dz, a, da, gc, comp in ((z_u.grad, a_u, da_u, g_cu, cu.detach()), (z_v.grad, a_v, da_v, g_cv, cv.detach())):
        dot = (a * da).sum(-1, keepdim=True)
        assert torch.allclose(dz, a * (da - dot), atol=1e-12)
        assert float(dz.sum(-1).abs().max()) < 1e-12
        assert torch.allclose(dot.squeeze(-1), (gc * comp).sum(-1), atol=1e-12)


def test_attention_logits_is_the_producer_without_softmax():
    g = torch.Generator().manual_seed(7)
    sep = torch.randn(2, 3, 4, 2, 9, generator=g, dtype=torch.float64)
    w = torch.randn(3, 2, 3, 3, 3, generator=g, dtype=torch.float64)
    b = torch.randn(3, generator=g, dtype=torch.float64)
    z = O.attention_logits(sep, w, b)
    assert torch.allclose(z.softmax(-1), O.attention_weights(sep, w, b), atol=1e-13)
    # a one-tap filter at the centre copies channel 0 (plus bias)
    w1 = torch.zeros(1, 2, 3, 3, 3, dtype=torch.float64); w1[0, 0, 1, 1, 1] = 1.0
    assert torch.allclose(O.attention_logits(sep, w1, torch.tensor([0.5], dtype=torch.float64))[:, :, :, 0], sep[:, :, :, 0] + 0.5)
