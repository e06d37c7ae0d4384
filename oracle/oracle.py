"""CPU oracle for the memory-saving cost-volume separation.  TEST INFRASTRUCTURE ONLY.

This file restates, with plain library routines on the CPU, what the reference
computes on its full-4D path.  It is the checker that the HIP kernels are
compared with; nothing in the shipped package imports it.  Only tests,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
use it.

Axis naming follows the reference's kernels: ``u`` indexes fmap2 rows
(0..H2), ``v`` indexes fmap2 columns (0..W2).  A tensor named ``*_u`` keeps the
u axis (it was reduced over v) and has last dimension H2; ``*_v`` keeps v.

Every function cites the reference lines it follows.  How each one is pinned
(closed forms, brute-force loops, invariants, fp64 gradcheck, the independent
C loop restatement in ``sepcorr_loops.c``) is listed in tests/test_oracle.py;
the reference stores no golden vectors for this path, so none are replayed.
The two lookups (``CorrBlock4D.lookup`` / ``lookup_direct`` for the 4D pyramid,
``CorrBlock1D`` / ``lookup1d_direct`` for the separated volumes) are pinned in
tests/test_lookup_oracle.py and tests/test_lookup1d_oracle.py: entries of the
stored volume at integer targets, affine volumes reproduced exactly at every
level, zero padding, the reference's clamp, and agreement of two independent
formulations in values and gradients.
"""
import math

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# op level: what the five native entry points compute
# --------------------------------------------------------------------------

def corr_volume(f1, f2):
    """Full 4D correlation S[b,i,j,u,v] = <f1[b,i,j,:], f2[b,u,v,:]>.

    No scaling: the caller pre-scales f1 (core/corr.py:419).  Follows
    scripts/test_maxavg_cuda.py:118-125 (matmul of flattened NHWC features).
    """
    B, H1, W1, C = f1.shape
    _, H2, W2, _ = f2.shape
    s = torch.matmul(f1.reshape(B, H1 * W1, C), f2.reshape(B, H2 * W2, C).transpose(1, 2))
    return s.reshape(B, H1, W1, H2, W2)


def pool_volume(s, level):
    """avg_pool2d(2,2) of the 4D volume over (u,v), `level` times.

    Follows core/corr.py:32-38 and scripts/test_maxavg_cuda.py:127-131.
    """
    B, H1, W1, H2, W2 = s.shape
    s = s.reshape(B * H1 * W1, 1, H2, W2)
    for _ in range(level):
        s = F.avg_pool2d(s, 2, stride=2)
    return s.reshape(B, H1, W1, s.shape[2], s.shape[3])


def pool_fmap2(f2, level):
    """avg_pool2d(2,2) of NHWC fmap2, `level` times (core/corr.py:377-382)."""
    x = f2.permute(0, 3, 1, 2)
    for _ in range(level):
        x = F.avg_pool2d(x, 2, stride=2)
    return x.permute(0, 2, 3, 1).contiguous()


def max_argmax_avg_from_volume(s):
    """max / mean / argmax over each displacement axis of a 4D volume.

    Follows core/corr.py:77-102 (max and mean over dim h2, then over dim w2)
    and scripts/test_maxavg_cuda.py:137-144.  Returns op-level layouts
    (libs/MemorySaver/functions/MemorySaver.py:17-18):
      out_u (B,H1,W1,2,H2): [max_v S, mean_v S];  argmax_u (B,H1,W1,1,H2) int32 = v index
      out_v (B,H1,W1,2,W2): [max_u S, mean_u S];  argmax_v (B,H1,W1,1,W2) int32 = u index
    Ties resolve to the lowest index as in the reference kernel's strict '<'
    update (MemorySaver_kernel_forward.cu:498-507); enforced here explicitly
    instead of relying on the library's tie rule.
    """
    max_u, _ = s.max(dim=4)
    max_v, _ = s.max(dim=3)
    avg_u = s.mean(dim=4)
    avg_v = s.mean(dim=3)
    W2 = s.shape[4]
    H2 = s.shape[3]
    iv = torch.arange(W2).view(1, 1, 1, 1, W2).expand_as(s)
    iu = torch.arange(H2).view(1, 1, 1, H2, 1).expand_as(s)
    big = max(H2, W2) + 1
    am_u = torch.where(s == max_u.unsqueeze(4), iv, torch.full_like(iv, big)).min(dim=4)[0]
    am_v = torch.where(s == max_v.unsqueeze(3), iu, torch.full_like(iu, big)).min(dim=3)[0]
    out_u = torch.stack((max_u, avg_u), dim=3)
    out_v = torch.stack((max_v, avg_v), dim=3)
    return out_u, out_v, am_u.unsqueeze(3).to(torch.int32), am_v.unsqueeze(3).to(torch.int32)


def max_avg_forward(f1, f2):
    """ComputeMaxAvgFunction.forward (functions/MemorySaver.py:6-28)."""
    out_u, out_v, _, _ = max_argmax_avg_from_volume(corr_volume(f1, f2))
    return out_u, out_v


def max_argmax_avg_forward(f1, f2):
    """ComputeMaxArgmaxAvgFunction.forward (functions/MemorySaver.py:40-68)."""
    return max_argmax_avg_from_volume(corr_volume(f1, f2))


def compression_from_volume(s, a_u, a_v):
    """Attention-weighted sums of a 4D volume; weights used as given (no softmax).

    Follows core/corr.py:128,140 and scripts/test_compression_cuda.py:105-159:
      comp_u[b,i,j,k,u] = sum_v S[b,i,j,u,v] * a_u[b,i,j,k,v]
      comp_v[b,i,j,k,v] = sum_u S[b,i,j,u,v] * a_v[b,i,j,k,u]
    a_u (B,H1,W1,K,W2), a_v (B,H1,W1,K,H2).
    """
    comp_u = torch.einsum('bijuv,bijkv->bijku', s, a_u)
    comp_v = torch.einsum('bijuv,bijku->bijkv', s, a_v)
    return comp_u, comp_v


def compression_forward(f1, f2, a_u, a_v):
    """ComputeSelfCompressionFunction.forward (functions/MemorySaver.py:107-137)."""
    return compression_from_volume(corr_volume(f1, f2), a_u, a_v)


def max_argmax_avg_grad_volume(am_u, am_v, g_u, g_v, H2, W2):
    """dL/dS for the max/avg op given upstream grads and argmax indices.

    Follows MemorySaver_kernel_max_avg_argmax_backward.cu:263-274 / :825-921:
      G = g_u[max]*[v==argmax_u] + g_u[avg]/W2 + g_v[max]*[u==argmax_v] + g_v[avg]/H2
    Indices are data: an index outside the axis selects nothing.
    """
    B, H1, W1 = g_u.shape[:3]
    iv = torch.arange(W2).view(1, 1, 1, 1, W2)
    iu = torch.arange(H2).view(1, 1, 1, H2, 1)
    amu = am_u[:, :, :, 0].long().unsqueeze(4)       # (B,H1,W1,H2,1)
    amv = am_v[:, :, :, 0].long().unsqueeze(3)       # (B,H1,W1,1,W2)
    G = (iv == amu).to(g_u.dtype) * g_u[:, :, :, 0].unsqueeze(4)
    G = G + g_u[:, :, :, 1].unsqueeze(4) / W2
    G = G + (iu == amv).to(g_u.dtype) * g_v[:, :, :, 0].unsqueeze(3)
    G = G + g_v[:, :, :, 1].unsqueeze(3) / H2
    return G


def grads_from_volume_grad(f1, f2, G):
    """dF1 = sum_{u,v} G f2,  dF2 = sum_{i,j} G f1  (argmax_backward.cu:200-251, 253-291)."""
    B, H1, W1, C = f1.shape
    _, H2, W2, _ = f2.shape
    Gm = G.reshape(B, H1 * W1, H2 * W2)
    d1 = torch.matmul(Gm, f2.reshape(B, H2 * W2, C)).reshape(B, H1, W1, C)
    d2 = torch.matmul(Gm.transpose(1, 2), f1.reshape(B, H1 * W1, C)).reshape(B, H2, W2, C)
    return d1, d2


def max_argmax_avg_backward(f1, f2, am_u, am_v, g_u, g_v):
    """ComputeMaxArgmaxAvgFunction.backward (functions/MemorySaver.py:70-105)."""
    G = max_argmax_avg_grad_volume(am_u, am_v, g_u, g_v, f2.shape[1], f2.shape[2])
    return grads_from_volume_grad(f1, f2, G)


def compression_backward(f1, f2, a_u, a_v, g_cu, g_cv):
    """ComputeSelfCompressionFunction.backward (functions/MemorySaver.py:139-177).

    Follows MemorySaver_kernel_compression_backward.cu:464-502:
      G = sum_k a_u[k,v] g_cu[k,u] + a_v[k,u] g_cv[k,v]
      da_u[k,v] = sum_u S g_cu[k,u];  da_v[k,u] = sum_v S g_cv[k,v]
    """
    s = corr_volume(f1, f2)
    G = torch.einsum('bijkv,bijku->bijuv', a_u, g_cu) + torch.einsum('bijku,bijkv->bijuv', a_v, g_cv)
    d1, d2 = grads_from_volume_grad(f1, f2, G)
    da_u = torch.einsum('bijuv,bijku->bijkv', s, g_cu)
    da_v = torch.einsum('bijuv,bijkv->bijku', s, g_cv)
    return d1, d2, da_u, da_v


def compression_from_logits(f1, f2, z_u, z_v):
    """The caller's softmax over the kept axis followed by the compression operator (core/corr.py:441-448):
    logits z_u (B,H1,W1,K,W2), z_v (B,H1,W1,K,H2) -> (comp_u (B,H1,W1,K,H2), comp_v (B,H1,W1,K,W2)).  In the
    operator's layout the kept axis is the last one.  Differentiable: torch autograd supplies the gradients of the
    features and of the logits that the fused operator is compared with."""
    return compression_forward(f1, f2, z_u.softmax(dim=-1), z_v.softmax(dim=-1))


def attention_logits(sep, weight, bias):
    """attention_weights without the softmax: the Conv3d output in the operator's layout (B,H1,W1,K,L)."""
    x = sep.permute(0, 3, 4, 1, 2)
    return F.conv3d(x, weight, bias, padding=1).permute(0, 3, 4, 1, 2).contiguous()


def attention_weights(sep, weight, bias):
    """The caller's attention-weight producer, op-level layout in and out.

    Follows core/corr.py:428-429 and 437-446 with core/sepflow.py:59-60: the (B,H1,W1,2,L) max/avg output is
    permuted to (B,2,L,H1,W1), passed through Conv3d(2,K,3,padding=1), softmax over dim 2 (L), and permuted
    back to (B,H1,W1,K,L).  Library routines only (conv3d is a cross-correlation).
    """
    vol = sep.permute(0, 3, 4, 1, 2)
    return F.conv3d(vol, weight, bias, padding=1).softmax(dim=2).permute(0, 3, 4, 1, 2).contiguous()


# --------------------------------------------------------------------------
# autograd through the stored 4D volume (what the reference's tests compare with)
# --------------------------------------------------------------------------

def autograd_max_avg(f1, f2, g_u, g_v):
    """Gradients of <out_u,g_u>+<out_v,g_v> by autograd through the 4D volume.

    Mirrors get_overall_grad_fullMem (scripts/test_maxavg_autograd.py:425-440)
    with a linear loss so that arbitrary upstream grads can be supplied.
    """
    f1 = f1.clone().requires_grad_(True)
    f2 = f2.clone().requires_grad_(True)
    s = corr_volume(f1, f2)
    max_u, _ = s.max(dim=4)
    max_v, _ = s.max(dim=3)
    out_u = torch.stack((max_u, s.mean(dim=4)), dim=3)
    out_v = torch.stack((max_v, s.mean(dim=3)), dim=3)
    ((out_u * g_u).sum() + (out_v * g_v).sum()).backward()
    return f1.grad, f2.grad


def autograd_compression(f1, f2, a_u, a_v, g_cu, g_cv):
    """Same for the compression op (scripts/test_compression_autograd.py:404-429)."""
    f1 = f1.clone().requires_grad_(True)
    f2 = f2.clone().requires_grad_(True)
    a_u = a_u.clone().requires_grad_(True)
    a_v = a_v.clone().requires_grad_(True)
    cu, cv = compression_forward(f1, f2, a_u, a_v)
    ((cu * g_cu).sum() + (cv * g_cv).sum()).backward()
    return f1.grad, f2.grad, a_u.grad, a_v.grad


# --------------------------------------------------------------------------
# brute-force loops for tiny inputs (scripts/test_maxavg_autograd.py:25-220,
# scripts/test_compression_autograd.py:27-135)
# --------------------------------------------------------------------------

def loops_forward(f1, f2, a_u=None, a_v=None):
    """Five nested Python loops; returns dict of op-level outputs.  Tiny inputs only."""
    B, H1, W1, C = f1.shape
    _, H2, W2, _ = f2.shape
    out_u = torch.zeros(B, H1, W1, 2, H2, dtype=f1.dtype)
    out_v = torch.zeros(B, H1, W1, 2, W2, dtype=f1.dtype)
    out_u[:, :, :, 0] = -math.inf
    out_v[:, :, :, 0] = -math.inf
    am_u = torch.zeros(B, H1, W1, 1, H2, dtype=torch.int32)
    am_v = torch.zeros(B, H1, W1, 1, W2, dtype=torch.int32)
    K = 0 if a_u is None else a_u.shape[3]
    cu = torch.zeros(B, H1, W1, K, H2, dtype=f1.dtype)
    cv = torch.zeros(B, H1, W1, K, W2, dtype=f1.dtype)
    for b in range(B):
        for i in range(H1):
            for j in range(W1):
                for u in range(H2):
                    for v in range(W2):
                        c = float(torch.dot(f1[b, i, j], f2[b, u, v]))
                        if c > out_u[b, i, j, 0, u]:
                            out_u[b, i, j, 0, u] = c
                            am_u[b, i, j, 0, u] = v
                        if c > out_v[b, i, j, 0, v]:
                            out_v[b, i, j, 0, v] = c
                            am_v[b, i, j, 0, v] = u
                        out_u[b, i, j, 1, u] += c / W2
                        out_v[b, i, j, 1, v] += c / H2
                        for k in range(K):
                            cu[b, i, j, k, u] += c * a_u[b, i, j, k, v]
                            cv[b, i, j, k, v] += c * a_v[b, i, j, k, u]
    return dict(out_u=out_u, out_v=out_v, am_u=am_u, am_v=am_v, cu=cu, cv=cv)


# --------------------------------------------------------------------------
# module level: the reference's full-4D CorrBlock, separate() only
# --------------------------------------------------------------------------

class CorrBlock4D:
    """Restatement of CorrBlock.__init__/corr_compute/separate (core/corr.py:19-165, 251-302).

    NCHW fmaps in, (corr1 (B,K*L,W,H1,W1), corr2 (B,K*L,H,H1,W1)) out.  `lookup`
    restates __call__ with coords (core/corr.py:193-248); NLF aggregation is not
    part of the path.
    """

    def __init__(self, fmap1, fmap2, num_levels=4):
        B, C, H, W = fmap1.shape
        # core/corr.py:275-283: matmul(fmap2^T, fmap1)/sqrt(C) -> (B,h2,w2,h1,w1) -> permute
        corr = torch.matmul(fmap2.reshape(B, C, H * W).transpose(1, 2), fmap1.reshape(B, C, H * W))
        corr = corr / torch.sqrt(torch.tensor(C).float()).to(fmap1.dtype)
        corr = corr.view(B, H, W, H, W).permute(0, 3, 4, 1, 2)
        self.shape = corr.shape
        corr = corr.reshape(B * H * W, 1, H, W)
        self.pyramid = [corr]
        for _ in range(num_levels - 1):
            corr = F.avg_pool2d(corr, 2, stride=2)
            self.pyramid.append(corr)

    def separate(self, attention_weights=None, argmax=None):
        """`argmax` (optional, tests of near-ties): per level a pair (argmax_u (B,h1,w1,1,hl), argmax_v (B,h1,w1,1,wl))
        in the operator's convention; the maxima are then read at these positions instead of being searched, so that
        the gradient of a maximum flows to the entry the checked implementation selected.  The caller verifies that
        every given index attains the true maximum to within rounding (tests/_util.py:check_argmax)."""
        B, h1, w1, h2, w2 = self.shape
        us, vs = [], []
        for lvl, corr in enumerate(self.pyramid):
            hl, wl = corr.shape[2], corr.shape[3]
            s = corr.reshape(B, h1, w1, hl, wl)
            if argmax is None:
                max_over_u, max_over_v = s.max(dim=3)[0], s.max(dim=4)[0]
            else:
                am_u, am_v = argmax[lvl]
                max_over_v = torch.gather(s, 4, am_u[:, :, :, 0, :, None].long()).squeeze(4)
                max_over_u = torch.gather(s, 3, am_v[:, :, :, 0, None, :].long()).squeeze(3)
            # core/corr.py:77-91: reduce over dim=2 (rows u) -> keeps v: sep_u (B,2,wl,h1,w1)
            sep_u = torch.stack((max_over_u, s.mean(dim=3)), dim=1).permute(0, 1, 4, 2, 3)
            # core/corr.py:96-102: reduce over columns v -> keeps u: sep_v (B,2,hl,h1,w1)
            sep_v = torch.stack((max_over_v, s.mean(dim=4)), dim=1).permute(0, 1, 4, 2, 3)
            if attention_weights is not None:
                att1, att2 = attention_weights
                a_u = att1(sep_u).softmax(dim=2)          # (B,K',wl,h1,w1)  core/corr.py:116-122
                a_v = att2(sep_v).softmax(dim=2)          # (B,K',hl,h1,w1)  core/corr.py:131-134
                ad_u = torch.einsum('bkvij,bijuv->bkuij', a_u, s)   # core/corr.py:128
                ad_v = torch.einsum('bkuij,bijuv->bkvij', a_v, s)   # core/corr.py:140
                sep_v = torch.cat((sep_v, ad_u), dim=1)             # core/corr.py:143
                sep_u = torch.cat((sep_u, ad_v), dim=1)             # core/corr.py:145
            us.append(F.interpolate(sep_u, [w2, h1, w1], mode='trilinear', align_corners=True))
            vs.append(F.interpolate(sep_v, [h2, h1, w1], mode='trilinear', align_corners=True))
        return torch.cat(us, dim=1), torch.cat(vs, dim=1)


    def lookup(self, coords, radius=4):
        """Windowed bilinear lookup in every pyramid level (core/corr.py:193-248).

        coords (B,2,h1,w1): channel 0 = x (fmap2 column), channel 1 = y (fmap2 row),
        in level-0 pixels.  Returns (B, levels*(2r+1)^2, h1, w1); within a level the
        channel index is a*(2r+1)+b and samples (x/2^l + a - r, y/2^l + b - r): the
        x offset runs with the *first* window index, because the reference stacks
        meshgrid(dy, dx) onto (x, y) coordinates (core/corr.py:213, 226).  Sampling is
        grid_sample(bilinear, align_corners=True, zero padding) on pixel coordinates
        normalised as core/utils/utils.py:110-118.
        """
        r = radius
        B, h1, w1, _, _ = self.shape
        coords = coords.permute(0, 2, 3, 1)
        d = torch.linspace(-r, r, 2 * r + 1, dtype=coords.dtype)
        delta = torch.stack(torch.meshgrid(d, d, indexing='ij'), dim=-1).view(1, 2 * r + 1, 2 * r + 1, 2)
        out = []
        for i, corr in enumerate(self.pyramid):
            H, W = corr.shape[-2:]
            c = coords.reshape(B * h1 * w1, 1, 1, 2) / 2 ** i + delta
            xg = 2 * c[..., 0:1] / (W - 1) - 1
            yg = 2 * c[..., 1:2] / (H - 1) - 1
            smp = F.grid_sample(corr, torch.cat([xg, yg], dim=-1), mode='bilinear', padding_mode='zeros',
                                align_corners=True)
            out.append(smp.view(B, h1, w1, -1))
        return torch.cat(out, dim=-1).permute(0, 3, 1, 2).contiguous()


def lookup_direct(fmap1, fmap2, coords, num_levels=4, radius=4):
    """The same lookup from its definition, without a 4D volume and without grid_sample.

    Bilinear sampling is linear in the sampled image and the level-l volume is
    S(f1, avgpool^l f2) (pooling commutes with the contraction), so every sample is
    <fmap1[:,i,j], bilinear(avgpool^l fmap2)(x, y)> / sqrt(C) with corners outside the
    image counted as zero.  Independent of `CorrBlock4D.lookup` in everything but the
    definition; the two are compared in tests/test_oracle.py.
    """
    B, C, h1, w1 = fmap1.shape
    r = radius
    n = 2 * r + 1
    f1 = fmap1.permute(0, 2, 3, 1)                                 # (B,h1,w1,C)
    x = coords[:, 0]
    y = coords[:, 1]
    off = torch.arange(-r, r + 1, dtype=coords.dtype)
    outs = []
    f2 = fmap2
    for lvl in range(num_levels):
        if lvl:
            f2 = F.avg_pool2d(f2, 2, stride=2)
        H, W = f2.shape[-2:]
        f2n = f2.permute(0, 2, 3, 1)                               # (B,H,W,C)
        xs = (x / 2 ** lvl)[..., None, None] + off.view(1, 1, 1, n, 1)   # (B,h1,w1,a,1): x moves with a
        ys = (y / 2 ** lvl)[..., None, None] + off.view(1, 1, 1, 1, n)   # (B,h1,w1,1,b): y moves with b
        xs, ys = torch.broadcast_tensors(xs, ys)
        x0 = torch.floor(xs)
        y0 = torch.floor(ys)
        fx = xs - x0
        fy = ys - y0
        acc = torch.zeros(B, h1, w1, n, n, dtype=fmap1.dtype)
        bidx = torch.arange(B).view(B, 1, 1, 1, 1).expand_as(x0)
        for dy, wy in ((0, 1 - fy), (1, fy)):
            for dx, wx in ((0, 1 - fx), (1, fx)):
                xi = (x0 + dx).long()
                yi = (y0 + dy).long()
                ok = (xi >= 0) & (xi < W) & (yi >= 0) & (yi < H)
                g = f2n[bidx, yi.clamp(0, H - 1), xi.clamp(0, W - 1)]          # (B,h1,w1,n,n,C)
                dot = (g * f1[:, :, :, None, None, :]).sum(-1)
                acc = acc + torch.where(ok, wx * wy * dot, torch.zeros_like(dot))
        outs.append(acc.reshape(B, h1, w1, n * n))
    # the reference divides by the fp32 square root (core/corr.py:282, 509)
    out = torch.cat(outs, dim=-1) / torch.sqrt(torch.tensor(C).float()).to(fmap1.dtype)
    return out.permute(0, 3, 1, 2).contiguous()


class CorrBlock1D:
    """Restatement of the reference's CorrBlock1D (core/corr.py:513-624): lookup in the two 3D volumes.

    corr1 (B,dim,W2,H1,W1) and corr2 (B,dim,H2,H1,W1) are pooled by two along the displacement axis into a pyramid
    (avg_pool2d [1,2], core/corr.py:546-550); every level is sampled with grid_sample (bilinear, align_corners=True,
    zero padding) at coords/2^l + dx, dx = -r..r.  coords channel 0 addresses corr1, channel 1 corr2.  For corr1 the
    reference clamps the *pixel* positions to [-1, 1] before sampling (core/corr.py:593); that is kept.
    Output channel = level*dim*(2r+1) + d*(2r+1) + k.
    """

    def __init__(self, corr1, corr2, num_levels=4, radius=4):
        self.num_levels, self.radius = num_levels, radius
        self.pyr = []
        for corr in (corr1, corr2):
            c = corr.permute(0, 3, 4, 1, 2)
            b, h1, w1, dim, L = c.shape
            c = c.reshape(b * h1 * w1, dim, 1, L)
            levels = [c]
            for _ in range(num_levels):
                c = F.avg_pool2d(c, [1, 2], stride=[1, 2])
                levels.append(c)
            self.pyr.append(levels)

    def __call__(self, coords):
        r = self.radius
        B, _, h1, w1 = coords.shape
        outs = []
        for which in (0, 1):
            x = coords[:, which:which + 1].permute(0, 2, 3, 1).reshape(B * h1 * w1, 1, 1, 1)
            per_level = []
            for i in range(self.num_levels):
                corr = self.pyr[which][i]
                W = corr.shape[-1]
                dx = torch.linspace(-r, r, 2 * r + 1, dtype=coords.dtype).view(1, 1, 2 * r + 1, 1)
                x0 = dx + x / 2 ** i
                y0 = torch.zeros_like(x0)
                if which == 0:
                    x0 = torch.clamp(x0, -1, 1)                       # core/corr.py:593
                grid = torch.cat([2 * x0 / (W - 1) - 1, y0], dim=-1)   # core/corr.py:555-560: y is not normalised
                smp = F.grid_sample(corr, grid, mode='bilinear', padding_mode='zeros', align_corners=True)
                per_level.append(smp.view(B, h1, w1, -1))
            outs.append(torch.cat(per_level, dim=-1).permute(0, 3, 1, 2).contiguous())
        return outs[0], outs[1]


def lookup1d_direct(corr, x, num_levels=4, radius=4, clamp_unit=False):
    """One volume of the above from its definition: explicit pair means for the pyramid, explicit linear weights.

    corr (B,dim,L,H1,W1), x (B,H1,W1) -> (B, levels*dim*(2r+1), H1, W1).  Independent of CorrBlock1D in everything
    but the definition (no avg_pool2d, no grid_sample).
    """
    B, dim, L, h1, w1 = corr.shape
    r = radius
    outs = []
    lvl = corr
    for i in range(num_levels):
        if i:
            n = lvl.shape[2] // 2
            lvl = 0.5 * (lvl[:, :, 0:2 * n:2] + lvl[:, :, 1:2 * n:2])
        Li = lvl.shape[2]
        vals = []
        for k in range(2 * r + 1):
            pos = x / 2 ** i + (k - r)
            if clamp_unit:
                pos = pos.clamp(-1, 1)
            p0 = torch.floor(pos)
            f = (pos - p0)[:, None]
            acc = torch.zeros(B, dim, h1, w1, dtype=corr.dtype)
            for d, wgt in ((0, 1 - f), (1, f)):
                idx = (p0 + d).long()
                ok = ((idx >= 0) & (idx < Li))[:, None]
                g = torch.gather(lvl, 2, idx.clamp(0, Li - 1)[:, None, None].expand(B, dim, 1, h1, w1))[:, :, 0]
                acc = acc + torch.where(ok, wgt * g, torch.zeros_like(g))
            vals.append(acc)
        outs.append(torch.stack(vals, dim=2).reshape(B, dim * (2 * r + 1), h1, w1))
    return torch.cat(outs, dim=1)


def make_inputs(B, H, W, C, seed=1234, dtype=torch.float32):
    """Seeded N(0,1) NCHW fmaps and the NHWC op inputs derived as core/corr.py:419-422."""
    g = torch.Generator().manual_seed(seed)
    fmap1 = torch.randn(B, C, H, W, generator=g, dtype=dtype)
    fmap2 = torch.randn(B, C, H, W, generator=g, dtype=dtype)
    f1 = fmap1.permute(0, 2, 3, 1).contiguous() / torch.sqrt(torch.tensor(C).float()).to(dtype)
    f2 = fmap2.permute(0, 2, 3, 1).contiguous()
    return fmap1, fmap2, f1, f2
