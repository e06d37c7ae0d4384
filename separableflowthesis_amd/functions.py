"""The three autograd Functions of the reference's libs/MemorySaver/functions/MemorySaver.py.

Same class names, argument order, outputs, layouts and saved-tensor order, so that
core/corr.py:425 (`.apply(fmap1, fmap2)`) and :448 (`.apply(fmap1, fmap2, a_u, a_v)`) work
unchanged.  `backward` may also be called directly with an object exposing `saved_tensors`,
as the reference's debug helpers do (scripts/test_maxavg_autograd.py:560-562).
"""
import torch
from torch.autograd import Function

from . import MemorySaver


def _contig(*ts):
    assert all(bool(t.is_contiguous()) for t in ts), "inputs must be contiguous"


class ComputeMaxAvgFunction(Function):
    """Max and mean of the 4D correlation volume over each displacement axis; forward only.

    Mirrors functions/MemorySaver.py:6-38.
    """

    @staticmethod
    def forward(ctx, img1_features_l0, img2_features_lk):
        _contig(img1_features_l0, img2_features_lk)
        with torch.cuda.device_of(img1_features_l0):
            out_u, out_v = MemorySaver.max_avg_forward(img1_features_l0, img2_features_lk)
        return out_u.contiguous(), out_v.contiguous()

    @staticmethod
    def backward(ctx, gradOutput_u, gradOutput_v):
        raise NotImplementedError("max avg backward pass is not implemented: use max argmax avg")


class ComputeMaxArgmaxAvgFunction(Function):
    """As above, with argmax saved so that the backward pass exists (functions/MemorySaver.py:40-105)."""

    @staticmethod
    def forward(ctx, img1_features_l0, img2_features_lk):
        _contig(img1_features_l0, img2_features_lk)
        with torch.cuda.device_of(img1_features_l0):
            out_u, out_v, am_u, am_v = MemorySaver.max_argmax_avg_forward(img1_features_l0, img2_features_lk)
        ctx.save_for_backward(img1_features_l0, img2_features_lk, am_u, am_v)
        return out_u.contiguous(), out_v.contiguous()

    @staticmethod
    def backward(ctx, grad_MaxAvg_u, grad_MaxAvg_v):
        f1, f2, am_u, am_v = ctx.saved_tensors
        grad_MaxAvg_u = grad_MaxAvg_u.contiguous()
        grad_MaxAvg_v = grad_MaxAvg_v.contiguous()
        _contig(f1, f2, am_u, am_v)
        with torch.cuda.device_of(grad_MaxAvg_u):
            d1, d2 = MemorySaver.max_argmax_avg_backward(f1, f2, am_u, am_v, grad_MaxAvg_u, grad_MaxAvg_v)
        return d1.contiguous(), d2.contiguous()


class ComputeSelfCompressionFunction(Function):
    """Attention-weighted sums of the 4D volume (functions/MemorySaver.py:107-177), any K."""

    @staticmethod
    def forward(ctx, img1_features_l0, img2_features_lk, attention_weights_u, attention_weights_v):
        _contig(img1_features_l0, img2_features_lk, attention_weights_u, attention_weights_v)
        with torch.cuda.device_of(img1_features_l0):
            cu, cv = MemorySaver.compression_forward(img1_features_l0, img2_features_lk,
                                                     attention_weights_u, attention_weights_v)
        ctx.save_for_backward(img1_features_l0, img2_features_lk, attention_weights_u, attention_weights_v)
        return cu.contiguous(), cv.contiguous()

    @staticmethod
    def backward(ctx, grad_compressed_output_u, grad_compressed_output_v):
        f1, f2, a_u, a_v = ctx.saved_tensors
        grad_compressed_output_u = grad_compressed_output_u.contiguous()
        grad_compressed_output_v = grad_compressed_output_v.contiguous()
        _contig(f1, f2, a_u, a_v)
        with torch.cuda.device_of(grad_compressed_output_u):
            d1, d2, da_u, da_v = MemorySaver.compression_backward(
                f1, f2, a_u, a_v, grad_compressed_output_u, grad_compressed_output_v)
        return d1.contiguous(), d2.contiguous(), da_u.contiguous(), da_v.contiguous()


class ComputeSelfCompressionFromLogitsFunction(Function):
    """ComputeSelfCompressionFunction with the softmax inside: apply(fmap1, fmap2, logits_u, logits_v) equals
    ComputeSelfCompressionFunction.apply(fmap1, fmap2, logits_u.softmax(-1), logits_v.softmax(-1)) in values and
    gradients (core/corr.py:441-448, functions/MemorySaver.py:107-177).  Not a class of the reference.

    Saved for backward: the logits, their row statistics (max, sum of exp) and the outputs; no tensor of softmax
    outputs or of their gradients exists in either direction.
    """

    @staticmethod
    def forward(ctx, img1_features_l0, img2_features_lk, logits_u, logits_v, stats_u=None, stats_v=None):
        """stats_u, stats_v (optional): row statistics (max, sum of exp) of the logits, as AttentionLogitsFunction
        returns them; computed here when absent."""
        _contig(img1_features_l0, img2_features_lk, logits_u, logits_v)
        with torch.cuda.device_of(img1_features_l0):
            cu, cv, st_u, st_v = MemorySaver.compression_forward_from_logits(img1_features_l0, img2_features_lk,
                                                                             logits_u, logits_v, stats_u, stats_v)
        ctx.save_for_backward(img1_features_l0, img2_features_lk, logits_u, logits_v, st_u, st_v, cu, cv)
        return cu, cv

    @staticmethod
    def backward(ctx, grad_compressed_output_u, grad_compressed_output_v):
        f1, f2, z_u, z_v, st_u, st_v, cu, cv = ctx.saved_tensors
        with torch.cuda.device_of(f1):
            d1, d2, dz_u, dz_v = MemorySaver.compression_backward_from_logits(
                f1, f2, z_u, z_v, st_u, st_v, cu, cv,
                grad_compressed_output_u.contiguous(), grad_compressed_output_v.contiguous())
        return d1, d2, dz_u, dz_v, None, None


class AttentionLogitsFunction(Function):
    """Conv3d(2 -> K, 3, padding=1) of a max/avg volume in the operator's layout: the attention module's output
    before the softmax (core/corr.py:441-442 applies softmax(dim=2) to it).  Not a class of the reference.
    -> (logits (B,H1,W1,K,L), stats (B,H1,W1,K,2)); stats = per row (max, sum of exp), a by-product without gradient
    that ComputeSelfCompressionFromLogitsFunction takes."""

    @staticmethod
    def forward(ctx, sep, weight, bias):
        _contig(sep, weight)
        z, st = MemorySaver.attention_logits_forward(sep, weight, bias)
        ctx.save_for_backward(sep, weight)
        ctx.has_bias = bias is not None
        ctx.mark_non_differentiable(st)
        return z, st

    @staticmethod
    def backward(ctx, grad_z, _grad_stats=None):
        sep, weight = ctx.saved_tensors
        d_sep, d_w, d_b = MemorySaver.attention_logits_backward(sep, weight, grad_z.contiguous(), need_bias=ctx.has_bias)
        return d_sep, d_w, d_b


class AttentionWeightsFunction(Function):
    """softmax over L of Conv3d(2 -> K, 3, padding=1) of a max/avg volume, in the operator's layout.

    Not a class of the reference: it stands for the torch ops the caller runs between the two operators
    (core/corr.py:437-446: attention(sep).softmax(dim=2) wrapped in two permutes), with the same result.
    """

    @staticmethod
    def forward(ctx, sep, weight, bias):
        _contig(sep, weight)
        a = MemorySaver.attention_forward(sep, weight, bias)
        ctx.save_for_backward(sep, weight, a)
        ctx.has_bias = bias is not None
        return a

    @staticmethod
    def backward(ctx, grad_a):
        sep, weight, a = ctx.saved_tensors
        d_sep, d_w, d_b = MemorySaver.attention_backward(sep, weight, a, grad_a.contiguous(), need_bias=ctx.has_bias)
        return d_sep, d_w, d_b


class SeparateLevelFunction(Function):
    """One pyramid level of the caller's loop (core/corr.py:416-457) as a single autograd node:
    max/argmax/avg forward -> attention logits of both volumes -> compression forward from the logits.

    Not a class of the reference.  Results equal the chain ComputeMaxArgmaxAvgFunction ->
    AttentionWeightsFunction x2 -> ComputeSelfCompressionFunction; the point is the backward pass: the
    gradient of the max/avg outputs is complete before any feature gradient is needed, so dL/dS of both
    operators is added and contracted once (3 sweeps over the volume instead of 5).

    forward(f1, f2, weight1, bias1, weight2, bias2) -> (max_avg_u, max_avg_v, comp_u, comp_v), operator layouts;
    attention 1 reads max_avg_v and weights the sums over v, attention 2 reads max_avg_u (core/corr.py:437-448).
    """

    @staticmethod
    def forward(ctx, f1, f2, weight1, bias1, weight2, bias2):
        _contig(f1, f2, weight1, weight2)
        with torch.cuda.device_of(f1):
            out_u, out_v, am_u, am_v = MemorySaver.max_argmax_avg_forward(f1, f2)
            # the attention modules stop at the logits (and hand over the row statistics of their softmax, which
            # they have at hand); the softmax itself happens where the compression sweep loads its weights
            z_u, st_u = MemorySaver.attention_logits_forward(out_v, weight1, bias1)
            z_v, st_v = MemorySaver.attention_logits_forward(out_u, weight2, bias2)
            cu, cv, _, _ = MemorySaver.compression_forward_from_logits(f1, f2, z_u, z_v, st_u, st_v)
        ctx.save_for_backward(f1, f2, am_u, am_v, out_u, out_v, z_u, z_v, st_u, st_v, cu, cv, weight1, weight2)
        ctx.has_bias = (bias1 is not None, bias2 is not None)
        return out_u, out_v, cu, cv

    @staticmethod
    def backward(ctx, g_u, g_v, g_cu, g_cv):
        f1, f2, am_u, am_v, out_u, out_v, z_u, z_v, st_u, st_v, cu, cv, weight1, weight2 = ctx.saved_tensors
        g_u, g_v, g_cu, g_cv = (g.contiguous() for g in (g_u, g_v, g_cu, g_cv))
        with torch.cuda.device_of(f1):
            # gradients of the logits straight from the weight-gradient sweep (no d_a tensors, no softmax backward)
            _, _, dz_u, dz_v = MemorySaver.compression_backward_from_logits(f1, f2, z_u, z_v, st_u, st_v, cu, cv, g_cu, g_cv,
                                                                            need_features=False)
            d_out_v, d_w1, d_b1 = MemorySaver.attention_logits_backward(out_v, weight1, dz_u, need_bias=ctx.has_bias[0])
            d_out_u, d_w2, d_b2 = MemorySaver.attention_logits_backward(out_u, weight2, dz_v, need_bias=ctx.has_bias[1])
            del dz_u, dz_v
            d_out_u += g_u
            d_out_v += g_v
            # the combined feature-gradient contraction reads the weights themselves: formed here from the saved
            # statistics, for the duration of this call only
            a_u = MemorySaver.softmax_from_stats(z_u, st_u)
            a_v = MemorySaver.softmax_from_stats(z_v, st_v)
            d1, d2 = MemorySaver.fused_backward(f1, f2, am_u, am_v, d_out_u, d_out_v, a_u, a_v, g_cu, g_cv)
        return d1, d2, d_w1, d_b1, d_w2, d_b2


class SeparatePyramidFunction(Function):
    """All pyramid levels of the caller's loop (core/corr.py:416-457) as one autograd node; per level the same results
    as SeparateLevelFunction.  The forward-type sweeps of several levels share one launch where the shapes allow
    (MemorySaver.*_levels): the small levels then fill the chip together instead of one after the other.

    apply(f1, weight1, bias1, weight2, bias2, first_alone, *f2_levels)
      -> (max_avg_u_0, max_avg_v_0, comp_u_0, comp_v_0, max_avg_u_1, ...), operator layouts.
    first_alone: level 0 keeps launches of its own (the kernels without row groups, which wide rows run fastest in)
    and only the levels above it share launches.  Not a class of the reference.
    """

    @staticmethod
    def forward(ctx, f1, weight1, bias1, weight2, bias2, first_alone, *f2_levels):
        lv = list(f2_levels)
        _contig(f1, weight1, weight2, *lv)
        n = len(lv)
        split = 1 if (first_alone and n > 1) else 0
        with torch.cuda.device_of(f1):
            ma = [MemorySaver.max_argmax_avg_forward(f1, lv[0])] if split else []
            ma += MemorySaver.max_argmax_avg_forward_levels(f1, lv[split:])
            out_u, out_v, am_u, am_v = (list(t) for t in zip(*ma))
            # each attention module on the volumes of all levels in shared launches
            z_u, st_u = MemorySaver.attention_logits_forward_levels(out_v, weight1, bias1)
            z_v, st_v = MemorySaver.attention_logits_forward_levels(out_u, weight2, bias2)
            comp = [MemorySaver.compression_forward_from_logits(f1, lv[0], z_u[0], z_v[0], st_u[0], st_v[0])[:2]] if split else []
            comp += MemorySaver.compression_forward_from_logits_levels(f1, lv[split:], z_u[split:], z_v[split:],
                                                                       st_u[split:], st_v[split:])
            cu, cv = (list(t) for t in zip(*comp))
        ctx.save_for_backward(f1, weight1, weight2, *lv, *am_u, *am_v, *out_u, *out_v, *z_u, *z_v, *st_u, *st_v, *cu, *cv)
        ctx.n, ctx.split = n, split
        ctx.has_bias = (bias1 is not None, bias2 is not None)
        out = []
        for l in range(n):
            out += [out_u[l], out_v[l], cu[l], cv[l]]
        return tuple(out)

    @staticmethod
    def backward(ctx, *grads):
        n, split = ctx.n, ctx.split
        saved = ctx.saved_tensors
        f1, weight1, weight2 = saved[:3]
        groups = [list(saved[3 + i * n: 3 + (i + 1) * n]) for i in range(11)]
        lv, am_u, am_v, out_u, out_v, z_u, z_v, st_u, st_v, cu, cv = groups
        g_u = [grads[4 * l].contiguous() for l in range(n)]
        g_v = [grads[4 * l + 1].contiguous() for l in range(n)]
        g_cu = [grads[4 * l + 2].contiguous() for l in range(n)]
        g_cv = [grads[4 * l + 3].contiguous() for l in range(n)]
        with torch.cuda.device_of(f1):
            dz = []
            if split:
                dz.append(MemorySaver.compression_backward_from_logits(f1, lv[0], z_u[0], z_v[0], st_u[0], st_v[0], cu[0], cv[0],
                                                                       g_cu[0], g_cv[0], need_features=False)[2:])
            dz += MemorySaver.compression_logit_gradients_levels(f1, lv[split:], z_u[split:], z_v[split:], st_u[split:],
                                                                 st_v[split:], cu[split:], cv[split:], g_cu[split:], g_cv[split:])
            # both attention modules backwards over all levels in shared launches: weight and bias gradients come out
            # summed over the levels, the gradients of the max/avg volumes with the upstream ones already added
            d_out_v, d_w1, d_b1 = MemorySaver.attention_logits_backward_levels(out_v, weight1, [z[0] for z in dz], g_v,
                                                                               need_bias=ctx.has_bias[0])
            d_out_u, d_w2, d_b2 = MemorySaver.attention_logits_backward_levels(out_u, weight2, [z[1] for z in dz], g_u,
                                                                               need_bias=ctx.has_bias[1])
            del dz   # (157 MiB at B=2, 55x128, K=4: not needed by the feature-gradient kernels below)
            d_f1 = None
            d_f2 = []
            for l in range(n):
                a_u = MemorySaver.softmax_from_stats(z_u[l], st_u[l])
                a_v = MemorySaver.softmax_from_stats(z_v[l], st_v[l])
                # (the gradient of fmap1 is the sum over the levels: every level after the first adds to the same tensor)
                d_f1, d2 = MemorySaver.fused_backward(f1, lv[l], am_u[l], am_v[l], d_out_u[l], d_out_v[l], a_u, a_v, g_cu[l], g_cv[l],
                                                      add_to_grad_fmap1=d_f1)
                d_f2.append(d2)
        return (d_f1, d_w1, d_b1, d_w2, d_b2, None, *d_f2)


class AssembleVolumeFunction(Function):
    """Operator outputs of all levels -> one module-level volume (B, channels, L0, H1, W1).

    Not a class of the reference: it stands for the caller's permute / cat / trilinear interpolate / cat
    chain (core/corr.py:428-429, 451-475) with the same result.
    """

    @staticmethod
    def forward(ctx, L0, *srcs):
        _contig(*srcs)
        ctx.shapes = [tuple(t.shape) for t in srcs]
        return MemorySaver.assemble_forward(srcs, L0)

    @staticmethod
    def backward(ctx, grad):
        return (None,) + tuple(MemorySaver.assemble_backward(grad.contiguous(), ctx.shapes))


class FeaturePyramidFunction(Function):
    """A (B,C,H,W) feature map -> its levels in the operator's layout: apply(fmap, num_levels, divisor) returns
    num_levels tensors, level l in (B, H >> l, W >> l, C); level 0 = fmap.permute(0,2,3,1) / divisor, level l =
    F.avg_pool2d of level l - 1 (2, stride 2).

    Not a class of the reference: it stands for the pooling chain of the block's constructor and the
    permute(0,2,3,1).contiguous() (/ sqrt(fdim)) in front of every operator call (core/corr.py:376-382, 419-422),
    one kernel per direction instead of 2 to 8 torch kernels.
    """

    @staticmethod
    def forward(ctx, fmap, num_levels, divisor):
        _contig(fmap)
        ctx.divisor = divisor
        with torch.cuda.device_of(fmap):
            return tuple(MemorySaver.feature_pyramid_forward(fmap, num_levels, divisor))

    @staticmethod
    def backward(ctx, *grads):
        with torch.cuda.device_of(grads[0]):
            return MemorySaver.feature_pyramid_backward([g.contiguous() for g in grads], ctx.divisor), None, None


class LookupFunction(Function):
    """corr_fn(coords) of the block that never stores the 4D volume: windowed bilinear lookup in every pyramid level.

    apply(coords, radius, scale, f1, *f2_levels): f1 (B,H1,W1,C) and the pooled fmap2 levels (B,H2_l,W2_l,C) in NHWC,
    coords (B,2,H1,W1) -> (B, levels*(2*radius+1)^2, H1, W1).  Values as CorrBlock.__call__ (core/corr.py:193-248);
    the reference's own draft of this call raises NotImplementedError (core/corr.py:491-509).  Gradients go to f1 and
    to every level; coords get none (the flow iterations detach them, core/sepflow.py:194).
    """

    @staticmethod
    def forward(ctx, coords, radius, scale, f1, *f2_levels):
        _contig(coords, f1, *f2_levels)
        with torch.cuda.device_of(f1):
            out = MemorySaver.lookup_forward(f1, f2_levels, coords, radius, scale)
        ctx.save_for_backward(coords, f1, *f2_levels)
        ctx.radius, ctx.scale = radius, scale
        return out

    @staticmethod
    def backward(ctx, grad_out):
        coords, f1, *f2_levels = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        with torch.cuda.device_of(grad_out):
            d_f1, d_f2 = MemorySaver.lookup_backward(f1, f2_levels, coords, grad_out, ctx.radius, ctx.scale)
        return (None, None, None, d_f1, *d_f2)


class Lookup1DFunction(Function):
    """Lookup in one separated 3D volume, the reference's CorrBlock1D per volume (core/corr.py:565-624).

    apply(corr, coords, coord_channel, clamp_unit, num_levels, radius): corr (B,dim,L,H1,W1), coords (B,2,H1,W1)
    -> (B, num_levels*dim*(2*radius+1), H1, W1).  The gradient goes to corr; coords get none (the flow iterations
    detach them, core/sepflow.py:194).
    """

    @staticmethod
    def forward(ctx, corr, coords, coord_channel, clamp_unit, num_levels, radius):
        _contig(corr, coords)
        with torch.cuda.device_of(corr):
            out = MemorySaver.lookup1d_forward(corr, coords, coord_channel, clamp_unit, num_levels, radius)
        ctx.save_for_backward(coords)
        ctx.args = (tuple(corr.shape), coord_channel, clamp_unit, num_levels, radius)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        coords, = ctx.saved_tensors
        shape, coord_channel, clamp_unit, num_levels, radius = ctx.args
        with torch.cuda.device_of(grad_out):
            d = MemorySaver.lookup1d_backward(coords, grad_out.contiguous(), shape, coord_channel, clamp_unit,
                                              num_levels, radius)
        return d, None, None, None, None, None
