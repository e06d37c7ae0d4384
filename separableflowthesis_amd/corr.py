"""Host-side caller of the op: the reference's AlternateCorrBlockSepflow (core/corr.py:335-510).

Builds the two separated 3D correlation volumes over a 4-level fmap2 pyramid without ever
holding the 4D volume.  Behaviour kept from the reference: NLF guidance is refused, the
function class is picked by `support_backward`, outputs are
  corr1 (B, K*levels, W, H1, W1)  and  corr2 (B, K*levels, H, H1, W1),
channel order [max, avg, att_0..] per level, levels concatenated on dim 1, every level
trilinearly upsampled (align_corners=True) to the level-0 displacement length.
"""
import torch
import torch.nn.functional as F

from . import MemorySaver
from .functions import (AssembleVolumeFunction, AttentionLogitsFunction, AttentionWeightsFunction,
                        FeaturePyramidFunction,
                        ComputeMaxArgmaxAvgFunction, ComputeMaxAvgFunction, ComputeSelfCompressionFromLogitsFunction,
                        ComputeSelfCompressionFunction, Lookup1DFunction, LookupFunction, SeparateLevelFunction,
                        SeparatePyramidFunction)


def _is_reference_attention(m):
    """True for the module the reference builds: Conv3d(2, K, 3, padding=1) (core/sepflow.py:59-60)."""
    return (isinstance(m, torch.nn.Conv3d) and m.in_channels == 2 and m.out_channels <= 8
            and tuple(m.kernel_size) == (3, 3, 3) and tuple(m.padding) == (1, 1, 1) and tuple(m.stride) == (1, 1, 1)
            and tuple(m.dilation) == (1, 1, 1) and m.groups == 1 and m.padding_mode == 'zeros'
            and m.weight.dtype == torch.float32)


def produce_attention(sep_oplevel, sep_modlevel, module):
    """a = softmax_L(module(volume)) as (B,H1,W1,K,L): fused kernel for the reference's Conv3d, torch otherwise."""
    if _is_reference_attention(module) and sep_oplevel.is_cuda:
        return AttentionWeightsFunction.apply(sep_oplevel, module.weight.contiguous(), module.bias)
    return module(sep_modlevel).softmax(dim=2).permute(0, 3, 4, 1, 2).contiguous()


class AlternateCorrBlockSepflow:
    def __init__(self, fmap1, fmap2, guid, num_levels=4, radius=4, support_backward=False):
        if guid is not None:
            # core/corr.py:356-358: NLF couples entries of the 4D volume, which is never stored here
            raise Exception("Cannot use NLF while not storing the 4d correlation volume")
        self.max_avg_function = ComputeMaxArgmaxAvgFunction if support_backward else ComputeMaxAvgFunction
        self.num_levels = num_levels
        self.radius = radius
        self.fmap1_l0 = fmap1
        self._lookup_inputs = None
        # how the fused path runs the pyramid: "all" (every level in the same launches; fastest measured), "first_alone"
        # (level 0 in launches of its own, the levels above it together) or "level" (one autograd node per level)
        self.pyramid_mode = "all"
        self.fmap2_l0 = fmap2
        self._pyramid = None

    @property
    def pyramid(self):
        """fmap2 and its 2x2 average poolings in (B,C,H,W) (core/corr.py:376-382); built when first asked for: the
        path that runs all levels in shared launches takes its levels from FeaturePyramidFunction instead."""
        if self._pyramid is None:
            fmap2 = self.fmap2_l0
            self._pyramid = [fmap2]
            for _ in range(self.num_levels - 1):
                fmap2 = F.avg_pool2d(fmap2, 2, stride=2)
                self._pyramid.append(fmap2)
        return self._pyramid

    def separate(self, attention_weights):
        batch, fdim, h1, w1 = self.fmap1_l0.shape
        h2, w2 = h1, w1
        fused = self.fmap1_l0.is_cuda and max(h2, w2) <= 500 and (
            attention_weights is None or all(_is_reference_attention(m) for m in attention_weights))
        parts_u, parts_v = [], []      # operator outputs in final channel order (fused path)
        sep_u_lvls, sep_v_lvls = [], []
        # (the optional bf16-plane contraction exists in the single-level sweeps only: it keeps the per-level path)
        # (without support for the backward pass the same node serves as long as no graph is recorded: the argmax it
        # also computes is simply dropped; with a graph the per-level path keeps the reference's NotImplementedError)
        if (fused and attention_weights is not None
                and (self.max_avg_function is ComputeMaxArgmaxAvgFunction or not torch.is_grad_enabled())
                and 1 < self.num_levels <= 4 and self.pyramid_mode != "level"
                and MemorySaver.set_contraction(-1) == MemorySaver.CONTRACT_FP32):
            # the whole pyramid as one autograd node; the levels above level 0 share launches
            attention1, attention2 = attention_weights
            if (self.fmap1_l0.dtype == torch.float32 and self.fmap2_l0.dtype == torch.float32
                    and min(h2, w2) >> (self.num_levels - 1) >= 1 and batch * ((fdim + 31) // 32) < 65536):
                # layout change, scaling and pooling in one pass per feature map
                (fmap1,) = FeaturePyramidFunction.apply(self.fmap1_l0.contiguous(), 1,
                                                        float(torch.sqrt(torch.tensor(fdim).float())))
                levels = FeaturePyramidFunction.apply(self.fmap2_l0.contiguous(), self.num_levels, 1.0)
            else:
                fmap1 = self.fmap1_l0.permute(0, 2, 3, 1).contiguous() / torch.sqrt(torch.tensor(fdim).float())
                levels = [p.permute(0, 2, 3, 1).contiguous() for p in self.pyramid]
            res = SeparatePyramidFunction.apply(fmap1, attention1.weight.contiguous(), attention1.bias,
                                                attention2.weight.contiguous(), attention2.bias,
                                                self.pyramid_mode == "first_alone", *levels)
            for i in range(self.num_levels):
                maxavg_u, maxavg_v, adaptive_corr_u, adaptive_corr_v = res[4 * i: 4 * i + 4]
                parts_u += [maxavg_v, adaptive_corr_v]
                parts_v += [maxavg_u, adaptive_corr_u]
            return AssembleVolumeFunction.apply(w2, *parts_u), AssembleVolumeFunction.apply(h2, *parts_v)
        # the scaled NHWC copy of fmap1 is level independent; made once (the reference redoes it per level)
        fmap1 = self.fmap1_l0.permute(0, 2, 3, 1).contiguous() / torch.sqrt(torch.tensor(fdim).float())
        for i in range(self.num_levels):
            fmap2 = self.pyramid[i].permute(0, 2, 3, 1).contiguous()
            if fused and attention_weights is not None and self.max_avg_function is ComputeMaxArgmaxAvgFunction:
                # the whole level as one autograd node: its backward contracts dL/dS of both operators once
                attention1, attention2 = attention_weights
                maxavg_u, maxavg_v, adaptive_corr_u, adaptive_corr_v = SeparateLevelFunction.apply(
                    fmap1, fmap2, attention1.weight.contiguous(), attention1.bias,
                    attention2.weight.contiguous(), attention2.bias)
                parts_u += [maxavg_v, adaptive_corr_v]
                parts_v += [maxavg_u, adaptive_corr_u]
                continue
            maxavg_u, maxavg_v = self.max_avg_function.apply(fmap1, fmap2)
            if fused:
                # everything stays in the operator's layout; one kernel per output assembles the result
                parts_u.append(maxavg_v)
                parts_v.append(maxavg_u)
                if attention_weights is not None:
                    attention1, attention2 = attention_weights
                    z_u, st_u = AttentionLogitsFunction.apply(maxavg_v, attention1.weight.contiguous(), attention1.bias)
                    z_v, st_v = AttentionLogitsFunction.apply(maxavg_u, attention2.weight.contiguous(), attention2.bias)
                    adaptive_corr_u, adaptive_corr_v = ComputeSelfCompressionFromLogitsFunction.apply(
                        fmap1, fmap2, z_u, z_v, st_u, st_v)
                    parts_v.append(adaptive_corr_u)
                    parts_u.append(adaptive_corr_v)
                continue
            sep_v = maxavg_u.permute(0, 3, 4, 1, 2).contiguous()   # (B,2,H2_i,h1,w1)
            sep_u = maxavg_v.permute(0, 3, 4, 1, 2).contiguous()   # (B,2,W2_i,h1,w1)
            if attention_weights is not None:
                attention1, attention2 = attention_weights
                # core/corr.py:437-446; sep_u is the permuted maxavg_v, sep_v the permuted maxavg_u
                a_u = produce_attention(maxavg_v, sep_u, attention1)
                a_v = produce_attention(maxavg_u, sep_v, attention2)
                adaptive_corr_u, adaptive_corr_v = ComputeSelfCompressionFunction.apply(fmap1, fmap2, a_u, a_v)
                sep_v = torch.cat((sep_v, adaptive_corr_u.permute(0, 3, 4, 1, 2)), dim=1)
                sep_u = torch.cat((sep_u, adaptive_corr_v.permute(0, 3, 4, 1, 2)), dim=1)
            sep_u_lvls.append(F.interpolate(sep_u, [w2, h1, w1], mode='trilinear', align_corners=True))
            sep_v_lvls.append(F.interpolate(sep_v, [h2, h1, w1], mode='trilinear', align_corners=True))
        if fused:
            return AssembleVolumeFunction.apply(w2, *parts_u), AssembleVolumeFunction.apply(h2, *parts_v)
        return torch.cat(sep_u_lvls, dim=1), torch.cat(sep_v_lvls, dim=1)

    def __call__(self, coords, sep=False, attention_weights=None):
        if sep:
            return self.separate(attention_weights)
        return self.lookup(coords)

    def lookup(self, coords):
        """corr_fn(coords) without the 4D volume: (B, levels*(2r+1)^2, H1, W1).

        The reference stops here with NotImplementedError (core/corr.py:491-492) because the native part its
        draft calls (alt_cuda_corr.forward per level, core/corr.py:494-509) is not in its tree; the values are
        those of the stored-volume block (CorrBlock.__call__, core/corr.py:193-248).  Gradients reach fmap1 and
        fmap2 (through the pooled pyramid); coords get none, as the flow iterations detach them.
        """
        if self._lookup_inputs is None:
            # NHWC copies are made once per block and shared by all flow iterations (the draft redoes them per call)
            b, c, h, w = self.fmap1_l0.shape
            if (self.fmap1_l0.is_cuda and self.fmap1_l0.dtype == torch.float32 and self.fmap2_l0.dtype == torch.float32
                    and 1 <= self.num_levels <= 4 and min(h, w) >> (self.num_levels - 1) >= 1
                    and b * ((c + 31) // 32) < 65536):
                (f1,) = FeaturePyramidFunction.apply(self.fmap1_l0.contiguous(), 1, 1.0)
                self._lookup_inputs = (f1, list(FeaturePyramidFunction.apply(self.fmap2_l0.contiguous(), self.num_levels, 1.0)))
            else:
                f1 = self.fmap1_l0.permute(0, 2, 3, 1).contiguous().float()
                self._lookup_inputs = (f1, [p.permute(0, 2, 3, 1).contiguous().float() for p in self.pyramid])
        f1, f2s = self._lookup_inputs
        scale = 1.0 / float(torch.sqrt(torch.tensor(f1.shape[3]).float()))
        return LookupFunction.apply(coords.detach().contiguous().float(), self.radius, scale, f1, *f2s)


class CorrBlock1D:
    """Lookup in the two separated 3D volumes: the reference's CorrBlock1D (core/corr.py:513-624).

    corr1 (B,dim,W2,H1,W1) and corr2 (B,dim,H2,H1,W1) as separate() (or the cost aggregation after it) returns them.
    `__call__(coords)` -> (out1, out2), each (B, num_levels*dim*(2*radius+1), H1, W1).  The reference stores a
    pyramid of permuted copies per block and samples it with grid_sample once per level, volume and flow iteration;
    here the volumes stay in the layout they arrive in, the pyramid is formed on the fly, and one kernel per volume does
    the whole lookup.  The clamp of the sampling positions to [-1, 1] that the reference applies to its first volume only
    (core/corr.py:593) is reproduced (`clamp_first=False` drops it).
    """

    def __init__(self, corr1, corr2, num_levels=4, radius=4, clamp_first=True):
        assert corr1.shape[:2] == corr2.shape[:2] and corr1.shape[3:] == corr2.shape[3:]
        # core/corr.py:536: the displacement axes must be as long as the image axes
        assert corr1.shape[2] == corr1.shape[4] and corr2.shape[2] == corr2.shape[3]
        self.num_levels = num_levels
        self.radius = radius
        self.clamp_first = clamp_first
        self.corr1 = corr1.contiguous().float()
        self.corr2 = corr2.contiguous().float()

    def __call__(self, coords):
        coords = coords.detach().contiguous().float()
        out1 = Lookup1DFunction.apply(self.corr1, coords, 0, self.clamp_first, self.num_levels, self.radius)
        out2 = Lookup1DFunction.apply(self.corr2, coords, 1, False, self.num_levels, self.radius)
        return out1, out2
