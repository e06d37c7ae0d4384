"""MI355X-native memory-saving separation of the 4D correlation volume (Separable Flow).

Drop-in for the reference's libs/MemorySaver package: the same three autograd Functions, the
module wrapper and the caller class, backed by hand-written gfx950 kernels in libsepcorr.so.
"""
from .functions import ComputeMaxArgmaxAvgFunction, ComputeMaxAvgFunction, ComputeSelfCompressionFunction
from .modules import ComputeMaxAvgModule
from .corr import AlternateCorrBlockSepflow, CorrBlock1D

__all__ = [
    "ComputeMaxAvgFunction", "ComputeMaxArgmaxAvgFunction", "ComputeSelfCompressionFunction",
    "ComputeMaxAvgModule", "AlternateCorrBlockSepflow", "CorrBlock1D",
]
