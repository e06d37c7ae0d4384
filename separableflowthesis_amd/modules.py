"""nn.Module wrapper of the max/avg op (libs/MemorySaver/modules/MemorySaver.py:10-14)."""
from torch.nn.modules.module import Module

from .functions import ComputeMaxAvgFunction


class ComputeMaxAvgModule(Module):
    def forward(self, img1_features_l0, img2_features_lk):
        return ComputeMaxAvgFunction.apply(img1_features_l0, img2_features_lk)
