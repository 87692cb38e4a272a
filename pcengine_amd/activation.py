"""ReLU and LeakyReLU on sparse tensors (the modules of script/activation.py:6-15).

Constructor arguments and results are those of ``torch.nn.ReLU`` / ``torch.nn.LeakyReLU`` applied to the
feature matrix; coordinates, strides and the map cache pass through untouched.  Each module also names itself
in the form the fused epilogues take (``conv3d.forward(act=...)``, ``BatchNorm.forward(act=...)``), so a block
can hand its activation to the kernel that produces the features instead of running it as a pass of its own.
"""
import torch.nn.functional as F
from torch import nn

from .sptensor import spTensor


class _OnFeatures(nn.Module):
    """An element-wise function of the features; ``inplace`` overwrites the feature matrix as torch's does."""

    def __init__(self, inplace: bool = False):
        super().__init__()
        self.inplace = bool(inplace)

    def _apply_to(self, feats):
        raise NotImplementedError

    def as_epilogue(self):
        """The ``act`` argument of the fused epilogues that computes the same function."""
        raise NotImplementedError

    def forward(self, x: spTensor) -> spTensor:
        return x._like(self._apply_to(x.feats))


class ReLU(_OnFeatures):
    def _apply_to(self, feats):
        return F.relu(feats, inplace=self.inplace)

    def as_epilogue(self):
        return "relu"

    def extra_repr(self) -> str:
        return "inplace=True" if self.inplace else ""


class LeakyReLU(_OnFeatures):
    def __init__(self, negative_slope: float = 0.01, inplace: bool = False):
        super().__init__(inplace)
        self.negative_slope = float(negative_slope)

    def _apply_to(self, feats):
        return F.leaky_relu(feats, self.negative_slope, inplace=self.inplace)

    def as_epilogue(self):
        return ("leaky_relu", self.negative_slope)

    def extra_repr(self) -> str:
        return f"negative_slope={self.negative_slope}" + (", inplace=True" if self.inplace else "")
