"""Activations over the feature matrix of a sparse tensor (script/activation.py:6-15)."""
from torch import nn

from .sptensor import spTensor
from .utils import fapply


class ReLU(nn.ReLU):
    def forward(self, input: spTensor) -> spTensor:
        return fapply(input, super().forward)


class LeakyReLU(nn.LeakyReLU):
    def forward(self, input: spTensor) -> spTensor:
        return fapply(input, super().forward)
