"""Batch normalisation over the feature matrix of a sparse tensor (script/batchnorm.py:7-10).

The reference wraps ``torch.nn.BatchNorm1d``.  Parameters, buffers and their semantics (momentum,
``track_running_stats``, the unbiased variance in ``running_var``) are kept; on the GPU a pass is three
launches of the library (``pce_bn_forward`` / ``pce_bn_backward``: partial column sums, one thread per
channel for statistics and coefficients, one affine map) instead of torch's channels-last kernels,
which are an order of magnitude off the memory roofline on [N, C] matrices of 10^5 rows."""
import torch
from torch import nn

from . import backend
from .sptensor import spTensor
from .utils import fapply


class _BatchNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, running_mean, running_var, use_batch_stats, momentum, eps):
        y, mean, rstd = backend.bn_forward(x, weight, bias, running_mean, running_var, use_batch_stats, momentum, eps)
        ctx.save_for_backward(x, weight, mean, rstd)
        ctx.use_batch_stats = use_batch_stats
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, mean, rstd = ctx.saved_tensors
        dx, gw, gb = backend.bn_backward(x, dy, weight, mean, rstd, ctx.use_batch_stats)
        gw = gw.to(weight.dtype) if weight is not None and ctx.needs_input_grad[1] else None
        gb = gb.to(weight.dtype if weight is not None else x.dtype) if ctx.has_bias and ctx.needs_input_grad[2] else None
        return dx, gw, gb, None, None, None, None, None


class BatchNorm(nn.BatchNorm1d):
    def _features(self, x: torch.Tensor) -> torch.Tensor:
        native = x.is_cuda and x.dim() == 2 and x.dtype in (torch.float16, torch.float32) and x.shape[0] > 0
        if native and self.track_running_stats:
            native = self.running_mean.dtype == torch.float32 and self.running_var.dtype == torch.float32
        if not native:
            return super().forward(x)       # CPU tensors, other dtypes: torch's own kernels
        use_batch_stats = self.training or not self.track_running_stats
        momentum = -1.0
        if self.training and self.track_running_stats:
            self.num_batches_tracked += 1
            momentum = self.momentum if self.momentum is not None else 1.0 / float(self.num_batches_tracked)
        return _BatchNormFunction.apply(x, self.weight, self.bias, self.running_mean, self.running_var, use_batch_stats,
                                        momentum, self.eps)

    def forward(self, input: spTensor) -> spTensor:
        return fapply(input, self._features)
