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
    """``act(batch_norm(x) + residual)``; ``residual`` and ``act`` may be None."""

    @staticmethod
    def forward(ctx, x, weight, bias, running_mean, running_var, use_batch_stats, momentum, eps, residual, act):
        y, mean, rstd = backend.bn_forward(x, weight, bias, running_mean, running_var, use_batch_stats, momentum, eps,
                                           act=act, residual=None if residual is None else residual.detach())
        ctx.save_for_backward(x, weight, mean, rstd, y if act is not None else None)
        ctx.use_batch_stats = use_batch_stats
        ctx.has_bias = bias is not None
        ctx.act = act
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, mean, rstd, y = ctx.saved_tensors
        act, dres = ctx.act, None
        if ctx.needs_input_grad[8]:
            # the residual's gradient is the masked incoming gradient itself: form it once and hand it on
            if act is not None:
                dy = dy.to(y.dtype)
                if act == "relu":
                    dy = torch.ops.aten.threshold_backward(dy, y, 0.0)
                else:
                    dy = torch.where(y > 0, dy, dy * float(act[1]))
                act = None
            dres = dy
        dx, gw, gb = backend.bn_backward(x, dy, weight, mean, rstd, ctx.use_batch_stats, y_act=y, act=act)
        gw = gw.to(weight.dtype) if weight is not None and ctx.needs_input_grad[1] else None
        gb = gb.to(weight.dtype if weight is not None else x.dtype) if ctx.has_bias and ctx.needs_input_grad[2] else None
        return dx, gw, gb, None, None, None, None, None, dres, None


class BatchNorm(nn.BatchNorm1d):
    def _features(self, x: torch.Tensor, residual=None, act=None) -> torch.Tensor:
        native = x.is_cuda and x.dim() == 2 and x.dtype in (torch.float16, torch.float32) and x.shape[0] > 0
        if native and self.track_running_stats:
            native = self.running_mean.dtype == torch.float32 and self.running_var.dtype == torch.float32
        if native and residual is not None:
            native = residual.dtype == x.dtype and residual.shape == x.shape
        if native and self.training and x.shape[0] == 1:
            native = False                  # torch refuses batch statistics of a single row: keep its error
        if not native:                      # CPU tensors, other dtypes: torch's own kernels
            y = super().forward(x)
            if residual is not None:
                y = y + residual
            if act == "relu":
                y = torch.relu(y)
            elif act is not None:
                y = torch.nn.functional.leaky_relu(y, act[1])
            return y
        use_batch_stats = self.training or not self.track_running_stats
        momentum = -1.0
        if self.training and self.track_running_stats:
            self.num_batches_tracked += 1
            momentum = self.momentum if self.momentum is not None else 1.0 / float(self.num_batches_tracked)
        return _BatchNormFunction.apply(x, self.weight, self.bias, self.running_mean, self.running_var, use_batch_stats,
                                        momentum, self.eps, residual, act)

    def forward(self, input: spTensor, residual: spTensor = None, act=None) -> spTensor:
        """``act(norm(input) + residual)``: the residual sum and the activation that follow the norm in a
        residual block ride on the norm's own passes.  ``act``: None, 'relu' or ('leaky_relu', slope > 0)."""
        if act is not None and act != "relu" and not (isinstance(act, tuple) and len(act) == 2 and act[0] == "leaky_relu"
                                                      and act[1] > 0):
            raise ValueError(f"unsupported activation {act!r}")
        res = None if residual is None else residual.feats
        return fapply(input, lambda f: self._features(f, res, act))
