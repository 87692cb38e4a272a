"""MinkUNet-style sparse residual U-Net composed from this package's front-end modules.

The reference ships no network; this is the composition its primitives are meant for
(conv3d, BatchNorm, ReLU, cat, spTensor.__add__; script/spconv.py, script/utils.py:152-164,
script/sptensor.py:80-91): a stem, four encoder stages (k2s2 down-sampling + two residual
blocks), four decoder stages (transposed k2s2 + skip concatenation + two residual blocks) and a
1x1 head.  ``fuse_bn()`` folds every BatchNorm into the preceding convolution (inference mode).
"""
from __future__ import annotations

import os
from typing import List, Sequence

import torch
from torch import nn

from . import backend
from .activation import ReLU
from .batchnorm import BatchNorm
from .spconv import conv3d, prebuild_maps
from .sptensor import spTensor
from .utils import cat


class ConvBN(nn.Module):
    """conv3d followed by BatchNorm and an optional ReLU; the norm can be folded into the conv."""

    def __init__(self, cin, cout, ks=3, stride=1, transposed=False, relu=True, dataflow="auto"):
        super().__init__()
        self.conv = conv3d(cin, cout, ks, stride, transposed=transposed, dataflow=dataflow)
        self.bn = BatchNorm(cout)
        self.relu = ReLU(True) if relu else None

    def fuse(self) -> None:
        if self.bn is None:
            return
        bn = self.bn
        scale = bn.weight.detach() / torch.sqrt(bn.running_var + bn.eps)
        shift = bn.bias.detach() - bn.running_mean * scale
        with torch.no_grad():
            self.conv.kernel.mul_(scale.to(self.conv.kernel.dtype))
            b = shift.to(self.conv.kernel.dtype)
            if self.conv.bias is not None:
                b = b + self.conv.bias * scale.to(self.conv.kernel.dtype)
            self.conv.bias = nn.Parameter(b)
        self.bn = None

    def forward(self, x: spTensor, residual: spTensor = None, relu_after_residual: bool = False, out=None) -> spTensor:
        """With the norm folded away, bias, the optional residual and the ReLU run inside the conv kernels, and
        the features can go straight to `out` (a column slice of a wider matrix, see SparseResUNet.forward)."""
        act = self.relu.as_epilogue() if self.relu is not None else ("relu" if relu_after_residual else None)
        if self.bn is None:
            return self.conv(x, act=act, residual=residual, out=out)
        # training form: the residual sum and the ReLU ride on the norm's affine pass
        return self.bn(self.conv(x), residual=residual, act=act)


class ResidualBlock(nn.Module):
    def __init__(self, cin, cout, dataflow="auto"):
        super().__init__()
        self.a = ConvBN(cin, cout, 3, dataflow=dataflow)
        self.b = ConvBN(cout, cout, 3, relu=False, dataflow=dataflow)
        self.shortcut = None if cin == cout else ConvBN(cin, cout, 1, relu=False)
        self.relu = ReLU(True)

    def forward(self, x: spTensor, out=None) -> spTensor:
        s = x if self.shortcut is None else self.shortcut(x)
        return self.b(self.a(x), residual=s, relu_after_residual=True, out=out)      # relu(b(a(x)) + s)


class SparseResUNet(nn.Module):
    """enc = channels of the four encoder stages, dec = channels of the four decoder stages."""

    def __init__(self, in_channels: int = 4, num_classes: int = 20, stem: int = 32,
                 enc: Sequence[int] = (32, 64, 128, 256), dec: Sequence[int] = (256, 128, 96, 96),
                 dataflow: str = "auto"):
        super().__init__()
        df = dataflow
        self.stem = nn.Sequential(ConvBN(in_channels, stem, 3, dataflow=df), ConvBN(stem, stem, 3, dataflow=df))
        self.down = nn.ModuleList()
        self.enc = nn.ModuleList()
        c = stem
        skips: List[int] = [stem]
        for ce in enc:
            self.down.append(ConvBN(c, c, 2, 2, dataflow=df))
            self.enc.append(nn.Sequential(ResidualBlock(c, ce, df), ResidualBlock(ce, ce, df)))
            c = ce
            skips.append(c)
        skips.pop()                       # the deepest output is not a skip
        self.up = nn.ModuleList()
        self.dec = nn.ModuleList()
        for cd in dec:
            self.up.append(ConvBN(c, cd, 2, 2, transposed=True, dataflow=df))
            cs = skips.pop()
            self.dec.append(nn.Sequential(ResidualBlock(cd + cs, cd, df), ResidualBlock(cd, cd, df)))
            c = cd
        self.head = conv3d(c, num_classes, 1, bias=True)

    def fuse_bn(self) -> "SparseResUNet":
        for m in self.modules():
            if isinstance(m, ConvBN):
                m.fuse()
        self._in_place_ok = None
        return self

    def use_planner(self, on: bool = True) -> "SparseResUNet":
        """Build the kernel maps of every forward through the native planner (``spconv.MapPlanner``): one allocation,
        kept and reused from cloud to cloud, and two library calls for the whole pyramid.  The maps of a cloud then
        live until the next forward of this module; leave it off where maps must outlive that (a tensor whose
        ``kmaps`` are reused after another cloud went through the network).  In inference the layer outputs, routing
        arrays and the staging buffer then come from one allocation as well (``backend.ForwardArena``): from the
        second forward over clouds of one size on, a forward allocates no device memory, and the tensor it returns is
        valid until the next forward."""
        from .spconv import MapPlanner
        self._planner = MapPlanner() if on else None
        self._arena = None         # made on the first planned forward, on the device of its input
        return self

    def map_plan(self, dtype=None):
        """(kernel_size, stride, padding[, table_only]) of the layers that need a kernel map, in execution order.
        With ``dtype`` (an inference forward in that dtype) the 3x3x3 map of a level whose layers ALL have widths the
        ordered output-stationary dataflow takes is marked table-only: the selector gives such layers the ordered or
        the plain output-stationary dataflow, neither of which reads pair lists, so the build skips them (a layer
        that asks for them after all -- a forced dataflow -- gets them built then)."""
        lean = [False] * (len(self.down) + 1)
        if dtype in (torch.float16, torch.float32):
            code = backend.PCE_F16 if dtype == torch.float16 else backend.PCE_F32
            takes = backend._lib.load().pce_conv_oso_takes
            widths = [[] for _ in lean]           # (c_in, c_out) of the 3x3x3 layers of every level
            auto = [True]
            def add(level, module):
                for m in module.modules():
                    if isinstance(m, conv3d) and m.kernel_volume == 27 and not m.transposed and list(m.stride) == [1, 1, 1]:
                        widths[level].append((max(m.in_channels, 16), m.out_channels))
                        auto[0] = auto[0] and m.dataflow == "auto"
            add(0, self.stem)
            for l, enc in enumerate(self.enc):
                add(l + 1, enc)
            for i, dec in enumerate(self.dec):
                add(len(self.down) - 1 - i, dec)
            if auto[0] and not os.environ.get("PCENGINE_DATAFLOW"):
                lean = [bool(w) and all(takes(code, ci, co, 27, 13) for ci, co in w) for w in widths]
        plan = [(3, 1, 0, lean[0])]
        for l in range(len(self.down)):
            plan += [(2, 2, 0), (3, 1, 0, lean[l + 1])]
        return plan

    def forward(self, x: spTensor) -> spTensor:
        planner = getattr(self, "_planner", None)
        if planner is not None and x.feats.is_cuda and not (torch.is_grad_enabled() and (
                x.feats.requires_grad or any(p.requires_grad for p in self.parameters()))):
            if getattr(self, "_arena", None) is None or self._arena.device != x.feats.device:
                self._arena = backend.ForwardArena(x.feats.device)
            with backend.allocate_from(self._arena):
                return self._forward(x, planner)
        return self._forward(x, planner)

    def _forward(self, x: spTensor, planner) -> spTensor:
        # no host wait is left between the layers below; with a planner (see use_planner) all maps of the cloud are
        # laid out and built by the library in one allocation
        inference = not (torch.is_grad_enabled() and (x.feats.requires_grad or any(p.requires_grad for p in self.parameters())))
        prebuild_maps(x, self.map_plan(x.feats.dtype if inference else None), planner)
        if self._skips_in_place(x):
            return self._forward_skips_in_place(x)
        x = self.stem(x)
        feats = [x]
        for down, enc in zip(self.down, self.enc):
            x = enc(down(x))
            feats.append(x)
        feats.pop()
        for up, dec in zip(self.up, self.dec):
            x = up(x)
            x = dec(cat([x, feats.pop()]))
        return self.head(x)

    def _skips_in_place(self, x: spTensor) -> bool:
        """Inference with every norm folded, on the GPU, all widths multiples of 8 channels: the two producers of
        a skip connection can then write their halves of the concatenated matrix themselves."""
        if torch.is_grad_enabled() and (x.feats.requires_grad or any(p.requires_grad for p in self.parameters())):
            return False        # autograd results are fresh tensors: nothing can be written in place
        if not x.feats.is_cuda:
            return False
        ok = getattr(self, "_in_place_ok", None)
        if ok is None:      # what depends on the modules alone: looked up once, again after fuse_bn()
            widths = [self.stem[1].conv.out_channels] + [e[1].b.conv.out_channels for e in self.enc] + \
                     [u.conv.out_channels for u in self.up]
            ok = all(w % 8 == 0 for w in widths) and \
                not any(isinstance(m, ConvBN) and m.bn is not None for m in self.modules())
            self._in_place_ok = ok
        return ok

    def _forward_skips_in_place(self, x: spTensor) -> spTensor:
        """The same network with the concatenation of each decoder stage done by its producers: the encoder layer
        whose output is kept writes the right-hand columns of a [rows, c_up + c_skip] matrix, the transposed layer
        the left-hand ones later, and the decoder block reads the matrix; the layers that consume the kept output
        on the way down gather from its columns in place.  Same kernels, same values, no pass that copies."""
        def joined(rows, like, c_up, c_skip):
            return backend._new((rows, c_up + c_skip), like.dtype, like.device)
        ups = [u.conv.out_channels for u in self.up][::-1]      # c_up of the stage that ends at level 0, 1, ...
        x = self.stem[0](x)
        buf = joined(x.feats.shape[0], x.feats, ups[0], self.stem[1].conv.out_channels)
        x = self.stem[1](x, out=buf[:, ups[0]:])
        bufs = [buf]
        last = len(self.enc) - 1
        for lv, (down, enc) in enumerate(zip(self.down, self.enc)):
            x = enc[0](down(x))
            if lv < last:
                buf = joined(x.feats.shape[0], x.feats, ups[lv + 1], enc[1].b.conv.out_channels)
                x = enc[1](x, out=buf[:, ups[lv + 1]:])
                bufs.append(buf)
            else:
                x = enc[1](x)            # the deepest output is not a skip
        for up, dec in zip(self.up, self.dec):
            buf = bufs.pop()
            x = up(x, out=buf[:, :up.conv.out_channels])
            x = dec(x._like(buf))
        return self.head(x)
