"""conv3d: sparse 3-D convolution with the reference's module interface
(script/spconv.py:15-106) over the MI355X backend.

Differences a user can see, all supersets of the reference:
* ``dataflow='auto'|'fod'|'gms'|'os'|'fds'`` constructor argument (and the PCENGINE_DATAFLOW
  environment variable) on top of the reference's ``init_tag`` list.  A tensor whose
  ``init_tag`` starts with 'D1' / 'D2' pins the next newly built map to gather-GEMM-scatter /
  fetch-on-demand exactly as in the reference (script/spconv.py:343, 388); the default tag
  ('end') lets the selector decide per layer.
* every strided layer uses the generic output-coordinate rule, also when stride == kernel size.
* training: when gradients are enabled and the features or the parameters require them, the layer
  runs through an autograd function whose backward uses the same kernels (feature gradient =
  convolution of the output gradient with the transposed kernel over the swapped map; kernel
  gradient = ``pce_conv_wgrad``).  The reference has a backward for gather-GEMM-scatter only
  (script/spconv.py:172-201); here it serves every dataflow.
* ``forward(input, act=None, residual=None)``: an activation ('relu' or ('leaky_relu', slope)) and
  a residual tensor (same coordinates) are applied inside the convolution kernels together with
  the bias, instead of as separate passes over the output.
"""
from __future__ import annotations

import math
import os
from typing import List, Optional, Union

import numpy as np
import torch
import torch.nn as nn

from . import backend
from .backend import DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS, DATAFLOW_OSO
from .sptensor import spTensor
from .utils import conv_info_decoder, conv_info_encoder, output_stride_compute

_UNIT = conv_info_encoder([1, 1, 1])
_DATAFLOWS = {"fod": DATAFLOW_FOD, "d2": DATAFLOW_FOD, "gms": DATAFLOW_GMS, "d1": DATAFLOW_GMS, "os": DATAFLOW_OS,
              "fds": DATAFLOW_FDS, "oso": DATAFLOW_OSO}

# one record per executed layer when enabled: (N_in, N_out, M, C_in, C_out, dataflow)
layer_log: Optional[list] = None


def _triple(v, what: str) -> List[int]:
    if isinstance(v, int):
        return [v, v, v]
    if isinstance(v, list):
        return v
    raise NotImplementedError(f"{what} must be an int or a list of three ints")


class conv3d(nn.Module):

    def __init__(self, in_channels: int = 16, out_channels: int = 32, kernel_size: Union[int, List[int]] = 3,
                 stride: Union[int, List[int]] = 1, padding: Union[int, List[int]] = 0, bias: bool = False,
                 transposed: bool = False, tc_mode: bool = True, dataflow: str = "auto") -> None:
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.transposed = transposed
        self.kernel_size = _triple(kernel_size, "kernel_size")
        self.kernel_size_code = conv_info_encoder(self.kernel_size)
        self.kernel_volume = int(np.prod(self.kernel_size, dtype=int))
        self.stride = _triple(stride, "stride")
        self.stride_code = conv_info_encoder(self.stride)
        self.padding = _triple(padding, "padding")
        self.padding_code = conv_info_encoder(self.padding)
        self.tensorcore = tc_mode
        if dataflow != "auto" and dataflow.lower() not in _DATAFLOWS:
            raise NotImplementedError(f"unknown dataflow {dataflow!r}")
        self.dataflow = dataflow.lower()
        shape = (self.kernel_volume, in_channels, out_channels) if self.kernel_volume > 1 else (in_channels, out_channels)
        self.kernel = nn.Parameter(torch.zeros(shape))
        self.bias = nn.Parameter(torch.zeros((out_channels,))) if bias else None
        self.reset_parameters()

    def extra_repr(self) -> str:
        s = f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}"
        if self.stride_code != _UNIT:
            s += f", stride={self.stride}"
        if self.bias is None:
            s += ", bias=False"
        if self.transposed:
            s += ", transposed=True"
        return s

    def reset_parameters(self) -> None:
        # U(-1/sqrt(C_out*kv), +1/sqrt(C_out*kv)) for kernel and bias (script/spconv.py:101-106)
        bound = 1.0 / math.sqrt(self.out_channels * self.kernel_volume)
        with torch.no_grad():
            self.kernel.uniform_(-bound, bound)
            if self.bias is not None:
                self.bias.uniform_(-bound, bound)

    def _weights_for(self, dtype):
        """Kernel in the feature dtype plus its packed fp16 copy, rebuilt only when the parameter changes."""
        k = self.kernel
        key = (k.data_ptr(), k._version, dtype, k.device)
        if getattr(self, "_wcache_key", None) != key:
            w = k.detach()
            w = w if w.dtype == dtype else w.to(dtype)
            if dtype == torch.float16 and w.is_cuda and w.dim() == 3 and w.shape[1] < 16:
                # a 3- or 4-channel input layer: zero rows up to 16 input channels make the rows 16-byte
                # multiples, which the vector kernels need (the features are padded to match in _run)
                w = torch.nn.functional.pad(w, (0, 0, 0, 16 - w.shape[1]))
            w = w.contiguous()
            self._wcache = (w, backend.pack_weights(w) if w.is_cuda else None)
            self._wcache_key = key
        return self._wcache

    def _bias_for(self, dtype):
        b = self.bias
        if b is None:
            return None
        key = (b.data_ptr(), b._version, dtype, b.device)
        if getattr(self, "_bcache_key", None) != key:
            self._bcache = b.detach().to(dtype).contiguous()
            self._bcache_key = key
        return self._bcache

    def forward(self, input: spTensor, act=None, residual: Optional[spTensor] = None,
                out: Optional[torch.Tensor] = None) -> spTensor:
        """``out`` (inference only): where the output features go -- a preallocated matrix or a column slice of a
        wider one, e.g. this layer's half of a concatenated skip connection."""
        if _wants_grad(input.feats, self.kernel, self.bias):
            # training: the parameters themselves go to the autograd function (no cached copies)
            return conv_func(input=input, in_channel=self.in_channels, out_channel=self.out_channels, kernel=self.kernel,
                             kernel_size_code=self.kernel_size_code, stride_code=self.stride_code,
                             padding_code=self.padding_code, bias=self.bias, transposed=self.transposed,
                             tensorcore=self.tensorcore, dataflow=self.dataflow, packed=None, act=act,
                             residual=None if residual is None else residual.feats, out=out)
        w, packed = self._weights_for(input.feats.dtype)
        return conv_func(input=input, in_channel=self.in_channels, out_channel=self.out_channels, kernel=w,
                         kernel_size_code=self.kernel_size_code, stride_code=self.stride_code,
                         padding_code=self.padding_code, bias=self._bias_for(input.feats.dtype),
                         transposed=self.transposed, tensorcore=self.tensorcore, dataflow=self.dataflow, packed=packed,
                         act=act, residual=None if residual is None else residual.feats, out=out)


def _pick_dataflow(km: backend.KernelMap, requested: str, c_in: int, c_out: int, dtype, transposed: bool) -> int:
    env = os.environ.get("PCENGINE_DATAFLOW", "").lower()
    forced = _DATAFLOWS.get(env, _DATAFLOWS.get(requested))
    if forced is not None:
        if forced == DATAFLOW_OSO and not backend.oso_takes(km, c_in, c_out, dtype, transposed):
            return DATAFLOW_FDS     # the ordered dataflow exists for narrow layers only (backend.oso_takes)
        return forced
    if km.tag == "D1":
        return DATAFLOW_GMS
    if km.tag == "D2":
        return DATAFLOW_FOD
    picks = km.__dict__.setdefault("_picks", {})      # the selector's answer per layer shape on this map
    key = (c_in, c_out, dtype, transposed)
    df = picks.get(key)
    if df is None:
        df = picks[key] = backend.select_dataflow(km, c_in, c_out, dtype, transposed)
    return df


class _ConvFunction(torch.autograd.Function):
    """conv (+ bias) with gradients for features, kernel and bias (conv_d1 / conv_d2,
    script/spconv.py:110-288)."""

    @staticmethod
    def forward(ctx, feats, kernel, bias, km, df, transposed, buffer):
        k = kernel.detach()
        out = backend.conv_forward(feats.detach(), k, km, df, transposed=transposed, buffer=buffer,
                                   packed=backend.pack_weights(k), bias=None if bias is None else bias.detach())
        ctx.save_for_backward(feats, kernel)
        ctx.km, ctx.transposed, ctx.has_bias = km, transposed, bias is not None
        return out

    @staticmethod
    def backward(ctx, grad_out):
        feats, kernel = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        gf, gw = backend.conv_backward(feats.detach(), kernel.detach(), ctx.km, grad_out, transposed=ctx.transposed,
                                       need_feats=ctx.needs_input_grad[0], need_weight=ctx.needs_input_grad[1])
        gb = grad_out.sum(0) if (ctx.has_bias and ctx.needs_input_grad[2]) else None
        return gf, gw, gb, None, None, None, None


class _DenseFunction(torch.autograd.Function):
    """The 1x1 layer (feats @ kernel + bias) with the same backward kernels."""

    @staticmethod
    def forward(ctx, feats, kernel, bias):
        k = kernel.detach()
        out = backend.dense_forward(feats.detach(), k, backend.pack_weights(k), bias=None if bias is None else bias.detach())
        ctx.save_for_backward(feats, kernel)
        ctx.has_bias = bias is not None
        return out

    @staticmethod
    def backward(ctx, grad_out):
        feats, kernel = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        gf = gw = None
        if ctx.needs_input_grad[0]:
            kt = kernel.detach().t().contiguous()
            gf = backend.dense_forward(grad_out, kt, backend.pack_weights(kt))
        if ctx.needs_input_grad[1]:
            gw = backend.dense_wgrad(feats.detach(), grad_out).to(kernel.dtype)
        gb = grad_out.sum(0) if (ctx.has_bias and ctx.needs_input_grad[2]) else None
        return gf, gw, gb


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def _no_out_with_grad(out) -> None:
    """``out=`` names memory the kernels write in place; a result autograd has to track is a fresh tensor, so
    the combination is refused instead of leaving ``out`` unwritten."""
    if out is not None:
        raise ValueError("conv3d: out= is for inference; features or parameters that require grad (with grad enabled) "
                         "produce a new tensor -- call under torch.no_grad() or drop out=")


def _apply_unfused(out: torch.Tensor, residual, act) -> torch.Tensor:
    """Residual and activation as differentiable torch ops (the training path does not fuse them)."""
    if residual is not None:
        out = out + residual
    if act == "relu":
        out = torch.relu(out)
    elif isinstance(act, tuple) and act[0] == "leaky_relu":
        out = torch.nn.functional.leaky_relu(out, act[1])
    elif act is not None:
        raise ValueError(f"unknown activation {act!r}")
    return out


def _run(input: spTensor, km: backend.KernelMap, kernel, in_channel, out_channel, transposed, dataflow, packed,
         bias=None, residual=None, act=None, out=None) -> torch.Tensor:
    feats = input.feats
    if _wants_grad(feats, kernel, bias):
        _no_out_with_grad(out)
        k = kernel if kernel.dtype == feats.dtype else kernel.to(feats.dtype)
        b = bias if bias is None or bias.dtype == feats.dtype else bias.to(feats.dtype)
        df = _pick_dataflow(km, dataflow, in_channel, out_channel, feats.dtype, transposed)
        out = _ConvFunction.apply(feats, k, b, km, df, transposed, input.buffer)
        return _apply_unfused(out, residual, act)
    if kernel.dtype != feats.dtype:
        kernel, packed = kernel.to(feats.dtype), None
    if kernel.dim() == 3 and feats.shape[1] < kernel.shape[1]:
        # see conv3d._weights_for (the padded copy comes from the forward's arena where one is active)
        padded = backend._new((feats.shape[0], kernel.shape[1]), feats.dtype, feats.device)
        padded[:, feats.shape[1]:].zero_()
        padded[:, :feats.shape[1]].copy_(feats)
        feats = padded
    # the selector sees the width the kernels run at (a 3- or 4-channel input layer runs padded to 16)
    df = _pick_dataflow(km, dataflow, feats.shape[1], out_channel, feats.dtype, transposed)
    out = backend.conv_forward(feats, kernel.detach(), km, df, transposed=transposed, buffer=input.buffer, packed=packed,
                               out=out, bias=bias, residual=residual, act=act)
    if layer_log is not None:
        layer_log.append((feats.shape[0], out.shape[0], km.M, in_channel, out_channel, df))
    return out


def _map_request(input: spTensor, kernel_size_code: int, stride_code: int, padding_code: int):
    """Cache lookup of one layer's map.  Returns (map or None, build request or None, cache key, tag,
    output tensor stride, output coords_min, output coords_max)."""
    output_stride = output_stride_compute(stride_code, input.stride, 0)
    key = (kernel_size_code, input.stride, stride_code)
    km = input.kmaps.get(key)
    subm = stride_code == _UNIT
    coords_max = list(input.coords_max[:3])
    coords_min = list(input.coords_min[:3])
    ks = conv_info_decoder(kernel_size_code)
    stride = conv_info_decoder(stride_code)
    pad = conv_info_decoder(padding_code)
    if not subm:
        coords_max = backend.strided_coords_max(input.coords_max, ks, stride, pad)   # script/spconv.py:358-360
    tag = request = None
    if km is None:
        tag = input.init_tag[0] if input.init_tag else 'end'
        if tag not in ('D1', 'D2', 'end', 'auto'):
            raise NotImplementedError(f"unknown init_tag entry {tag!r}")
        auto = tag in ('end', 'auto')
        request = dict(in_coords=input.coords, ks=ks, stride=stride, pad=pad, cmin=coords_min, cmax_out=coords_max,
                       subm=subm, want_csr=(tag == 'D1' or auto), want_nbr_out=auto, want_nbr_in=auto and not subm,
                       batchsize=input.batchsize)
        if tag in ('D1', 'D2'):
            input.init_tag = input.init_tag[1:]
    return km, request, key, tag, output_stride, coords_min, coords_max


def _map_store(input: spTensor, km: backend.KernelMap, key, tag, output_stride) -> None:
    km.tag = tag if tag in ('D1', 'D2') else 'auto'
    input.kmaps[key] = km
    input.cbook[output_stride] = km.out_coords


def ensure_map(input: spTensor, kernel_size_code: int, stride_code: int, padding_code: int):
    """Kernel map of a (non-transposed) layer on this tensor: looked up in the shared cache or built
    and stored there (script/spconv.py:331-437).  Returns (map, output tensor stride, output
    coords_min, output coords_max).  Maps depend on coordinates only, so a network can ask for all of
    them before the first convolution (``prebuild_maps``)."""
    km = input.kmaps.get((kernel_size_code, input.stride, stride_code))
    if km is not None and not isinstance(km, backend._MapJob):
        # the usual case inside a network (its maps were built ahead): nothing to decode but the output bound
        input.cbook.setdefault(input.stride, input.coords)
        if stride_code == _UNIT:
            return km, input.stride, input.coords_min, input.coords_max
        return km, output_stride_compute(stride_code, input.stride, 0), input.coords_min, list(km._cmax)
    km, request, key, tag, output_stride, coords_min, coords_max = _map_request(input, kernel_size_code, stride_code, padding_code)
    if request is not None:
        km = backend.build_kernel_map(**request)
        _map_store(input, km, key, tag, output_stride)
    input.cbook.setdefault(input.stride, input.coords)
    return km, output_stride, coords_min, coords_max


def _chain_out_coords(input: spTensor, layers) -> dict:
    """{index in `layers`: output coordinates} of the strided entries, computed with one wait of the host for all
    of them; empty where that does not apply (fewer than two strided entries, one of them cached, no batch count,
    a level the library's chained build does not take)."""
    if not input.coords.is_cuda or not input.batchsize or input.batchsize <= 0:
        return {}
    geoms, idx = [], []
    stride, cmax, cmin = input.stride, list(input.coords_max[:3]), list(input.coords_min[:3])
    for i, entry in enumerate(layers):
        ks, st, pad, _ = _layer_entry(entry)
        ksc, sc, pc = (conv_info_encoder(_triple(v, "layer")) for v in (ks, st, pad))
        if sc == _UNIT:
            continue
        if (ksc, stride, sc) in input.kmaps:
            return {}
        k3, s3, p3 = conv_info_decoder(ksc), conv_info_decoder(sc), conv_info_decoder(pc)
        cmax = backend.strided_coords_max(cmax, k3, s3, p3)
        geoms.append(backend.Geom.make(k3, s3, p3, cmin, cmax, False))
        idx.append(i)
        stride = output_stride_compute(sc, stride, 0)
    if len(geoms) < 2 or len(geoms) > backend.MAX_CHAIN:
        return {}
    outs = backend.build_out_coords_chain(input.coords.contiguous(), geoms, input.batchsize)
    return dict(zip(idx, outs)) if outs is not None else {}


def _layer_entry(entry):
    """(kernel_size, stride, padding, table_only) of an entry of a layer list: the fourth element is optional and
    says that every layer that will use the map takes a dataflow that reads the neighbour table and the row order
    only (the ordered or the plain output-stationary one), so that a 3x3x3 submanifold map may be built without its
    pair lists (``PCE_KMAP_TABLE_ONLY``; they are built on first use should a layer ask for them after all)."""
    if len(entry) == 4:
        return entry[0], entry[1], entry[2], bool(entry[3])
    ks, stride, pad = entry
    return ks, stride, pad, False


class MapPlanner:
    """Keeps the native plans (``backend.PyramidPlan``: one allocation for all maps of a network on one cloud) a network
    has used, one per (layer list, coordinate box, batch count); a plan is reused for every cloud of at most its
    capacity in rows and replaced by a larger one when a cloud exceeds it.  The maps of a cloud live in the plan's
    allocation until the next cloud is built with it: a caller that keeps maps across forwards (a prefetcher, two
    clouds in flight) uses one planner per cloud in flight, or none."""

    def __init__(self, headroom: float = 1.125):
        self.plans = {}
        self.headroom = headroom

    def plan_for(self, key, n: int, make):
        plan = self.plans.get(key)
        if plan is None or plan.n_cap < n:
            cap = -(-int(n * self.headroom) // 4096) * 4096
            plan = self.plans[key] = make(cap)
        return plan


def _prebuild_planned(input: spTensor, layers, planner: MapPlanner):
    """The maps `layers` asks for through the native planner, or None where it does not apply (a map already cached,
    reference tags, no batch count, a strided layer whose kernel differs from its stride or that is padded, a cloud
    that is not sorted): the caller then builds them map by map.  Same maps, same cache entries."""
    if not input.coords.is_cuda or not input.batchsize or input.batchsize <= 0:
        return None
    if input.init_tag and input.init_tag[0] not in ('end', 'auto'):      # the reference's D1 / D2 tags: map by map
        return None
    entries, strided, requests = [], [], []
    stride_code, cmin, cmax, level = input.stride, list(input.coords_min[:3]), list(input.coords_max[:3]), 0
    seen = {}
    for entry in layers:
        ks, st, pad, table_only = _layer_entry(entry)
        ksc, sc, pc = (conv_info_encoder(_triple(v, "layer")) for v in (ks, st, pad))
        if ksc == _UNIT and sc == _UNIT:
            continue
        key = (ksc, stride_code, sc)
        if key in input.kmaps:
            return None
        k3, s3, p3 = conv_info_decoder(ksc), conv_info_decoder(sc), conv_info_decoder(pc)
        subm = sc == _UNIT
        if subm:
            if key not in seen:
                seen[key] = len(requests)
                lean = table_only and k3 == (3, 3, 3)
                requests.append((level, level, k3, s3, p3, cmin, cmax, True, not lean, False, lean))
                entries.append((key, stride_code, level, level))
            continue
        if k3 != s3 or any(p3) or key in seen:
            return None
        cmax = backend.strided_coords_max(cmax, k3, s3, p3)
        out_stride = output_stride_compute(sc, stride_code, 0)
        strided.append(backend.Geom.make(k3, s3, p3, cmin, cmax, False))
        seen[key] = len(requests)
        requests.append((level, level + 1, k3, s3, p3, cmin, cmax, False, True, True, False))
        entries.append((key, out_stride, level, level + 1))
        stride_code, level = out_stride, level + 1
    if not requests:
        return None
    coords = input.coords if input.coords.is_contiguous() else input.coords.contiguous()
    n = coords.shape[0]
    pkey = (tuple(map(tuple, ((r[0], r[1], r[10]) + tuple(r[2]) + tuple(r[6]) for r in requests))), tuple(input.coords_min[:3]),
            int(input.batchsize), coords.device)
    try:
        plan = planner.plan_for(pkey, n, lambda cap: backend.PyramidPlan(cap, strided, requests, input.batchsize, coords.device))
        level_coords, maps = plan.build(coords)
    except backend.PlanNotApplicable:
        return None
    level_stride = {0: input.stride}
    for (key, out_stride, lin, lout), km in zip(entries, maps):
        km.tag = 'auto'
        input.kmaps[key] = km
        level_stride[lout] = out_stride
    input.cbook.setdefault(input.stride, input.coords)
    for lv in range(1, len(level_coords)):
        input.cbook[level_stride[lv]] = level_coords[lv]
    return maps


def _prebuild(input: spTensor, layers, planner: Optional[MapPlanner] = None):
    """Builds the maps `layers` asks for, starting at `input`.  Returns (the tensor at the coordinates the last
    entry leaves, the maps that were built now)."""
    layers = list(layers)
    if planner is not None:
        built = _prebuild_planned(input, layers, planner)
        if built is not None:
            return input, built
    x = input
    pending, done = [], []
    chained = _chain_out_coords(input, layers)
    try:
        for i, entry in enumerate(layers):
            ks, stride, pad, table_only = _layer_entry(entry)
            ksc, sc, pc = (conv_info_encoder(_triple(v, "layer")) for v in (ks, stride, pad))
            if ksc == _UNIT and sc == _UNIT:
                continue
            km, request, key, tag, out_stride, cmin, cmax = _map_request(x, ksc, sc, pc)
            if request is not None:
                if i in chained:
                    request["out_coords"] = chained[i]
                if table_only and sc == _UNIT and tag not in ('D1', 'D2') and tuple(conv_info_decoder(ksc)) == (3, 3, 3):
                    request["want_csr"], request["want_pairs"] = False, False
                km = backend.prepare_map(**request)
                pending.append((x, km, key, tag, out_stride))
                x.kmaps[key] = km          # placeholder: a later entry with the same key is the same map
            x.cbook.setdefault(x.stride, x.coords)
            if sc != _UNIT:
                nxt = spTensor(feats=x.feats, coords=km.out_coords, buffer=x.buffer, batchsize=x.batchsize,
                               stride=out_stride, init_tag=x.init_tag, coords_max=cmax, coords_min=cmin)
                nxt.kmaps, nxt.cbook = x.kmaps, x.cbook
                x = nxt
        if pending:
            built = backend.build_kernel_maps([job for _, job, _, _, _ in pending], defer=True)
            torch.cuda.current_stream(input.coords.device).synchronize()
            for (t, _, key, tag, out_stride), pm in zip(pending, built):
                km = pm.finish()
                _map_store(t, km, key, tag, out_stride)
                done.append(km)
    finally:
        for t, job, key, _, _ in pending:       # a failed build leaves no placeholder behind
            if t.kmaps.get(key) is job:
                del t.kmaps[key]
    return x, done


def prebuild_maps(input: spTensor, layers, planner: Optional[MapPlanner] = None) -> None:
    """Build, ahead of any convolution, the maps a network will ask for.  ``layers`` lists
    (kernel_size, stride, padding) in network order (ints or triples; transposed layers and 1x1
    layers need no entry; an optional fourth element True marks a 3x3x3 submanifold map whose layers all read the
    neighbour table only, ``_layer_entry``); a strided entry moves on to its output coordinates, as the network does.
    The output coordinates of the strided layers are computed first, level by level (their number has
    to reach the host); then all maps are built together, every stage of the build as one launch over
    all layers, and their pair counts are read back in one copy.  The layers that follow find every
    map in the cache.  With a ``planner`` the whole pyramid is laid out and built by the library in one allocation
    (``MapPlanner``); where that does not apply the maps are built as described."""
    _prebuild(input, layers, planner)


class MapPrefetcher:
    """Kernel maps of the next cloud, built on a second stream while the network still runs the current one.

    A map build ends in waits of the host for counts; on the stream the convolutions run on, such a wait first drains
    everything queued there.  A serving loop that knows its next cloud calls ``submit(next)`` right after it has
    queued the forward of the current one: the host then waits on the second stream only, and the GPU builds the
    maps beside the convolutions.  ``take(x)`` makes the current stream wait for the maps of ``x`` (a no-op on the
    GPU by then) -- the layers that follow find every map in the cache.

    The coordinates of a submitted tensor must be complete when ``submit`` is called (they were copied or computed
    earlier and the stream that did it has been waited for): the second stream does not wait for the first.  Map
    memory is allocated on the second stream and announced to the consuming one with ``Tensor.record_stream``, so
    dropping a tensor's maps while convolutions still read them is safe."""

    def __init__(self, layers, device=None):
        self.layers = list(layers)
        self.stream = torch.cuda.Stream(device)
        self.pending = {}

    def submit(self, input: spTensor) -> None:
        with torch.cuda.stream(self.stream):
            _, built = _prebuild(input, self.layers)
            done = torch.cuda.Event()
            done.record(self.stream)
        self.pending[id(input)] = (input, built, done)

    def take(self, input: spTensor) -> None:
        entry = self.pending.pop(id(input), None)
        if entry is None:
            return
        _, built, done = entry
        main = torch.cuda.current_stream(input.coords.device)
        main.wait_event(done)
        for km in built:
            for t in km.device_tensors():
                t.record_stream(main)


def conv_func(input: spTensor, in_channel, out_channel, kernel, kernel_size_code, stride_code, padding_code, bias,
              transposed, tensorcore, dataflow: str = "auto", packed=None, act=None, residual=None, out=None) -> spTensor:
    """Map cache lookup / build, dataflow dispatch, bias (+ optional residual and activation, all
    inside the kernels), metadata propagation (script/spconv.py:291-464)."""
    if kernel_size_code == _UNIT and stride_code == _UNIT:
        # 1x1 stride 1: plain matrix product, coordinates unchanged, no map (script/spconv.py:297-304)
        if _wants_grad(input.feats, kernel, bias):
            _no_out_with_grad(out)
            k = kernel if kernel.dtype == input.feats.dtype else kernel.to(input.feats.dtype)
            b = bias if bias is None or bias.dtype == input.feats.dtype else bias.to(input.feats.dtype)
            return input._like(_apply_unfused(_DenseFunction.apply(input.feats, k, b), residual, act))
        if kernel.dtype != input.feats.dtype:
            kernel, packed = kernel.to(input.feats.dtype), None
        out_feats = backend.dense_forward(input.feats, kernel.detach(), packed, bias=bias, residual=residual, act=act)
        if out is not None:
            out.copy_(out_feats)
            out_feats = out
        return input._like(out_feats)

    if transposed:
        # replay the cached strided map backwards (script/spconv.py:306-329)
        output_stride = output_stride_compute(stride_code, input.stride, 1)
        km = input.kmaps.get((kernel_size_code, output_stride, stride_code))
        if km is None:
            raise KeyError("transposed conv3d found no cached map for this (kernel, stride): "
                           "the matching strided conv3d must run first on the same tensor family")
        out_coords = input.cbook[output_stride]
        out_feats = _run(input, km, kernel, in_channel, out_channel, True, dataflow, packed, bias, residual, act, out)
        output = spTensor(feats=out_feats, coords=out_coords, buffer=input.buffer, batchsize=input.batchsize,
                          stride=output_stride, init_tag=input.init_tag, coords_max=input.coords_max,
                          coords_min=input.coords_min)
        output.kmaps, output.cbook = input.kmaps, input.cbook
        return output

    km, output_stride, coords_min, coords_max = ensure_map(input, kernel_size_code, stride_code, padding_code)
    out_feats = _run(input, km, kernel, in_channel, out_channel, False, dataflow, packed, bias, residual, act, out)
    output = spTensor(feats=out_feats, coords=km.out_coords, buffer=input.buffer, batchsize=input.batchsize,
                      stride=output_stride, init_tag=input.init_tag, coords_max=coords_max, coords_min=coords_min)
    output.kmaps, output.cbook = input.kmaps, input.cbook
    return output
