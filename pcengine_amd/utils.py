"""Front-end helpers with the reference's names and meaning (script/utils.py)."""
from __future__ import annotations

from itertools import repeat
from typing import Any, Callable, Dict, List, Tuple, Union

import numpy as np
import torch

from .sptensor import spTensor

_A, _B = 94273, 311


def conv_info_encoder(info) -> int:
    """script/utils.py:233-234."""
    return _A * info[0] + _B * info[1] + info[2]


def conv_info_decoder(code: int) -> Tuple[int, int, int]:
    """script/utils.py:237-242."""
    x = code // _A
    rest = code - x * _A
    return (x, rest // _B, rest - rest // _B * _B)


def output_stride_compute(l_stride_code: int, t_stride_code: int, transposed: bool = False) -> int:
    """Tensor stride after a layer: product for a conv, quotient for a transposed conv
    (script/utils.py:116-138)."""
    ls, ts = conv_info_decoder(l_stride_code), conv_info_decoder(t_stride_code)
    if transposed:
        return conv_info_encoder([t // l for t, l in zip(ts, ls)])
    return conv_info_encoder([t * l for t, l in zip(ts, ls)])


def load_file(file_name):
    """script/utils.py:11-15; needs open3d, which is optional."""
    try:
        import open3d as o3d
    except ImportError as e:  # pragma: no cover
        raise ImportError("load_file needs open3d, which is not installed") from e
    pcd = o3d.io.read_point_cloud(file_name)
    return np.array(pcd.points), np.array(pcd.colors), pcd


def ravel_hash(x: np.ndarray) -> np.ndarray:
    """Mixed-radix code of integer rows (script/utils.py:18-30)."""
    assert x.ndim == 2, x.shape
    x = (x - x.min(axis=0)).astype(np.uint64, copy=False)
    radix = x.max(axis=0).astype(np.uint64) + 1
    h = np.zeros(x.shape[0], dtype=np.uint64)
    for k in range(x.shape[1] - 1):
        h = (h + x[:, k]) * radix[k + 1]
    return h + x[:, -1]


def sparse_quantize(coords, voxel_size: Union[float, Tuple[float, ...]] = 1, *, return_index: bool = False,
                    return_inverse: bool = False):
    """floor(coords / voxel) and one representative per voxel (script/utils.py:33-55).

    A NumPy array is handled on the host exactly as in the reference; a device tensor [P,3] goes
    through the GPU voxelisation and device tensors come back (coords int32 [V,3], indices int64)."""
    if isinstance(voxel_size, (float, int)):
        voxel_size = tuple(repeat(voxel_size, 3))
    assert isinstance(voxel_size, tuple) and len(voxel_size) == 3
    if isinstance(coords, torch.Tensor) and coords.is_cuda:
        from . import backend
        res = backend.voxelize(coords, voxel_size, 0, return_index=return_index, return_inverse=return_inverse)
        outs = [res[0][:, 1:].contiguous()] + [t.long() for t in res[1:-1]]
        return outs[0] if len(outs) == 1 else outs
    q = np.floor(coords / np.array(voxel_size)).astype(np.int32)
    _, idx, inv = np.unique(ravel_hash(q), return_index=True, return_inverse=True)
    outs = [q[idx]]
    if return_index:
        outs.append(idx)
    if return_inverse:
        outs.append(inv)
    return outs[0] if len(outs) == 1 else outs


def build_conv_buffer(channel_list: Dict, nnz: int, data_type, device):
    """script/utils.py:58-79."""
    ks = max(channel_list["kernel"])
    factor = {3: 16, 5: 48, 2: 8}.get(ks, ks ** 3 - 1)
    size = (max(channel_list["in"]) + max(channel_list["out"])) * nnz * factor
    return torch.zeros((size,), dtype=data_type, device=device)


def init_layer_scheduler(conv_info: Dict) -> str:
    """The reference's (uncalled) hint: layers at the input resolution wider than 32 channels
    should not use the simple fetch-on-demand map (script/utils.py:82-113)."""
    stride, cin, cout = conv_info['stride'], conv_info['in'], conv_info['out']
    for i, s in enumerate(stride):
        if s > 1:
            break
        if cin[i] > 32 or cout[i] > 32:
            return 'whole'
    return 'simple'


def fapply(input: spTensor, fn: Callable[..., torch.Tensor], *args, **kwargs) -> spTensor:
    """Apply a feature-only function, keep coordinates and shared metadata (script/utils.py:141-149)."""
    return input._like(fn(input.feats, *args, **kwargs))


def cat(inputs: List[spTensor]) -> spTensor:
    """Channel concatenation of tensors on the same coordinates (script/utils.py:152-164)."""
    feats = [x.feats for x in inputs]
    if len(feats) == 2:
        return inputs[0]._like(_Concat2.apply(feats[0], feats[1]))
    return inputs[0]._like(torch.cat(feats, dim=1))


class _Concat2(torch.autograd.Function):
    """Two feature matrices side by side: one streaming kernel of the library where the layout fits it
    (torch.cat is three times off the memory roofline on [10^6, C] matrices), torch.cat otherwise."""

    @staticmethod
    def forward(ctx, a, b):
        from . import backend
        ctx.split = a.shape[1]
        out = backend.concat_cols(a, b)
        return out if out is not None else torch.cat([a, b], dim=1)

    @staticmethod
    def backward(ctx, grad):
        return grad[:, :ctx.split], grad[:, ctx.split:]


def sparse_collate(inputs: List[spTensor]) -> spTensor:
    """Stack samples, batch index in coordinate column 0 (script/utils.py:167-196)."""
    coords, feats = [], []
    stride = inputs[0].stride
    for k, x in enumerate(inputs):
        if isinstance(x.coords, np.ndarray):
            x.coords = torch.tensor(x.coords)
        if isinstance(x.feats, np.ndarray):
            x.feats = torch.tensor(x.feats)
        assert isinstance(x.coords, torch.Tensor), type(x.coords)
        assert isinstance(x.feats, torch.Tensor), type(x.feats)
        assert x.stride == stride, (x.stride, stride)
        b = torch.full((x.coords.shape[0], 1), k, device=x.coords.device, dtype=torch.int)
        coords.append(torch.cat((b, x.coords.int()), dim=1))
        feats.append(x.feats)
    coords = torch.cat(coords, dim=0)
    feats = torch.cat(feats, dim=0)
    cmax = coords[:, 1:].max(dim=0).values.cpu().numpy().tolist()
    return spTensor(coords=coords, feats=feats, stride=stride, batchsize=len(inputs), buffer=None,
                    coords_min=[0, 0, 0], coords_max=cmax)


def sparse_collate_fn(inputs: List[Any]) -> Any:
    """script/utils.py:199-217."""
    if not isinstance(inputs[0], dict):
        return inputs
    out = {}
    for name, first in inputs[0].items():
        vals = [x[name] for x in inputs]
        if isinstance(first, dict):
            out[name] = sparse_collate_fn(vals)
        elif isinstance(first, np.ndarray):
            out[name] = torch.cat([torch.tensor(v) for v in vals], dim=0)
        elif isinstance(first, torch.Tensor):
            out[name] = torch.cat(vals, dim=0)
        elif isinstance(first, spTensor):
            out[name] = sparse_collate(vals)
        else:
            out[name] = vals
    return out


def make_ntuple(x, ndim: int) -> Tuple[int, ...]:
    """script/utils.py:220-230."""
    if isinstance(x, int):
        x = tuple(repeat(x, ndim))
    elif isinstance(x, list):
        x = tuple(x)
    elif isinstance(x, torch.Tensor):
        x = tuple(x.view(-1).cpu().numpy().tolist())
    assert isinstance(x, tuple) and len(x) == ndim, x
    return x
