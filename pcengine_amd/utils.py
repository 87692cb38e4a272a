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


def _as_tensor(v):
    return torch.from_numpy(v) if isinstance(v, np.ndarray) else v


def sparse_collate(inputs: List[spTensor]) -> spTensor:
    """Samples stacked into one batch: sample ``k`` contributes its rows with ``k`` prepended as coordinate column 0,
    in the order given; numpy members are converted (and left converted on the sample, as the reference leaves
    them); all samples must share one tensor stride.  The batch's box is [0, max of the spatial columns]
    (behaviour of script/utils.py:167-196)."""
    if len(inputs) == 0:
        raise ValueError("sparse_collate needs at least one sample")
    stride = inputs[0].stride
    sizes = []
    for sample in inputs:
        sample.coords, sample.feats = _as_tensor(sample.coords), _as_tensor(sample.feats)
        for member in (sample.coords, sample.feats):
            if not isinstance(member, torch.Tensor):
                raise AssertionError(type(member))
        if sample.stride != stride:
            raise AssertionError((sample.stride, stride))
        sizes.append(sample.coords.shape[0])
    spatial = torch.cat([sample.coords.int() for sample in inputs], dim=0)
    index = torch.repeat_interleave(torch.arange(len(inputs), dtype=torch.int32, device=spatial.device),
                                    torch.tensor(sizes, device=spatial.device))
    coords = torch.cat((index.unsqueeze(1), spatial), dim=1)
    feats = torch.cat([sample.feats for sample in inputs], dim=0)
    upper = [int(v) for v in spatial.amax(dim=0).tolist()]
    return spTensor(coords=coords, feats=feats, stride=stride, batchsize=len(inputs), buffer=None,
                    coords_min=[0, 0, 0], coords_max=upper)


def sparse_collate_fn(inputs: List[Any]) -> Any:
    """Collate function for a data loader whose samples are dictionaries: per key, nested dictionaries recurse,
    arrays and tensors are concatenated along rows, sparse tensors go through ``sparse_collate``, anything else
    stays a list; samples that are not dictionaries are returned as they came (behaviour of script/utils.py:199-217)."""
    head = inputs[0]
    if not isinstance(head, dict):
        return inputs
    joiners = ((dict, sparse_collate_fn),
               (np.ndarray, lambda vals: torch.cat([torch.from_numpy(v) for v in vals], dim=0)),
               (torch.Tensor, lambda vals: torch.cat(vals, dim=0)),
               (spTensor, sparse_collate))
    batch = {}
    for key, first in head.items():
        column = [sample[key] for sample in inputs]
        join = next((fn for kind, fn in joiners if isinstance(first, kind)), None)
        batch[key] = column if join is None else join(column)
    return batch


def make_ntuple(x, ndim: int) -> Tuple[int, ...]:
    """``x`` as a tuple of ``ndim`` entries: an int is repeated, a list or a tensor is spread out; anything that
    does not end up with ``ndim`` entries fails the assertion (behaviour of script/utils.py:220-230)."""
    if isinstance(x, torch.Tensor):
        x = x.reshape(-1).tolist()
    if isinstance(x, int):
        x = (x,) * ndim
    elif isinstance(x, list):
        x = tuple(x)
    assert isinstance(x, tuple) and len(x) == ndim, x
    return x
