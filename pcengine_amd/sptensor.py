"""Sparse tensor container with the reference's fields and aliases (script/sptensor.py:4-91).

A tensor is a coordinate list ``coords`` (int32 [N, 4] = batch, x, y, z) and a feature matrix ``feats`` [N, C].
What convolutions learn about the coordinates travels with it: ``kmaps`` caches the kernel map of every
(kernel size, tensor stride, layer stride) seen so far, ``cbook`` the coordinate list of every tensor stride.
Both dictionaries are shared, not copied, by every tensor derived from the same input, so a map built in the
encoder is found again by the decoder.  ``init_tag`` is the reference's dataflow tag list: 'D1' / 'D2' entries
are consumed one per newly built map, 'end' (or no list) leaves the choice to the selector.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

DEFAULT_STRIDE_CODE = 94585  # (1,1,1) packed as 94273*x + 311*y + z

# rows of staging buffer per input row that the reference reserves for gather-GEMM-scatter, by kernel size
# (script/sptensor.py:63-78); other sizes reserve the full kernel volume
_BUFFER_ROWS_PER_VOXEL = {2: 8, 3: 16, 5: 48}


class _Alias:
    """A second name for an attribute (``F`` for ``feats``, ``C`` for ``coords``)."""

    def __init__(self, target: str):
        self.target = target

    def __get__(self, obj, owner=None):
        return self if obj is None else getattr(obj, self.target)

    def __set__(self, obj, value) -> None:
        setattr(obj, self.target, value)


class spTensor:
    F = _Alias("feats")
    C = _Alias("coords")

    def __init__(self, feats: torch.Tensor, coords: torch.Tensor, buffer: Optional[torch.Tensor] = None,
                 coords_min: Optional[list] = None, coords_max: Optional[list] = None, batchsize: int = 1,
                 stride: int = DEFAULT_STRIDE_CODE, init_tag: Optional[List[str]] = None) -> None:
        self.feats, self.coords, self.buffer = feats, coords, buffer
        self.stride, self.batchsize = stride, batchsize
        self.kmaps: Dict = {}
        self.cbook: Dict = {}
        self.init_tag = init_tag if init_tag is not None else ['end']
        self.coords_min = coords_min if coords_min is not None else [0, 0, 0]
        if coords_max is None:      # one read-back; callers that know the extent pass it
            coords_max = coords[:, 1:].max(dim=0).values.cpu().tolist()
        self.coords_max = coords_max

    # -- movement: in place, returning self, as the reference's methods do -------------------------------
    def _moved(self, fn) -> "spTensor":
        self.coords, self.feats = fn(self.coords), fn(self.feats)
        return self

    def cpu(self) -> "spTensor":
        return self._moved(lambda t: t.cpu())

    def cuda(self) -> "spTensor":
        return self._moved(lambda t: t.cuda())

    def detach(self) -> "spTensor":
        return self._moved(lambda t: t.detach())

    def to(self, device, non_blocking: bool = True) -> "spTensor":
        return self._moved(lambda t: t.to(device, non_blocking=non_blocking))

    # -- derived tensors ------------------------------------------------------------------------------
    def _like(self, feats: torch.Tensor) -> "spTensor":
        """New features on the same coordinates; the map cache and the coordinate book stay shared."""
        out = spTensor(feats, self.coords, self.buffer, self.coords_min, self.coords_max, self.batchsize, self.stride,
                       self.init_tag)
        out.kmaps, out.cbook = self.kmaps, self.cbook
        return out

    def __add__(self, other: "spTensor") -> "spTensor":
        return self._like(self.feats + other.feats)

    def __len__(self) -> int:
        return int(self.coords.shape[0])

    def __repr__(self) -> str:
        return (f"spTensor(N={len(self)}, C={self.feats.shape[1] if self.feats.dim() > 1 else 1}, "
                f"dtype={self.feats.dtype}, device={self.feats.device}, stride_code={self.stride})")

    def build_buffer(self, cinfo: Dict, device) -> None:
        """Staging buffer for gather-GEMM-scatter, sized as the reference sizes it: (widest input + widest
        output) channels times the rows reserved per voxel, fp32, zero-filled."""
        ks = max(cinfo["kernel"])
        rows = len(self) * _BUFFER_ROWS_PER_VOXEL.get(ks, ks ** 3)
        width = max(cinfo["in"]) + max(cinfo["out"])
        self.buffer = torch.zeros(width * rows, dtype=torch.float, device=device)
