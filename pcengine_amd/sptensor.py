"""Sparse tensor container with the reference's fields and aliases (script/sptensor.py:4-91)."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

DEFAULT_STRIDE_CODE = 94585  # (1,1,1) packed as 94273*x + 311*y + z


class spTensor:
    """coords int32 [N,4] = (b,x,y,z), feats [N,C]; ``kmaps`` and ``cbook`` are shared by
    reference among all tensors derived from one input, ``init_tag`` is the dataflow tag list
    ('D1' / 'D2' entries consumed one per newly built map, 'end' or None = automatic)."""

    def __init__(self, feats: torch.Tensor, coords: torch.Tensor, buffer: Optional[torch.Tensor] = None,
                 coords_min: Optional[list] = None, coords_max: Optional[list] = None, batchsize: int = 1,
                 stride: int = DEFAULT_STRIDE_CODE, init_tag: Optional[List[str]] = None) -> None:
        self.feats = feats
        self.coords = coords
        self.stride = stride
        self.batchsize = batchsize
        self.buffer = buffer
        self.kmaps: Dict = {}
        self.cbook: Dict = {}
        self.init_tag = ['end'] if init_tag is None else init_tag
        self.coords_min = [0, 0, 0] if coords_min is None else coords_min
        if coords_max is None:
            coords_max = coords[:, 1:].max(dim=0).values.cpu().tolist()
        self.coords_max = coords_max

    @property
    def F(self) -> torch.Tensor:
        return self.feats

    @F.setter
    def F(self, feats: torch.Tensor) -> None:
        self.feats = feats

    @property
    def C(self) -> torch.Tensor:
        return self.coords

    @C.setter
    def C(self, coords: torch.Tensor) -> None:
        self.coords = coords

    def cpu(self):
        self.coords, self.feats = self.coords.cpu(), self.feats.cpu()
        return self

    def cuda(self):
        self.coords, self.feats = self.coords.cuda(), self.feats.cuda()
        return self

    def detach(self):
        self.coords, self.feats = self.coords.detach(), self.feats.detach()
        return self

    def to(self, device, non_blocking: bool = True):
        self.coords = self.coords.to(device, non_blocking=non_blocking)
        self.feats = self.feats.to(device, non_blocking=non_blocking)
        return self

    def build_buffer(self, cinfo: Dict, device) -> None:
        """Staging buffer for gather-GEMM-scatter sized as the reference sizes it
        (script/sptensor.py:63-78): (max C_in + max C_out) * N * {16, 48, 8, k^3} elements."""
        per_row = {3: 16, 5: 48, 2: 8}
        ks = max(cinfo["kernel"])
        factor = per_row.get(ks, ks ** 3)
        n = self.coords.size(0)
        self.buffer = torch.zeros(((max(cinfo["in"]) + max(cinfo["out"])) * n * factor,), dtype=torch.float, device=device)

    def _like(self, feats: torch.Tensor) -> "spTensor":
        out = spTensor(feats=feats, coords=self.coords, buffer=self.buffer, coords_min=self.coords_min,
                       coords_max=self.coords_max, batchsize=self.batchsize, stride=self.stride, init_tag=self.init_tag)
        out.kmaps, out.cbook = self.kmaps, self.cbook
        return out

    def __add__(self, other: "spTensor") -> "spTensor":
        return self._like(self.feats + other.feats)
