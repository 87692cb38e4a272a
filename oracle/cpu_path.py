"""PyTorch CPU restatement of the hot path, timed by bench.py as the CPU baseline.
TEST / MEASUREMENT INFRASTRUCTURE ONLY (same rules as oracle/oracle.py).

The reference has no CPU path; this is its semantics in the plainest multi-threaded form:
exact-key map construction (oracle.kernel_map: sorted keys + searchsorted), then the centre
GEMM and one ``index_add_`` of ``feats[imap_k] @ W[k]`` per offset
(backend/spconv.cu:273-298 and backend/spconv.cuh:427-530).  fp32 arithmetic; fp16 workloads
are run on fp16-rounded inputs.
"""
from __future__ import annotations

import time

import numpy as np
import torch

from . import oracle as orc


def conv_forward_torch(feats: torch.Tensor, weight: torch.Tensor, km: orc.KernelMap, ks) -> torch.Tensor:
    out = feats @ weight[orc.mid_offset(ks)] if km.subm else torch.zeros((km.n_out, weight.shape[2]), dtype=feats.dtype)
    imap = torch.as_tensor(km.imap.astype(np.int64))
    omap = torch.as_tensor(km.omap.astype(np.int64))
    for kp in range(km.kv):
        a, b = int(km.kpos[kp]), int(km.kpos[kp + 1])
        if a < b:
            out.index_add_(0, omap[a:b], feats[imap[a:b]] @ weight[kp])
    return out


def time_layer(coords: np.ndarray, feats: np.ndarray, weight: np.ndarray, ks=(3, 3, 3), warmup: int = 3, runs: int = 10):
    """Median milliseconds of (map build, conv forward) on the host cores."""
    f = torch.as_tensor(feats, dtype=torch.float32)
    w = torch.as_tensor(weight, dtype=torch.float32)
    tm, tc = [], []
    km = None
    for it in range(warmup + runs):
        t0 = time.perf_counter()
        km = orc.kernel_map(coords, ks)
        t1 = time.perf_counter()
        out = conv_forward_torch(f, w, km, ks)
        t2 = time.perf_counter()
        if it >= warmup:
            tm.append((t1 - t0) * 1e3)
            tc.append((t2 - t1) * 1e3)
    return float(np.median(tm)), float(np.median(tc)), out.numpy(), km
