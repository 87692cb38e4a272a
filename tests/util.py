"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

from oracle import oracle as orc
from pcengine_amd import backend

DEV = "cuda:0"
TOL = {torch.float16: 1e-3, torch.float32: 1e-5}   # rel-L2 bars of the parity contract


def dev_coords(coords: np.ndarray) -> torch.Tensor:
    return torch.as_tensor(np.ascontiguousarray(coords, np.int32), device=DEV)


def gpu_map(coords: np.ndarray, ks, stride=(1, 1, 1), pad=(0, 0, 0), **kw) -> backend.KernelMap:
    subm = tuple(stride) == (1, 1, 1)
    cmax = coords[:, 1:].max(axis=0).tolist()
    if not subm:
        cmax = orc.strided_coords_max(cmax, ks, stride, pad)
    return backend.build_kernel_map(dev_coords(coords), ks, stride, pad, [0, 0, 0], cmax, subm, **kw)


def assert_map_equal(km: backend.KernelMap, ref: orc.KernelMap, csr: bool = False):
    assert km.n_in == ref.n_in and km.n_out == ref.n_out and km.M == ref.M and km.qsum == ref.qsum
    assert np.array_equal(km.out_coords.cpu().numpy(), ref.out_coords)
    assert np.array_equal(km.knnz.cpu().numpy(), ref.knnz)
    assert np.array_equal(km.kpos.cpu().numpy(), ref.kpos)
    assert np.array_equal(km.qkpos.cpu().numpy(), ref.qkpos)
    assert np.array_equal(km.imap.cpu().numpy(), ref.imap)
    assert np.array_equal(km.omap.cpu().numpy(), ref.omap)
    if km.nbr_out is not None:
        want = orc.dense_neighbour_table(ref)
        if ref.subm:
            want[orc.mid_offset(km.ks)] = np.arange(ref.n_out)
        assert np.array_equal(km.nbr_out.cpu().numpy().reshape(ref.kv, ref.n_out), want)
    if km.nbr_in is not None:
        want = -np.ones((ref.kv, ref.n_in), np.int32)
        kp_of = np.repeat(np.arange(ref.kv), ref.knnz.astype(np.int64))
        want[kp_of, ref.imap] = ref.omap
        assert np.array_equal(km.nbr_in.cpu().numpy().reshape(ref.kv, ref.n_in), want)
    if csr:
        icsr, icode, ocsr, ocode = orc.csr_maps(ref)
        assert np.array_equal(km.icsr.cpu().numpy(), icsr)
        assert np.array_equal(km.ocsr.cpu().numpy(), ocsr)
        assert np.array_equal(km.icode.cpu().numpy(), icode)
        assert np.array_equal(km.ocode.cpu().numpy(), ocode)
        # slot arrays are the inverse permutations of the CSR orders: entry slot[p] of the coded list is pair p
        kp_of = np.repeat(np.arange(ref.kv), ref.knnz.astype(np.int64))
        pair_code = (kp_of * orc.CSR_CODE + (np.arange(ref.M) - ref.kpos[:-1].astype(np.int64)[kp_of])).astype(np.int32)
        for slot, code in ((km.islot, icode), (km.oslot, ocode)):
            sl = slot.cpu().numpy()
            assert np.array_equal(np.sort(sl), np.arange(ref.M)) and np.array_equal(code[sl], pair_code)


def rounded(a: np.ndarray, dtype: torch.dtype) -> np.ndarray:
    """Values as the GPU sees them: rounded to the storage type, back in float64."""
    return torch.as_tensor(a).to(dtype).double().numpy()
