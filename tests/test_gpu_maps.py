"""Bit-exact parity of the HIP hash / output-coordinate / kernel-map path with the CPU oracle.
Everything goes through the C ABI (ctypes)."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from pcengine_amd import _lib, backend, synth
from tests.util import DEV, assert_map_equal, dev_coords, gpu_map

pytestmark = pytest.mark.gpu

GEOMS = [
    ((3, 3, 3), (1, 1, 1), (0, 0, 0)),
    ((2, 2, 2), (2, 2, 2), (0, 0, 0)),
    ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
    ((3, 3, 3), (2, 2, 2), (0, 0, 0)),
    ((3, 1, 3), (1, 1, 1), (0, 0, 0)),
    ((2, 3, 1), (2, 1, 1), (0, 1, 0)),
    ((5, 5, 5), (1, 1, 1), (0, 0, 0)),
    ((1, 1, 1), (2, 2, 2), (0, 0, 0)),
]


def test_hash_build_and_query_membership():
    lib = _lib.load()
    coords = synth.random_cloud(seed=7, n=50000, extent=60, batches=3)
    n = len(coords)
    slots = lib.pce_hash_slots(n)
    assert slots == 2 * 2 ** int(np.ceil(np.log2(n)))          # backend/hash.cu:46
    table = torch.empty(lib.pce_hash_table_bytes(n), dtype=torch.uint8, device=DEV)
    status = torch.zeros(2, dtype=torch.int32, device=DEV)
    c = dev_coords(coords)
    s = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.pce_hash_build(table.data_ptr(), slots, c.data_ptr(), n, status.data_ptr(), s))
    # every inserted key is found at its own row; shifted keys are found iff they are members
    rng = np.random.default_rng(0)
    q = coords.copy()
    q[:, 1:] += rng.integers(-2, 3, size=(n, 3)).astype(np.int32)
    qd = dev_coords(np.concatenate([coords, q]))
    rows = torch.empty(2 * n, dtype=torch.int32, device=DEV)
    _lib.check(lib.pce_hash_query(table.data_ptr(), slots, qd.data_ptr(), 2 * n, rows.data_ptr(), s))
    rows = rows.cpu().numpy()
    assert status.cpu().tolist() == [0, 0]
    assert np.array_equal(rows[:n], np.arange(n))
    assert np.array_equal(rows[n:], orc.CoordIndex(coords).find(q))


def test_hash_duplicate_keys_keep_smallest_row():
    lib = _lib.load()
    coords = np.array([[0, 1, 2, 3], [0, 4, 5, 6], [0, 1, 2, 3], [0, 1, 2, 3]], np.int32)
    slots = lib.pce_hash_slots(4)
    table = torch.empty(lib.pce_hash_table_bytes(4), dtype=torch.uint8, device=DEV)
    status = torch.zeros(2, dtype=torch.int32, device=DEV)
    c = dev_coords(coords)
    s = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.pce_hash_build(table.data_ptr(), slots, c.data_ptr(), 4, status.data_ptr(), s))
    rows = torch.empty(4, dtype=torch.int32, device=DEV)
    _lib.check(lib.pce_hash_query(table.data_ptr(), slots, c.data_ptr(), 4, rows.data_ptr(), s))
    assert rows.cpu().tolist() == [0, 1, 0, 0]


@pytest.mark.parametrize("ks,stride,pad", GEOMS)
@pytest.mark.parametrize("seed,n,extent,batches", [(11, 500, 9, 3), (12, 20000, 40, 2), (13, 63, 5, 1), (14, 1, 3, 1)])
def test_kernel_map_bit_exact(ks, stride, pad, seed, n, extent, batches):
    coords = synth.random_cloud(seed=seed, n=n, extent=extent, batches=batches)
    ref = orc.kernel_map(coords, ks, stride, pad)
    if ref.n_out == 0:
        with pytest.raises(ValueError):
            gpu_map(coords, ks, stride, pad)
        return
    km = gpu_map(coords, ks, stride, pad, want_csr=True, want_nbr_out=True, want_nbr_in=True)
    assert_map_equal(km, ref, csr=True)


def test_kernel_map_config1_and_determinism():
    coords = synth.sphere_plane_cloud()
    ref = orc.kernel_map(coords, (3, 3, 3))
    a = gpu_map(coords, (3, 3, 3), want_csr=True, want_nbr_in=True)
    b = gpu_map(coords, (3, 3, 3), want_csr=True, want_nbr_in=True)
    assert_map_equal(a, ref, csr=True)
    for name in ("imap", "omap", "icode", "ocode", "icsr", "ocsr", "nbr_out", "nbr_in", "qkpos"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name


def test_kernel_map_config2_lidar_full_size():
    coords = synth.lidar_cloud()
    ref = orc.kernel_map(coords, (3, 3, 3))
    assert_map_equal(gpu_map(coords, (3, 3, 3), want_csr=True), ref, csr=True)
    ref2 = orc.kernel_map(coords, (2, 2, 2), (2, 2, 2))
    km2 = gpu_map(coords, (2, 2, 2), (2, 2, 2), want_csr=True, want_nbr_in=True)
    assert_map_equal(km2, ref2, csr=True)
    # size-independent properties of a k2s2 map: every input is in exactly one pair
    assert km2.M == len(coords)
    assert torch.equal(torch.sort(km2.imap).values, torch.arange(len(coords), dtype=torch.int32, device=DEV))
    oc = km2.out_coords.cpu().numpy().astype(np.int64)
    code = ((oc[:, 0] * 3259 + oc[:, 1]) * 3259 + oc[:, 2]) * 3259 + oc[:, 3]
    assert (np.diff(code) > 0).all()      # strictly ascending (b,x,y,z)


def test_unsorted_input_rows():
    coords = synth.random_cloud(seed=31, n=5000, extent=20, batches=2)
    coords = coords[np.random.default_rng(1).permutation(len(coords))]
    for ks, stride, pad in GEOMS[:4]:
        assert_map_equal(gpu_map(coords, ks, stride, pad, want_csr=True), orc.kernel_map(coords, ks, stride, pad), csr=True)


def test_indoor_scene_batch2():
    coords = synth.indoor_batch(seed=5, scenes=2, n_room=40000, n_box=800)
    assert_map_equal(gpu_map(coords, (3, 3, 3), want_csr=True), orc.kernel_map(coords, (3, 3, 3)), csr=True)
    assert_map_equal(gpu_map(coords, (2, 2, 2), (2, 2, 2)), orc.kernel_map(coords, (2, 2, 2), (2, 2, 2)))


def test_error_paths():
    bad = np.array([[0, 1, 2, 3], [0, 40000, 0, 0]], np.int32)
    with pytest.raises(ValueError):
        gpu_map(bad, (3, 3, 3))
    with pytest.raises(ValueError):      # not int32 [N,4]
        backend.build_kernel_map(torch.zeros((4, 3), dtype=torch.int32, device=DEV), (3, 3, 3), (1, 1, 1), (0, 0, 0),
                                 [0, 0, 0], [1, 1, 1], True)
    with pytest.raises(RuntimeError):    # host tensor: no CPU compute path
        backend.build_kernel_map(torch.zeros((4, 4), dtype=torch.int32), (3, 3, 3), (1, 1, 1), (0, 0, 0), [0, 0, 0],
                                 [1, 1, 1], True)
    lib = _lib.load()
    rc = lib.pce_kmap_build(None, 1, None, 1, None, None, 0, *([None] * 14), None)
    assert rc == _lib.PCE_EINVAL and b"null" in lib.pce_last_error()
