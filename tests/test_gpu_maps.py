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
    ((2, 2, 2), (1, 1, 1), (0, 0, 0)),   # stride 1 with even kernel sizes: the map has no mirror symmetry
    ((2, 3, 3), (1, 1, 1), (0, 0, 0)),
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
    # the same layer with the batch count stated: neighbours are looked up in the column grid instead of the hash
    # table, and a strided layer takes the occupancy-bitmap route to its output coordinates
    kb = gpu_map(coords, ks, stride, pad, want_csr=True, want_nbr_out=True, want_nbr_in=True, batchsize=batches)
    assert_map_equal(kb, ref, csr=True)


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
    assert torch.equal(gpu_map(coords, (2, 2, 2), (2, 2, 2), batchsize=1).out_coords, km2.out_coords)
    # size-independent properties of a k2s2 map: every input is in exactly one pair
    assert km2.M == len(coords)
    assert torch.equal(torch.sort(km2.imap).values, torch.arange(len(coords), dtype=torch.int32, device=DEV))
    oc = km2.out_coords.cpu().numpy().astype(np.int64)
    code = ((oc[:, 0] * 3259 + oc[:, 1]) * 3259 + oc[:, 2]) * 3259 + oc[:, 3]
    assert (np.diff(code) > 0).all()      # strictly ascending (b,x,y,z)


def _request(coords, ks, stride, pad, **kw):
    subm = tuple(stride) == (1, 1, 1)
    cmax = coords[:, 1:].max(axis=0).tolist()
    if not subm:
        cmax = orc.strided_coords_max(cmax, ks, stride, pad)
    return dict(in_coords=dev_coords(coords), ks=ks, stride=stride, pad=pad, cmin=[0, 0, 0], cmax_out=cmax, subm=subm, **kw)


@pytest.mark.parametrize("defer", [False, True])
def test_kernel_maps_batched_build_bit_exact(defer):
    """Several layers per call: every stage of the build is one launch over all problems.  Mixed
    geometries, sizes from one row to 20k, with and without the optional outputs; 19 problems, so the
    call is split into two batches."""
    cases = []
    for k, (ks, stride, pad) in enumerate(GEOMS + GEOMS + GEOMS[:3]):
        n, extent, batches = [(500, 9, 3), (20000, 40, 2), (63, 5, 1), (1, 3, 1), (3000, 20, 1)][k % 5]
        coords = synth.random_cloud(seed=100 + k, n=n, extent=extent, batches=batches)
        ref = orc.kernel_map(coords, ks, stride, pad)
        if ref.n_out == 0:
            continue
        full = k % 3 != 2
        cases.append((ref, full, _request(coords, ks, stride, pad, want_csr=full, want_nbr_out=True, want_nbr_in=full,
                                          batchsize=batches if k % 2 else 0)))
    assert len(cases) > backend.KMAP_MAX_BATCH
    maps = backend.build_kernel_maps([c[2] for c in cases], defer=defer)
    if defer:
        torch.cuda.synchronize()
        maps = [m.finish() for m in maps]
    for (ref, full, _), km in zip(cases, maps):
        assert_map_equal(km, ref, csr=full)


def test_kernel_maps_batch_argument_errors():
    lib = _lib.load()
    probs = (_lib.KmapProblem * 1)()
    assert lib.pce_kmap_build_batch(probs, 0, None) == _lib.PCE_EINVAL
    assert lib.pce_kmap_build_batch(probs, backend.KMAP_MAX_BATCH + 1, None) == _lib.PCE_EINVAL
    assert lib.pce_kmap_build_batch(probs, 1, None) == _lib.PCE_EINVAL          # zeroed problem: bad geometry
    assert backend.build_kernel_maps([]) == []


def _out_coords(coords, ks, stride, pad, cmin, cmax_out, n_batch):
    geom = _lib.Geom.make(ks, stride, pad, cmin, cmax_out, False)
    return backend.build_out_coords(dev_coords(coords), geom, n_batch).cpu().numpy()


@pytest.mark.parametrize("n_batch", [0, 4])
def test_out_coords_clipped_to_bounds(n_batch):
    """Bounds that cut candidates away on both sides, hash/sort and bitmap routes alike."""
    coords = synth.random_cloud(seed=41, n=30000, extent=50, batches=4)
    for ks, stride, pad, cmin, cmax in [((3, 3, 3), (2, 2, 2), (1, 1, 1), (3, 0, 5), (17, 25, 11)),
                                        ((2, 2, 2), (2, 2, 2), (0, 0, 0), (0, 2, 0), (24, 9, 24)),
                                        ((3, 2, 1), (2, 2, 1), (0, 0, 0), (1, 1, 1), (20, 20, 30))]:
        want = orc.out_coords_strided(coords, ks, stride, pad, cmin, cmax)
        got = _out_coords(coords, ks, stride, pad, cmin, cmax, n_batch)
        assert len(want) > 0 and np.array_equal(got, want)


def test_out_coords_bitmap_rejects_large_batch_index_and_front_end_recovers():
    lib = _lib.load()
    coords = synth.random_cloud(seed=42, n=4000, extent=20, batches=3)
    geom = _lib.Geom.make((2, 2, 2), (2, 2, 2), (0, 0, 0), [0, 0, 0], [9, 9, 9], False)
    c = dev_coords(coords)
    ws_bytes = lib.pce_outcoords_workspace_bytes(len(coords), geom, 2)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    n_out = _lib.c_int64(0)
    rc = lib.pce_outcoords_build(c.data_ptr(), len(coords), geom, 2, ws.data_ptr(), ws_bytes, n_out,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.PCE_EINVAL and b"n_batch" in lib.pce_last_error()
    # the front end redoes the build without the bound
    want = orc.out_coords_strided(coords, (2, 2, 2), (2, 2, 2), (0, 0, 0), (0, 0, 0), (9, 9, 9))
    assert np.array_equal(backend.build_out_coords(c, geom, 2).cpu().numpy(), want)


def test_out_coords_sparse_box_falls_back_to_sort():
    """A handful of points in a huge box: the bitmap would be mostly empty, the library sorts."""
    lib = _lib.load()
    rng = np.random.default_rng(43)
    coords = np.unique(np.concatenate([np.zeros((300, 1), np.int64), rng.integers(0, 3000, (300, 3))], 1), axis=0).astype(np.int32)
    geom = _lib.Geom.make((2, 2, 2), (2, 2, 2), (0, 0, 0), [0, 0, 0], [1499, 1499, 1499], False)
    assert lib.pce_outcoords_workspace_bytes(len(coords), geom, 1) == lib.pce_outcoords_workspace_bytes(len(coords), geom, 0)
    want = orc.out_coords_strided(coords, (2, 2, 2), (2, 2, 2), (0, 0, 0), (0, 0, 0), (1499, 1499, 1499))
    assert np.array_equal(backend.build_out_coords(dev_coords(coords), geom, 1).cpu().numpy(), want)


@pytest.mark.parametrize("chain", [
    [((2, 2, 2), (2, 2, 2), (0, 0, 0))] * 4,                                          # the levels of a U-Net
    [((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 2, 1), (2, 2, 1), (0, 0, 0))],
    [((2, 2, 2), (2, 2, 2), (0, 0, 0))],
    [((3, 3, 3), (3, 3, 3), (0, 0, 0)), ((2, 3, 1), (2, 3, 1), (0, 0, 0)), ((2, 2, 2), (2, 2, 2), (0, 0, 0))],   # kernel = stride, odd sizes too
    [((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (1, 1, 1))],
])
def test_out_coords_chain_equals_the_levels_built_one_by_one(chain):
    """The chained build (the counts of the levels stay on the device, one wait of the host; chains whose layers all
    have kernel = stride and no padding mark every level in one pass over the first level's points) against the
    oracle's coordinates level by level, and against the library's own single-level build."""
    coords = synth.random_cloud(seed=44, n=40000, extent=70, batches=3)
    cmin, cmax = [0, 0, 0], coords[:, 1:].max(0).tolist()
    geoms, want, cur = [], [], coords
    for ks, stride, pad in chain:
        cmax = orc.strided_coords_max(cmax, ks, stride, pad)
        geoms.append(_lib.Geom.make(ks, stride, pad, cmin, cmax, False))
        cur = orc.out_coords_strided(cur, ks, stride, pad, cmin, cmax)
        want.append(cur)
    got = backend.build_out_coords_chain(dev_coords(coords), geoms, 3)
    assert got is not None and len(got) == len(chain)
    src = dev_coords(coords)
    for g, w, geom in zip(got, want, geoms):
        assert len(w) > 0 and np.array_equal(g.cpu().numpy(), w)
        assert torch.equal(backend.build_out_coords(src, geom, 3), g)
        src = g


def test_out_coords_chain_declines_what_it_cannot_take():
    """No batch count, a batch index beyond the stated count, a box too sparse for the bitmap: None, and the
    front end builds level by level (same maps as ever)."""
    coords = synth.random_cloud(seed=45, n=5000, extent=24, batches=3)
    k2 = ((2, 2, 2), (2, 2, 2), (0, 0, 0))
    geoms = [_lib.Geom.make(*k2, [0, 0, 0], [11, 11, 11], False), _lib.Geom.make(*k2, [0, 0, 0], [5, 5, 5], False)]
    c = dev_coords(coords)
    assert backend.build_out_coords_chain(c, geoms, 0) is None
    assert backend.build_out_coords_chain(c, geoms, 2) is None           # batch index 2 present
    assert backend.build_out_coords_chain(c, geoms, 3) is not None
    rng = np.random.default_rng(46)
    far = np.unique(np.concatenate([np.zeros((300, 1), np.int64), rng.integers(0, 3000, (300, 3))], 1), axis=0).astype(np.int32)
    sparse = [_lib.Geom.make(*k2, [0, 0, 0], [1499] * 3, False), _lib.Geom.make(*k2, [0, 0, 0], [749] * 3, False)]
    assert backend.build_out_coords_chain(dev_coords(far), sparse, 1) is None
    lib = _lib.load()
    ws, cap = (_lib.c_int64 * 2)(), (_lib.c_int64 * 2)()
    assert lib.pce_outcoords_chain_plan(len(far), 2, (_lib.Geom * 2)(*sparse), 1, ws, cap) == backend.CHAIN_NOT_APPLICABLE
    assert lib.pce_outcoords_chain_plan(len(far), 9, None, 1, ws, cap) == _lib.PCE_EINVAL


def test_unsorted_input_rows():
    coords = synth.random_cloud(seed=31, n=5000, extent=20, batches=2)
    coords = coords[np.random.default_rng(1).permutation(len(coords))]
    for ks, stride, pad in GEOMS[:4]:
        assert_map_equal(gpu_map(coords, ks, stride, pad, want_csr=True), orc.kernel_map(coords, ks, stride, pad), csr=True)
        # with the batch count stated the build starts on the column grid, finds the rows unsorted and is redone
        # through the hash table
        assert_map_equal(gpu_map(coords, ks, stride, pad, want_csr=True, batchsize=2), orc.kernel_map(coords, ks, stride, pad),
                         csr=True)


def test_column_grid_falls_back_when_its_preconditions_fail():
    """The column grid needs rows strictly ascending in (b,x,y,z), inside the stated coordinate bounds and with batch
    indices below the stated count.  Each violation is detected on the device (status word 3) and the map is built
    again through the hash table: same result as without the batch count."""
    coords = synth.random_cloud(seed=32, n=6000, extent=24, batches=3)
    ref = orc.kernel_map(coords, (3, 3, 3))
    cd = dev_coords(coords)
    cmax = coords[:, 1:].max(axis=0).tolist()
    build = lambda c, cm, nb: backend.build_kernel_map(c, (3, 3, 3), (1, 1, 1), (0, 0, 0), [0, 0, 0], cm, True, want_csr=True,
                                                       batchsize=nb)
    assert_map_equal(build(cd, cmax, 3), ref, csr=True)                       # the grid itself
    assert_map_equal(build(cd, cmax, 2), ref, csr=True)                       # a batch index beyond the stated count
    assert_map_equal(build(cd, [c - 5 for c in cmax], 3), ref, csr=True)      # rows beyond the stated bounds
    swapped = coords.copy()
    swapped[[10, 11]] = swapped[[11, 10]]                                     # one inversion
    assert_map_equal(build(dev_coords(swapped), cmax, 3), orc.kernel_map(swapped, (3, 3, 3)), csr=True)
    # a long column (a wall): more rows in z than the four a probe reads ahead
    wall = np.array([[0, x, 7, z] for x in range(3) for z in range(0, 60)] + [[0, 5, 5, 5]], np.int32)
    wall = wall[np.lexsort((wall[:, 3], wall[:, 2], wall[:, 1], wall[:, 0]))]
    assert_map_equal(build(dev_coords(wall), wall[:, 1:].max(0).tolist(), 1), orc.kernel_map(wall, (3, 3, 3)), csr=True)


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


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_voxelize_matches_oracle(dtype):
    rng = np.random.default_rng(51)
    pts = rng.uniform(-20.0, 35.0, size=(200000, 3)).astype(np.float32 if dtype == torch.float32 else np.float64)
    pts[0:199995:5] = pts[2:199997:5]              # exact duplicates
    pd = torch.as_tensor(pts, device=DEV)
    for voxel in [(0.1, 0.1, 0.1), (0.5, 0.25, 2.0)]:
        coords, index, inverse, (cmin, cmax) = backend.voxelize(pd, voxel, batch_index=3, return_index=True, return_inverse=True)
        oc, oi, ov = orc.sparse_quantize(pts, voxel)
        c = coords.cpu().numpy()
        assert (c[:, 0] == 3).all() and np.array_equal(c[:, 1:], oc)
        assert np.array_equal(index.cpu().numpy(), oi) and np.array_equal(inverse.cpu().numpy(), ov)
        assert cmin == oc.min(0).tolist() and cmax == oc.max(0).tolist()
    # the reference's interface on a device tensor
    from pcengine_amd import utils
    c3, idx = utils.sparse_quantize(pd, 0.2, return_index=True)
    oc, oi, _ = orc.sparse_quantize(pts, (0.2, 0.2, 0.2))
    assert c3.dtype == torch.int32 and np.array_equal(c3.cpu().numpy(), oc) and np.array_equal(idx.cpu().numpy(), oi)


def test_voxelize_edge_cases():
    one = torch.tensor([[0.3, -0.2, 7.9]], device=DEV)
    coords, index, inverse, _ = backend.voxelize(one, 1.0, return_index=True, return_inverse=True)
    assert coords.cpu().tolist() == [[0, 0, -1, 7]] and index.cpu().tolist() == [0] and inverse.cpu().tolist() == [0]
    same = torch.zeros((1000, 3), device=DEV)
    coords, index, _ = backend.voxelize(same, 0.5, return_index=True)
    assert coords.cpu().tolist() == [[0, 0, 0, 0]] and index.cpu().tolist() == [0]
    with pytest.raises(_lib.PCEError):
        backend.voxelize(torch.tensor([[0.0, float("nan"), 0.0]], device=DEV), 1.0)
    with pytest.raises(_lib.PCEError):
        backend.voxelize(torch.tensor([[1e12, 0.0, 0.0]], device=DEV), 1.0)
    with pytest.raises(ValueError):
        backend.voxelize(torch.zeros((4, 3), device=DEV), -1.0)
    with pytest.raises(OverflowError):       # 1e9 cells along every axis exceed the 64-bit sort key
        backend.voxelize(torch.tensor([[0.0, 0.0, 0.0], [1.0e9, 1.0e9, 1.0e9]], dtype=torch.float64, device=DEV), 1.0)
    far = torch.tensor([[0.0, 0.0, 0.0], [1.0e9, 1000.0, 1000.0], [0.0, 0.0, 0.0]], dtype=torch.float64, device=DEV)
    coords, inverse, _ = backend.voxelize(far, 1.0, return_inverse=True)     # a huge but representable box
    assert coords.cpu().tolist() == [[0, 0, 0, 0], [0, 1000000000, 1000, 1000]] and inverse.cpu().tolist() == [0, 1, 0]


@pytest.mark.parametrize("shift", [31950, -31950])
def test_submanifold_map_at_the_edge_of_the_coordinate_range(shift):
    """Keys pack 16 bits per coordinate and 16 bits of batch index: clouds pushed against |c| < 32000 in both
    directions, with batch indices up to 32767, build the same maps as the oracle."""
    base = synth.random_cloud(seed=33, n=3000, extent=40, batches=3)
    coords = base.copy()
    coords[:, 1:] = coords[:, 1:] + (shift if shift > 0 else shift - 40)
    coords[:, 0] = np.array([0, 9, 32767], np.int32)[base[:, 0]]
    order = np.lexsort((coords[:, 3], coords[:, 2], coords[:, 1], coords[:, 0]))
    coords = np.ascontiguousarray(coords[order])
    assert np.abs(coords[:, 1:]).max() < 32000
    for ks in ((3, 3, 3), (5, 5, 5), (1, 3, 3)):
        assert_map_equal(gpu_map(coords, ks, want_csr=True), orc.kernel_map(coords, ks), csr=True)
