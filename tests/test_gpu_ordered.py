"""The ordered output-stationary dataflow: the row order (masks, sections, permutation) against the oracle's map,
and the layer against the float64 oracle through the C ABI.  Bar: rel-L2 <= 1e-3 (fp16 storage, fp32 accumulate)."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from pcengine_amd import _lib, backend, synth
from pcengine_amd.backend import DATAFLOW_FDS, DATAFLOW_OS, DATAFLOW_OSO
from tests.util import DEV, dev_coords, rounded

pytestmark = pytest.mark.gpu
K3, S1, P0 = (3, 3, 3), (1, 1, 1), (0, 0, 0)

CLOUDS = {
    "lidar": lambda: synth.lidar_cloud_100k()[::3].copy(),                  # rows mostly without neighbours
    "surface": lambda: synth.sphere_plane_cloud(),                          # 4.7 pairs per row: mostly heavy rows
    "dense": lambda: synth.random_cloud(seed=91, n=9000, extent=22, batches=2),
    "tiny": lambda: synth.random_cloud(seed=92, n=45, extent=5),
}


def _subm(coords, **kw):
    batches = int(coords[:, 0].max()) + 1
    return backend.build_kernel_map(dev_coords(coords), K3, S1, P0, [0, 0, 0], coords[:, 1:].max(0).tolist(), True, want_csr=True,
                                    batchsize=batches, **kw)


def _oracle_masks(coords):
    ref = orc.kernel_map(coords, K3)
    masks = np.zeros(len(coords), np.int64)
    for kp in range(27):
        if kp != 13:
            masks[ref.omap[ref.kpos[kp]:ref.kpos[kp + 1]]] |= 1 << kp
    return ref, masks


def _popcount(m):
    return np.array([bin(int(v)).count("1") for v in m])


def _key(m):
    """Sort key of a row with neighbours: rows with one neighbour by its offset, then rows with two by (lowest,
    second-lowest) offset, then rows with three or more likewise."""
    bits = [k for k in range(27) if (int(m) >> k) & 1]
    if len(bits) == 1:
        return bits[0]
    return (1024 if len(bits) >= 3 else 0) + 32 + bits[0] * 32 + bits[1]


@pytest.mark.parametrize("cloud", sorted(CLOUDS))
def test_row_order_built_with_the_map_and_on_its_own(cloud):
    """perm is a permutation; rows without neighbours come first, in ascending order within each block of 256; then the
    rows with one or two neighbours in ascending key order, then the rows with three or more likewise; the masks are
    the oracle's neighbour patterns and the count of heavy rows is theirs.  The order requested on its own
    (pce_row_order) has the same masks, sections and keys."""
    coords = CLOUDS[cloud]()
    ref, masks = _oracle_masks(coords)
    km = _subm(coords)
    n = len(coords)
    rec_at = (2 * n + 8192 + 3) // 4 * 4
    srec_at, srec_rows = rec_at + 4 * n, n // 8 + 32
    assert km.order is not None and km.order.numel() == srec_at + 32 * srec_rows == _lib.load().pce_row_order_elems(n)
    lazy = _subm(coords, want_order=False)
    assert lazy.order is None
    backend.row_order(lazy)
    pc = _popcount(masks)
    for m in (km, lazy):
        order = m.order.cpu().numpy()
        perm, got_masks = order[:n].astype(np.int64), order[n:2 * n].view(np.uint32).astype(np.int64)
        assert np.array_equal(got_masks, masks)
        assert np.array_equal(np.sort(perm), np.arange(n))
        assert m.order_heavy == int((pc >= 3).sum())
        assert m.order_nonzero == int((pc >= 1).sum()) and m.order_single == int((pc == 1).sum())
        n_plain, n_heavy = int((pc == 0).sum()), int((pc >= 3).sum())
        sect = masks[perm]
        assert (sect[:n_plain] == 0).all() and (sect[n_plain:] != 0).all()
        assert (_popcount(sect[n_plain:n - n_heavy]) <= 2).all() and (_popcount(sect[n - n_heavy:]) >= 3).all()
        keys = np.array([_key(v) for v in sect[n_plain:]])
        assert (np.diff(keys) >= 0).all()
        plain = perm[:n_plain]
        same_block = plain[1:] // 256 == plain[:-1] // 256
        assert (np.diff(plain)[same_block] > 0).all()        # a block's plain rows keep their order
        # the record of every row with a neighbour, at its position in the order: the row, its mask and its
        # neighbours at the two lowest offsets of the mask (the oracle's pairs)
        rec = order[rec_at:rec_at + 4 * n].reshape(n, 4).astype(np.int64)[n_plain:]
        rows = perm[n_plain:]
        assert np.array_equal(rec[:, 0], rows) and np.array_equal(rec[:, 1], masks[rows])
        nbr_of = {}
        for kp in range(27):
            if kp != 13:
                a, b = ref.kpos[kp], ref.kpos[kp + 1]
                nbr_of.update({(int(o), kp): int(i) for i, o in zip(ref.imap[a:b], ref.omap[a:b])})
        for (row, mask, nb0, nb1) in rec[:: max(1, len(rec) // 500)]:
            bits = [k for k in range(27) if (mask >> k) & 1]
            assert nb0 == nbr_of[(row, bits[0])]
            assert nb1 == (nbr_of[(row, bits[1])] if len(bits) > 1 else -1)
        # the 128-byte records of the rows with two neighbours or more, in the order's sequence: row, mask and the
        # neighbour at every offset (-1 where there is none); written where those rows are at most an eighth
        n_single = int((pc == 1).sum())
        shared = perm[n_plain + n_single:]
        if len(shared) <= srec_rows:
            srec = order[srec_at:srec_at + 32 * len(shared)].reshape(len(shared), 32).astype(np.int64)
            assert np.array_equal(srec[:, 0], shared) and np.array_equal(srec[:, 1], masks[shared])
            want = np.full((len(shared), 30), -1, np.int64)
            for i, row in enumerate(shared):
                for k in range(27):
                    if (masks[row] >> k) & 1:
                        want[i, k] = nbr_of[(int(row), k)]
            assert np.array_equal(srec[:, 2:], want)


@pytest.mark.parametrize("cloud", sorted(CLOUDS))
def test_map_built_without_pair_lists(cloud):
    """want_pairs=False: the 3x3x3 submanifold map over the column grid comes as neighbour table, row order and
    counts only (has_pairs False), all equal to the full build's; the ordered dataflow runs on it as it is; reading
    a pair list builds both, bit-equal to the oracle's; a build that cannot skip them (no batch count: the hash
    table) ignores the request."""
    coords = CLOUDS[cloud]()
    ref, masks = _oracle_masks(coords)
    full = _subm(coords)
    batches = int(coords[:, 0].max()) + 1
    build = lambda b: backend.build_kernel_map(dev_coords(coords), K3, S1, P0, [0, 0, 0], coords[:, 1:].max(0).tolist(), True,
                                               want_csr=False, batchsize=b, want_pairs=False)
    km = build(batches)
    assert not km.has_pairs and km.M == ref.M and km.qsum == full.qsum
    for name in ("nbr_out", "knnz", "kpos", "qkpos"):
        assert torch.equal(getattr(km, name), getattr(full, name)), name
    n = len(coords)
    assert km.order_heavy == full.order_heavy and torch.equal(km.order[n:2 * n], full.order[n:2 * n])
    assert backend.select_dataflow(km, 32, 32, torch.float16) == backend.select_dataflow(full, 32, 32, torch.float16)
    f = torch.as_tensor(synth.features(3, n, 32), device=DEV).half()
    w = torch.as_tensor(synth.weights(3, 27, 32, 32), device=DEV).half()
    assert torch.equal(backend.conv_forward(f, w, km, DATAFLOW_OSO), backend.conv_forward(f, w, full, DATAFLOW_OSO))
    assert not km.has_pairs
    assert np.array_equal(km.imap.cpu().numpy(), ref.imap) and np.array_equal(km.omap.cpu().numpy(), ref.omap)
    assert km.has_pairs
    assert build(0).has_pairs


@pytest.mark.parametrize("cloud", sorted(CLOUDS))
@pytest.mark.parametrize("c_in,c_out", [(64, 64), (32, 32), (16, 32), (48, 24), (64, 8), (16, 64),
                                        (64, 96), (96, 96), (64, 128), (96, 128), (128, 96), (96, 72),
                                        (80, 96), (112, 80), (80, 128)])   # from 64 -> 96 on: the K-stepped kernel
def test_ordered_dataflow_against_the_oracle(cloud, c_in, c_out):
    coords = CLOUDS[cloud]()
    ref, _ = _oracle_masks(coords)
    km = _subm(coords)
    n = len(coords)
    dt = torch.float16
    f, w = synth.features(c_in, n, c_in), synth.weights(c_out, 27, c_in, c_out)
    bias = np.random.default_rng(c_in).standard_normal(c_out) * 0.1
    res = synth.features(c_out + 1, n, c_out)
    fd, wd = torch.as_tensor(f, device=DEV).to(dt), torch.as_tensor(w, device=DEV).to(dt)
    bd, rd = torch.as_tensor(bias, device=DEV).to(dt), torch.as_tensor(res, device=DEV).to(dt)
    packed = backend.pack_weights(wd)
    plain = orc.conv_forward(rounded(f, dt), rounded(w, dt), ref, K3)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed)
    assert orc.rel_l2(out.double().cpu().numpy(), plain) <= 1e-3
    assert orc.rel_l2(backend.conv_forward(fd, wd, km, DATAFLOW_OSO).double().cpu().numpy(), plain) <= 1e-3    # packs on the fly
    want = np.maximum(plain + rounded(bias, dt) + rounded(res, dt), 0)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed, bias=bd, residual=rd, act="relu")
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3
    leaky = plain + rounded(bias, dt)
    leaky = np.where(leaky > 0, leaky, 0.1 * leaky)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed, bias=bd, act=("leaky_relu", 0.1))
    assert orc.rel_l2(out.double().cpu().numpy(), leaky) <= 1e-3
    # every row is computed by one wavefront (or one workgroup) alone: two runs agree bit for bit, whatever the
    # positions the rows of equal keys took in the order
    again = backend.conv_forward(fd, wd, _subm(coords), DATAFLOW_OSO, packed=packed, bias=bd, act=("leaky_relu", 0.1))
    assert torch.equal(out, again)


@pytest.mark.parametrize("cloud", sorted(CLOUDS))
@pytest.mark.parametrize("c_in,c_out", [(16, 16), (8, 32), (32, 8), (24, 24), (32, 32)])
def test_ordered_dataflow_fp32_against_the_oracle(cloud, c_in, c_out):
    """The fp32 form (at most 32 channels either side): 1e-5 against the float64 oracle, with and without the epilogue."""
    coords = CLOUDS[cloud]()
    ref, _ = _oracle_masks(coords)
    km = _subm(coords)
    n = len(coords)
    f, w = synth.features(c_in, n, c_in), synth.weights(c_out, 27, c_in, c_out)
    bias = (np.random.default_rng(c_in).standard_normal(c_out) * 0.1).astype(np.float32)
    res = synth.features(c_out + 1, n, c_out)
    fd, wd = torch.as_tensor(f, device=DEV).float(), torch.as_tensor(w, device=DEV).float()
    bd, rd = torch.as_tensor(bias, device=DEV).float(), torch.as_tensor(res, device=DEV).float()
    plain = orc.conv_forward(f.astype(np.float32), w.astype(np.float32), ref, K3)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO)
    assert orc.rel_l2(out.double().cpu().numpy(), plain) <= 1e-5
    want = np.maximum(plain + bias + res.astype(np.float32), 0)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, bias=bd, residual=rd, act="relu")
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-5
    leaky = plain + bias
    leaky = np.where(leaky > 0, leaky, 0.1 * leaky)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, bias=bd, act=("leaky_relu", 0.1))
    assert orc.rel_l2(out.double().cpu().numpy(), leaky) <= 1e-5
    again = backend.conv_forward(fd, wd, _subm(coords), DATAFLOW_OSO, bias=bd, act=("leaky_relu", 0.1))
    assert torch.equal(out, again)
    # column slices in and out, as the skip connections use them
    # (row strides of whole 32-byte groups, so that both views are read and written in place: no dense copy is made)
    wide_in = torch.full((n, c_in + 16), 7.0, dtype=torch.float32, device=DEV)
    wide_in[:, 8:8 + c_in] = fd
    wide_out = torch.full((n, c_out + 16), -3.0, dtype=torch.float32, device=DEV)
    assert backend._row_stride(wide_in[:, 8:8 + c_in]) == c_in + 16 and backend._row_stride(wide_out[:, 8:8 + c_out]) == c_out + 16
    got = backend.conv_forward(wide_in[:, 8:8 + c_in], wd, km, DATAFLOW_OSO, out=wide_out[:, 8:8 + c_out], bias=bd, act=("leaky_relu", 0.1))
    assert torch.equal(got, out) and bool((wide_out[:, :8] == -3.0).all()) and bool((wide_out[:, 8 + c_out:] == -3.0).all())


STRIDED = [((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((2, 3, 1), (2, 1, 1), (0, 1, 0))]
_strided_refs = {}


def _strided_ref(cloud, geom):
    """(coordinates, oracle map, offset mask of every output row) of a strided layer on a cloud, computed once."""
    if (cloud, geom) not in _strided_refs:
        coords = CLOUDS[cloud]()
        ks, stride, pad = STRIDED[geom]
        ref = orc.kernel_map(coords, ks, stride, pad)
        masks = np.zeros(len(ref.out_coords), np.int64)
        for kp in range(orc.kernel_volume(ks)):
            masks[ref.omap[ref.kpos[kp]:ref.kpos[kp + 1]]] |= 1 << kp
        _strided_refs[(cloud, geom)] = (coords, ref, masks)
    return _strided_refs[(cloud, geom)]


def _strided_map(coords, geom, **kw):
    ks, stride, pad = STRIDED[geom]
    cmax_out = orc.strided_coords_max(coords[:, 1:].max(0).tolist(), ks, stride, pad)
    return backend.build_kernel_map(dev_coords(coords), ks, stride, pad, [0, 0, 0], cmax_out, False, want_csr=True,
                                    batchsize=int(coords[:, 0].max()) + 1, **kw)


@pytest.mark.parametrize("cloud", sorted(CLOUDS))
@pytest.mark.parametrize("geom", range(len(STRIDED)))
def test_row_order_of_strided_maps(cloud, geom):
    """A strided layer has no centre offset: every output row has a pair, the masks cover all offsets, the sections
    are (one or two pairs, sorted by key) and (three or more, likewise).  Maps of at most 8 offsets come with their
    order; others get it on first use."""
    coords, ref, masks = _strided_ref(cloud, geom)
    km = _strided_map(coords, geom)
    n = km.n_out
    assert n == len(ref.out_coords) and (masks != 0).all()
    assert (km.order is not None) == (km.kv <= 8)
    backend.row_order(km)
    order = km.order.cpu().numpy()
    perm, got_masks = order[:n].astype(np.int64), order[n:2 * n].view(np.uint32).astype(np.int64)
    assert np.array_equal(got_masks, masks)
    assert np.array_equal(np.sort(perm), np.arange(n))
    pc = _popcount(masks)
    n_heavy = int((pc >= 3).sum())
    assert km.order_heavy == n_heavy
    sect = masks[perm]
    assert (_popcount(sect[:n - n_heavy]) <= 2).all() and (_popcount(sect[n - n_heavy:]) >= 3).all()
    assert (np.diff(np.array([_key(v) for v in sect])) >= 0).all()


@pytest.mark.parametrize("cloud", sorted(CLOUDS))
@pytest.mark.parametrize("geom", range(len(STRIDED)))
@pytest.mark.parametrize("c_in,c_out", [(32, 32), (64, 64), (16, 64), (48, 24), (64, 96), (128, 80), (80, 104)])
def test_ordered_dataflow_strided_against_the_oracle(cloud, geom, c_in, c_out):
    """The ordered rows without a centre term (strided layers, fp16): the float64 oracle within 1e-3, epilogue fused,
    bit-equal from run to run, column slices on both sides."""
    coords, ref, _ = _strided_ref(cloud, geom)
    ks = STRIDED[geom][0]
    kv = orc.kernel_volume(ks)
    km = _strided_map(coords, geom)
    n_in, n_out = len(coords), km.n_out
    dt = torch.float16
    f, w = synth.features(c_in + geom, n_in, c_in), synth.weights(c_out, kv, c_in, c_out)
    bias = np.random.default_rng(c_in).standard_normal(c_out) * 0.1
    res = synth.features(c_out + 1, n_out, c_out)
    fd, wd = torch.as_tensor(f, device=DEV).to(dt), torch.as_tensor(w, device=DEV).to(dt)
    bd, rd = torch.as_tensor(bias, device=DEV).to(dt), torch.as_tensor(res, device=DEV).to(dt)
    packed = backend.pack_weights(wd)
    assert backend.oso_takes(km, c_in, c_out, dt) and not backend.oso_takes(km, c_in, c_out, dt, transposed=True)
    plain = orc.conv_forward(rounded(f, dt), rounded(w, dt), ref, ks)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed)
    assert out.shape == (n_out, c_out)
    assert orc.rel_l2(out.double().cpu().numpy(), plain) <= 1e-3
    want = np.maximum(plain + rounded(bias, dt) + rounded(res, dt), 0)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed, bias=bd, residual=rd, act="relu")
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3
    again = backend.conv_forward(fd, wd, _strided_map(coords, geom), DATAFLOW_OSO, packed=packed, bias=bd, residual=rd, act="relu")
    assert torch.equal(out, again)
    wide_in = torch.full((n_in, c_in + 24), 5.0, dtype=dt, device=DEV)
    wide_in[:, 8:8 + c_in] = fd
    wide_out = torch.full((n_out, c_out + 16), -2.0, dtype=dt, device=DEV)
    got = backend.conv_forward(wide_in[:, 8:8 + c_in], wd, km, DATAFLOW_OSO, packed=packed, out=wide_out[:, 8:8 + c_out], bias=bd,
                               residual=rd, act="relu")
    assert torch.equal(got, out) and bool((wide_out[:, :8] == -2.0).all()) and bool((wide_out[:, 8 + c_out:] == -2.0).all())
    # the transposed layer has no ordered form: a request for it falls back to deferred scatter in the front end,
    # and the backend refuses it
    with pytest.raises(ValueError):
        backend.conv_forward(out, torch.zeros((kv, c_out, c_in), dtype=dt, device=DEV), km, DATAFLOW_OSO, transposed=True)


def test_selector_gives_narrow_stride_2_layers_to_the_ordered_rows():
    coords = CLOUDS["lidar"]()
    km = _strided_map(coords, 0)
    assert km.M / km.n_out <= 2.0
    assert backend.select_dataflow(km, 32, 32, torch.float16) == DATAFLOW_OSO
    assert backend.select_dataflow(km, 64, 64, torch.float16) == DATAFLOW_OSO
    assert backend.select_dataflow(km, 64, 128, torch.float16) == DATAFLOW_OSO       # the K-stepped kernel's shapes too
    assert backend.select_dataflow(km, 128, 128, torch.float16) != DATAFLOW_OSO
    assert backend.select_dataflow(km, 32, 32, torch.float32) != DATAFLOW_OSO
    assert backend.select_dataflow(km, 32, 32, torch.float16, transposed=True) != DATAFLOW_OSO
    dense = _strided_map(CLOUDS["dense"](), 0)          # a filled box: close to eight pairs per output row
    assert dense.M / dense.n_out > 2.0 and backend.select_dataflow(dense, 32, 32, torch.float16) == DATAFLOW_OS


def test_ordered_dataflow_on_column_slices_and_the_selector():
    coords = CLOUDS["lidar"]()
    km = _subm(coords)
    n, c = len(coords), 32
    wide_in = torch.full((n, c + 24), 5.0, dtype=torch.float16, device=DEV)
    f = torch.as_tensor(synth.features(1, n, c), device=DEV).half()
    wide_in[:, 8:8 + c] = f
    wide_out = torch.full((n, 2 * c + 16), -2.0, dtype=torch.float16, device=DEV)
    w = torch.as_tensor(synth.weights(1, 27, c, c), device=DEV).half()
    packed = backend.pack_weights(w)
    want = backend.conv_forward(f, w, km, DATAFLOW_OSO, packed=packed)
    got = backend.conv_forward(wide_in[:, 8:8 + c], w, km, DATAFLOW_OSO, packed=packed, out=wide_out[:, c:2 * c])
    assert torch.equal(got, want) and bool((wide_out[:, :c] == -2.0).all()) and bool((wide_out[:, 2 * c:] == -2.0).all())
    assert backend.select_dataflow(km, c, c, torch.float16) == DATAFLOW_OSO
    assert backend.select_dataflow(km, 16, 16, torch.float32) == DATAFLOW_OSO      # the fp32 form: up to 32 channels, by density
    assert backend.select_dataflow(km, 64, 64, torch.float32) != DATAFLOW_OSO
    assert backend.select_dataflow(km, 128, 128, torch.float16) != DATAFLOW_OSO
    assert backend.oso_takes(km, 96, 96, torch.float16) and backend.oso_takes(km, 128, 96, torch.float16)
    assert backend.oso_takes(km, 80, 96, torch.float16) and backend.oso_takes(km, 112, 72, torch.float16) and backend.oso_takes(km, 80, 128, torch.float16)
    assert not backend.oso_takes(km, 128, 128, torch.float16) and not backend.oso_takes(km, 192, 128, torch.float16)
    assert not backend.oso_takes(km, 112, 128, torch.float16)
    # the two pair-proportional dataflows agree to fp16 rounding (they round partial sums at different places)
    fds = backend.conv_forward(f, w, km, DATAFLOW_FDS, packed=packed)
    assert float((fds.float() - want.float()).norm() / want.float().norm()) <= 1e-3


SPARSE_CLOUDS = {
    "lidar": CLOUDS["lidar"],
    "scan": lambda: synth.lidar_cloud()[:40000].copy(),       # the benchmark's cloud: a few heavy rows, mostly none
    "thin": lambda: synth.random_cloud(seed=93, n=5000, extent=60, batches=2),   # 5 000 voxels in 2 x 60^3: nearly all alone
}


@pytest.mark.parametrize("cloud", sorted(SPARSE_CLOUDS))
@pytest.mark.parametrize("c_in,c_out", [(64, 64), (32, 32), (16, 64), (48, 24), (64, 8), (48, 64)])
def test_streamed_form_against_the_ordered_form(cloud, c_in, c_out):
    """Clouds where at most half the rows have a neighbour run as three kinds of workgroup (rows without neighbours
    streamed in storage order, rows with one by their records, the rest shared by four wavefronts): against the
    oracle, and against the kernel that visits every row through the order (what the same call runs when the count
    of rows with neighbours is not stated) -- bit-identical on rows with at most one neighbour, to rounding on the
    others --, with and without the epilogue."""
    coords = SPARSE_CLOUDS[cloud]()
    ref, masks = _oracle_masks(coords)
    km = _subm(coords)
    n = len(coords)
    assert km.order_nonzero == int((masks != 0).sum()) and 2 * km.order_nonzero <= n
    many = torch.as_tensor(_popcount(masks) >= 2, device=DEV)
    dt = torch.float16
    f, w = synth.features(c_in + 1, n, c_in), synth.weights(c_out + 2, 27, c_in, c_out)
    fd, wd = torch.as_tensor(f, device=DEV).to(dt), torch.as_tensor(w, device=DEV).to(dt)
    bd = torch.as_tensor(np.random.default_rng(5).standard_normal(c_out) * 0.1, device=DEV).to(dt)
    rd = torch.as_tensor(synth.features(c_out + 3, n, c_out), device=DEV).to(dt)
    packed = backend.pack_weights(wd)
    want = orc.conv_forward(rounded(f, dt), rounded(w, dt), ref, K3)
    for kw in ({}, dict(bias=bd, residual=rd, act="relu")):
        new = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed, **kw)
        nonzero, km.order_nonzero = km.order_nonzero, -1
        old = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed, **kw)
        km.order_nonzero = nonzero
        # rows with two neighbours or more are summed channel quarter by channel quarter here, offset by offset there
        assert torch.equal(new[~many], old[~many])
        assert torch.allclose(new[many].float(), old[many].float(), rtol=4e-3, atol=2e-3)
        if not kw:
            assert orc.rel_l2(new.double().cpu().numpy(), want) <= 1e-3
    # rows in a wider matrix, in and out
    wide_in = torch.full((n, c_in + 16), 7.0, dtype=dt, device=DEV)
    wide_in[:, 8:8 + c_in] = fd
    wide_out = torch.full((n, c_out + 24), -3.0, dtype=dt, device=DEV)
    got = backend.conv_forward(wide_in[:, 8:8 + c_in], wd, km, DATAFLOW_OSO, packed=packed, out=wide_out[:, 16:16 + c_out])
    assert torch.equal(got, backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=packed))
    assert bool((wide_out[:, :16] == -3.0).all()) and bool((wide_out[:, 16 + c_out:] == -3.0).all())


def test_ordered_dataflow_argument_errors():
    lib = _lib.load()
    coords = CLOUDS["tiny"]()
    km = _subm(coords)
    n = len(coords)
    s = torch.cuda.current_stream().cuda_stream
    f = torch.zeros((n, 32), dtype=torch.float16, device=DEV)
    w = torch.zeros((27, 32, 32), dtype=torch.float16, device=DEV)
    pk = backend.pack_weights(w)
    out = torch.zeros((n, 32), dtype=torch.float16, device=DEV)
    call = lambda dtype, c_in, c_out, mid, heavy, packed=pk, nonzero=-1, single=-1: lib.pce_conv_fwd_oso(
        f.data_ptr(), w.data_ptr(), packed.data_ptr() if packed is not None else None, out.data_ptr(), dtype, n, n, c_in, c_out, 27, mid,
        km.nbr_out.data_ptr(), km.order.data_ptr(), (_lib.c_int64 * 3)(heavy, nonzero, single), None, s)
    assert call(_lib.PCE_F16, 32, 32, 13, km.order_heavy) == _lib.PCE_OK
    assert call(_lib.PCE_F16, 32, 32, 13, km.order_heavy, nonzero=km.order_nonzero, single=km.order_single) == _lib.PCE_OK
    assert call(_lib.PCE_F16, 32, 32, 13, km.order_heavy, nonzero=km.order_heavy - 1) == _lib.PCE_EINVAL   # fewer than the heavy rows
    assert call(_lib.PCE_F16, 32, 32, 13, km.order_heavy, nonzero=n + 1) == _lib.PCE_EINVAL
    assert call(_lib.PCE_F16, 32, 32, 13, km.order_heavy, nonzero=km.order_nonzero, single=km.order_nonzero + 1) == _lib.PCE_EINVAL
    assert call(_lib.PCE_F32, 64, 32, 13, km.order_heavy) == _lib.PCE_EINVAL        # fp32 stops at 32 channels
    assert call(_lib.PCE_F32, 12, 32, 13, km.order_heavy) == _lib.PCE_EINVAL        # ... in multiples of 8
    assert call(_lib.PCE_F32, 32, 32, -1, km.order_heavy) == _lib.PCE_EINVAL        # fp32 needs a centre offset
    assert call(_lib.PCE_F16, 32, 32, 13, n + 1) == _lib.PCE_EINVAL
    assert call(_lib.PCE_F16, 32, 32, 13, km.order_heavy, None) == _lib.PCE_EINVAL    # weights not packed
    assert call(_lib.PCE_F16, 128, 32, 13, km.order_heavy) == _lib.PCE_EINVAL
    assert call(_lib.PCE_F16, 128, 128, 13, km.order_heavy) == _lib.PCE_EINVAL       # beyond the K-stepped kernel's shapes
    heavy = (_lib.c_int64 * 3)()
    order = torch.zeros(lib.pce_row_order_elems(n), dtype=torch.int32, device=DEV)
    assert lib.pce_row_order(km.nbr_out.data_ptr(), 27, n, 13, order.data_ptr(), order.numel() - 1, heavy, s) == _lib.PCE_EWORKSPACE
    assert lib.pce_row_order(km.nbr_out.data_ptr(), 125, n, 62, order.data_ptr(), order.numel(), heavy, s) == _lib.PCE_EINVAL
    with pytest.raises(ValueError):
        backend.conv_forward(torch.zeros((n, 192), dtype=torch.float16, device=DEV), torch.zeros((27, 192, 128), dtype=torch.float16, device=DEV),
                             km, DATAFLOW_OSO)


def _molecules(singles, dimers, trimers, blob, seed=0):
    """A cloud with chosen numbers of rows per neighbour count: isolated voxels, pairs of adjacent voxels (one
    neighbour each), lines of three (the middle voxel has two neighbours), and one filled blob of blob^3 voxels
    (three neighbours or more).  Groups sit on a lattice of pitch 4 so that they do not touch."""
    rng = np.random.default_rng(seed)
    groups = [np.zeros((1, 3), int)] * singles + [np.array([[0, 0, 0], [0, 0, 1]])] * dimers + \
             [np.array([[0, 0, 0], [0, 1, 0], [0, 2, 0]])] * trimers
    side = int(np.ceil(len(groups) ** (1 / 3))) + 1
    cells = rng.permutation(side ** 3)[:len(groups)]
    pts = [g + 4 * np.array([c // (side * side), (c // side) % side, c % side]) for g, c in zip(groups, cells)]
    if blob:
        b = np.stack(np.meshgrid(*[np.arange(blob)] * 3, indexing="ij"), -1).reshape(-1, 3) + 4 * side + 4
        pts.append(b)
    xyz = np.concatenate(pts, 0)
    c = np.concatenate([np.zeros((len(xyz), 1), int), xyz], 1)
    return np.unique(c, axis=0).astype(np.int32)


@pytest.mark.parametrize("mix", [(3000, 0, 0, 0), (3000, 400, 0, 0), (3000, 0, 300, 0), (5000, 300, 100, 0), (4000, 200, 100, 6),
                                 (2000, 0, 0, 5), (3001, 37, 1, 0)])
@pytest.mark.parametrize("c_in,c_out", [(64, 64), (48, 32)])
def test_three_kind_form_on_clouds_with_chosen_neighbour_counts(mix, c_in, c_out):
    """The three kinds of workgroup one at a time and together: clouds made of isolated voxels, pairs, lines of three
    and a filled blob, so that the sections of the order (no neighbour / one / two / three or more) are empty, tiny or
    ragged at will; the counts against their construction, the layer against the oracle."""
    singles, dimers, trimers, blob = mix
    coords = _molecules(*mix, seed=sum(mix))
    n = len(coords)
    assert n == singles + 2 * dimers + 3 * trimers + blob ** 3
    ref, masks = _oracle_masks(coords)
    pc = _popcount(masks)
    km = _subm(coords)
    assert km.order_single == 2 * dimers + 2 * trimers == int((pc == 1).sum())
    assert km.order_nonzero - km.order_single - km.order_heavy == trimers == int((pc == 2).sum())
    assert km.order_heavy == blob ** 3 == int((pc >= 3).sum())
    assert 2 * km.order_nonzero <= n and 8 * (km.order_nonzero - km.order_single) <= n        # the three-kind form takes it
    dt = torch.float16
    f, w = synth.features(c_in, n, c_in), synth.weights(c_out, 27, c_in, c_out)
    fd, wd = torch.as_tensor(f, device=DEV).to(dt), torch.as_tensor(w, device=DEV).to(dt)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_OSO, packed=backend.pack_weights(wd))
    want = orc.conv_forward(rounded(f, dt), rounded(w, dt), ref, K3)
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3
    # row by row: no row of any section is left unwritten or written by the wrong kind
    err = np.abs(out.double().cpu().numpy() - want).max(1)
    assert err.max() <= 2e-2, (int(err.argmax()), int(pc[err.argmax()]))
