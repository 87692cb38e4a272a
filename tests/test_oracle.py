"""Pins the CPU oracle: brute force, the literal C restatement of the reference kernels,
dense torch convolutions and closed forms.  No GPU, no reference import."""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import load_literal, oracle as orc
from pcengine_amd import synth

I32P = ctypes.POINTER(ctypes.c_int)


def _p(a):
    return a.ctypes.data_as(I32P)


def _i3(v):
    return (ctypes.c_int * 3)(*[int(x) for x in v])


GEOMS = [
    # ks, stride, pad
    ((3, 3, 3), (1, 1, 1), (0, 0, 0)),
    ((2, 2, 2), (2, 2, 2), (0, 0, 0)),
    ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
    ((3, 3, 3), (2, 2, 2), (0, 0, 0)),
    ((3, 1, 3), (1, 1, 1), (0, 0, 0)),
    ((2, 3, 1), (2, 1, 1), (0, 1, 0)),
    ((5, 5, 5), (1, 1, 1), (0, 0, 0)),
    ((1, 1, 1), (2, 2, 2), (0, 0, 0)),
    ((2, 2, 2), (1, 1, 1), (0, 0, 0)),   # stride 1, even kernel sizes: offsets are not mirror images (hash.cuh:147-149)
    ((2, 3, 3), (1, 1, 1), (0, 0, 0)),
]


def test_codes_roundtrip():
    # script/utils.py:233-242; default tensor stride 94585 == (1,1,1) (script/sptensor.py:13)
    assert orc.encode3([1, 1, 1]) == 94585
    for v in [(1, 1, 1), (2, 2, 2), (3, 1, 5), (16, 16, 16), (310, 302, 310)]:
        assert orc.decode3(orc.encode3(v)) == v
    assert orc.output_stride(orc.encode3([2, 2, 2]), orc.encode3([4, 4, 4])) == orc.encode3([8, 8, 8])
    assert orc.output_stride(orc.encode3([2, 2, 2]), orc.encode3([4, 4, 4]), True) == orc.encode3([2, 2, 2])


def test_offsets_closed_form():
    d = orc.offsets((3, 3, 3), strided=False)
    assert d.shape == (27, 3) and (d[0] == [-1, -1, -1]).all() and (d[13] == 0).all() and (d[26] == 1).all()
    assert (d[5] == [-1, 0, 1]).all()  # kp = (ix*3+iy)*3+iz, x slowest
    ds = orc.offsets((3, 3, 3), strided=True)
    assert (ds == d + 1).all()          # backend/hash.cuh:235-237
    assert (orc.offsets((2, 2, 2), True) == orc.offsets((2, 2, 2), False)).all()
    assert (orc.offsets((2, 2, 2), True)[7] == [1, 1, 1]).all()
    assert (orc.offsets((5, 5, 5), True)[0] == [-1, -1, -1]).all()  # idx - 1 for k = 5
    assert orc.mid_offset((3, 3, 3)) == 13 and orc.mid_offset((2, 2, 2)) == 0 and orc.mid_offset((3, 1, 3)) == 4


def test_scans_closed_form():
    knnz = np.array([0, 1, 128, 129, 300, 0, 5], np.int32)
    kpos, qkpos = orc.scans(knnz)
    assert kpos.tolist() == [0, 0, 1, 129, 258, 558, 558, 563]
    assert qkpos.tolist() == [0, 0, 128, 256, 512, 896, 896, 1024]


@pytest.mark.parametrize("ks,stride,pad", GEOMS)
def test_kernel_map_vs_brute_force(ks, stride, pad):
    coords = synth.random_cloud(seed=3, n=260, extent=7, batches=2)
    km = orc.kernel_map(coords, ks, stride, pad)
    subm = tuple(stride) == (1, 1, 1)
    pairs = orc.brute_force_pairs(coords, km.out_coords, ks, stride, pad, subm)
    kp_of = np.repeat(np.arange(km.kv), km.knnz)
    got = list(zip(kp_of.tolist(), km.imap.tolist(), km.omap.tolist()))
    assert got == pairs
    assert km.M == len(pairs) and km.kpos[-1] == len(pairs)
    if subm:
        if all(k % 2 == 1 for k in ks):
            assert (km.knnz == km.knnz[::-1]).all()   # symmetry of a submanifold map with odd kernel sizes
        assert km.knnz[orc.mid_offset(ks)] == 0
    else:
        # output set by brute force: every candidate (x + p - d)/s that divides and is in range
        cmax = orc.strided_coords_max(coords[:, 1:].max(0), ks, stride, pad)
        want = set()
        d = orc.offsets(ks, True)
        for c in coords.tolist():
            for kp in range(km.kv):
                cand = [c[1 + a] - int(d[kp, a]) + pad[a] for a in range(3)]
                if all(v % stride[a] == 0 and 0 <= v // stride[a] <= cmax[a] for a, v in enumerate(cand) if v >= 0) \
                        and all(v >= 0 for v in cand):
                    want.add((c[0],) + tuple(v // stride[a] for a, v in enumerate(cand)))
        assert [tuple(r) for r in km.out_coords.tolist()] == sorted(want)


def _literal_maps(coords, ks, stride, pad):
    lib = load_literal()
    subm = tuple(stride) == (1, 1, 1)
    kv = ks[0] * ks[1] * ks[2]
    n_in = len(coords)
    coords = np.ascontiguousarray(coords, np.int32)
    if subm:
        out = coords
        n_out = n_in
    else:
        cmax = orc.strided_coords_max(coords[:, 1:].max(0), ks, stride, pad)
        buf = np.zeros((n_in * kv, 4), np.int32)
        n_out = lib.lit_out_coords(n_in, _p(coords), _i3(ks), _i3(stride), _i3(pad), _i3((0, 0, 0)), _i3(cmax), _p(buf))
        out = np.ascontiguousarray(buf[:n_out])
    dense = -np.ones(kv * n_in, np.int32)
    knnz = np.zeros(kv, np.int32)
    kpos = np.zeros(kv + 1, np.int32)
    qkpos = np.zeros(kv + 1, np.int32)
    lib.lit_map_d2(n_in, _p(coords), n_out, _p(out), _i3(ks), _i3(stride), _i3(pad), int(subm),
                   _p(dense), _p(knnz), _p(kpos), _p(qkpos))
    nz = np.nonzero(dense != -1)[0]          # script/spconv.py:370-372
    omap = dense[nz]
    imap = (nz % n_in).astype(np.int32)
    imc = -np.ones(n_in * kv, np.int32)
    omc = -np.ones(n_out * kv, np.int32)
    icsr = np.zeros(n_in + 1, np.int32)
    ocsr = np.zeros(n_out + 1, np.int32)
    lib.lit_map_d1(n_in, n_out, kv, _p(dense), _p(imc), _p(omc), _p(icsr), _p(ocsr))
    M = int(kpos[-1])
    return out, imap, omap, knnz, kpos, qkpos, icsr, imc[:M], ocsr, omc[:M]


@pytest.mark.parametrize("ks,stride,pad", GEOMS)
@pytest.mark.parametrize("seed,n,extent", [(11, 500, 9), (12, 3000, 24)])
def test_oracle_vs_literal_reference_kernels(ks, stride, pad, seed, n, extent):
    coords = synth.random_cloud(seed=seed, n=n, extent=extent, batches=3)
    km = orc.kernel_map(coords, ks, stride, pad)
    out, imap, omap, knnz, kpos, qkpos, icsr, imc, ocsr, omc = _literal_maps(coords, ks, stride, pad)
    assert np.array_equal(out, km.out_coords)
    assert np.array_equal(knnz, km.knnz) and np.array_equal(kpos, km.kpos) and np.array_equal(qkpos, km.qkpos)
    assert np.array_equal(imap, km.imap) and np.array_equal(omap, km.omap)
    o_icsr, o_imc, o_ocsr, o_omc = orc.csr_maps(km)
    assert np.array_equal(icsr, o_icsr) and np.array_equal(ocsr, o_ocsr)
    assert np.array_equal(imc, o_imc) and np.array_equal(omc, o_omc)


def test_literal_on_config1_cloud():
    coords = synth.sphere_plane_cloud()
    km = orc.kernel_map(coords, (3, 3, 3))
    out, imap, omap, knnz, kpos, qkpos, *_ = _literal_maps(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0))
    assert np.array_equal(imap, km.imap) and np.array_equal(omap, km.omap) and np.array_equal(qkpos, km.qkpos)


def test_reference_hash_has_no_false_neighbours_in_coordinate_box():
    """The reference compares 64-bit linear hash values, not coordinates (backend/hash.cuh:156).
    Two coordinates collide iff 23783141*db + 73856093*dx + 19349669*dy + 83492791*dz == 0
    (no wrap: |sum| < 2**40).  Within one batch and the full [0,3259)^3 box there is no
    non-zero solution, so exact keys give the reference's result."""
    r = orc.COORD_BOUND - 1
    dy = np.arange(-r, r + 1, dtype=np.int64)
    hits = []
    for dx in range(0, r + 1):          # by symmetry dx >= 0 suffices
        s = 73856093 * dx + 19349669 * dy
        dz, rem = np.divmod(-s, 83492791)
        ok = (rem == 0) & (np.abs(dz) <= r)
        for j in np.nonzero(ok)[0]:
            if dx or dy[j] or dz[j]:
                hits.append((dx, int(dy[j]), int(dz[j])))
    assert hits == []
    # the two known cross-batch solutions in the full box (|db| <= 7)
    for v in [(5, -1215, 2146, 576), (6, -1204, -1155, 1331)]:
        assert 23783141 * v[0] + 73856093 * v[1] + 19349669 * v[2] + 83492791 * v[3] == 0
    a = np.array([[0, 1215, 0, 0]], np.int32)
    b = np.array([[5, 0, 2146, 576]], np.int32)
    assert orc.ref_linear_hash(a)[0] == orc.ref_linear_hash(b)[0]
    lib = load_literal()
    assert lib.lit_coord_hash(0, 1215, 0, 0) == int(orc.ref_linear_hash(a)[0])


def test_row_accumulation_paths_agree():
    """The oracle adds the products of an offset into their output rows through a 0/1 selection matrix when
    scipy is there, else with numpy.add.at: both are the same float64 sums (repeated rows included)."""
    rng = np.random.default_rng(5)
    rows = rng.integers(0, 300, size=5000)
    vals = rng.standard_normal((5000, 7))
    a = rng.standard_normal((300, 7))
    b = a.copy()
    orc._add_rows(a, rows, vals)
    np.add.at(b, rows, vals)
    assert np.abs(a - b).max() < 1e-12
    small = a.copy()
    orc._add_rows(small, rows[:10], vals[:10])          # below the switch-over: numpy.add.at itself
    np.add.at(b, rows[:10], vals[:10])
    assert np.array_equal(small, b) or np.abs(small - b).max() < 1e-12


def _densify(coords, feats, shape, nb):
    c = torch.as_tensor(coords.astype(np.int64))
    dense = torch.zeros((nb, feats.shape[1]) + tuple(shape), dtype=torch.float64)
    dense[c[:, 0], :, c[:, 1], c[:, 2], c[:, 3]] = torch.as_tensor(feats, dtype=torch.float64)
    return dense


def _dense_weight(w, ks):
    # [kv, Ci, Co] with kp = (ix*ksy+iy)*ksz+iz  ->  [Co, Ci, kx, ky, kz]
    kv, ci, co = w.shape
    return torch.as_tensor(w, dtype=torch.float64).reshape(ks[0], ks[1], ks[2], ci, co).permute(4, 3, 0, 1, 2).contiguous()


@pytest.mark.parametrize("ks", [(3, 3, 3), (3, 1, 3), (5, 5, 5), (1, 3, 1), (2, 2, 2), (2, 3, 3)])
def test_submanifold_values_vs_dense_conv3d(ks):
    coords = synth.random_cloud(seed=21, n=400, extent=8, batches=2)
    ci, co = 5, 7
    kv = ks[0] * ks[1] * ks[2]
    f = synth.features(1, len(coords), ci, np.float64)
    w = synth.weights(1, kv, ci, co, np.float64)
    km = orc.kernel_map(coords, ks)
    out = orc.conv_forward(f, w, km, ks)
    # one empty layer on the high side: with an even kernel size and padding (k-1)//2 the dense output is one
    # shorter than the input, and every voxel must still have its output
    dense = _densify(coords, f, (9, 9, 9), 2)
    ref = F.conv3d(dense, _dense_weight(w, ks), padding=[(k - 1) // 2 for k in ks])
    c = coords.astype(np.int64)
    want = ref[c[:, 0], :, c[:, 1], c[:, 2], c[:, 3]].numpy()
    assert orc.rel_l2(out, want) < 1e-12


@pytest.mark.parametrize("ks,stride,pad", [((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
                                           ((3, 3, 3), (2, 2, 2), (0, 0, 0)), ((2, 3, 1), (2, 1, 1), (0, 1, 0)),
                                           ((3, 3, 3), (1, 2, 1), (1, 0, 1))])
def test_strided_and_transposed_values_vs_dense(ks, stride, pad):
    ext = 9
    coords = synth.random_cloud(seed=22, n=300, extent=ext, batches=2)
    # make sure the extent is really reached so the dense size matches coords_max
    coords = np.unique(np.concatenate([coords, np.array([[0, ext - 1, ext - 1, ext - 1]], np.int32)]), axis=0)
    ci, co = 4, 6
    kv = ks[0] * ks[1] * ks[2]
    f = synth.features(2, len(coords), ci, np.float64)
    w = synth.weights(2, kv, ci, co, np.float64)
    km = orc.kernel_map(coords, ks, stride, pad)
    out = orc.conv_forward(f, w, km, ks)
    dense = _densify(coords, f, (ext,) * 3, 2)
    ref = F.conv3d(dense, _dense_weight(w, ks), stride=stride, padding=pad)
    occ = F.conv3d((dense.abs().sum(1, keepdim=True) > 0).double(), torch.ones((1, 1) + tuple(ks), dtype=torch.float64),
                   stride=stride, padding=pad)
    active = torch.nonzero(occ[:, 0] > 0).numpy()   # sorted (b,x,y,z)
    assert np.array_equal(active.astype(np.int32), km.out_coords)
    oc = km.out_coords.astype(np.int64)
    want = ref[oc[:, 0], :, oc[:, 1], oc[:, 2], oc[:, 3]].numpy()
    assert orc.rel_l2(out, want) < 1e-12
    # transposed conv back onto the original coordinates (script/spconv.py:306-329, 236-244)
    wt = synth.weights(3, kv, co, ci, np.float64)
    back = orc.conv_forward(out, wt, km, ks, transposed=True)
    dense_o = _densify(km.out_coords, out, tuple(ref.shape[2:]), 2)
    wdt = torch.as_tensor(wt).reshape(ks[0], ks[1], ks[2], co, ci).permute(3, 4, 0, 1, 2).contiguous()
    opad = [(ext + 2 * pad[a] - ks[a]) % stride[a] for a in range(3)]
    ref_t = F.conv_transpose3d(dense_o, wdt, stride=stride, padding=pad, output_padding=opad)
    assert tuple(ref_t.shape[2:]) == (ext,) * 3
    c = coords.astype(np.int64)
    want_t = ref_t[c[:, 0], :, c[:, 1], c[:, 2], c[:, 3]].numpy()
    assert orc.rel_l2(back, want_t) < 1e-12


def test_fast_path_divergence_is_documented():
    """k == stride shortcut of the reference (backend/hash.cu:110-139) leaves coordinates
    un-divided; the query kernel assumes divided ones.  The engine follows the generic path."""
    coords = np.array([[0, x, y, z] for x in range(6) for y in (0, 1) for z in (0, 1)], np.int32)
    lit = orc.out_coords_fast_path_literal(coords, (2, 2, 2))
    assert lit[:, 1].tolist() == [0, 2, 4] and not lit[:, 2:].any()
    km = orc.kernel_map(coords, (2, 2, 2), (2, 2, 2))
    assert km.out_coords[:, 1].tolist() == [0, 1, 2] and not km.out_coords[:, 2:].any()
    assert sorted(km.imap.tolist()) == list(range(24))      # every input is mapped exactly once
    # literal fast-path coordinates queried as the reference would: inputs with x in {2,3} are lost
    idx = orc.CoordIndex(coords)
    d = orc.offsets((2, 2, 2), True)
    hit = set()
    for o in lit.astype(np.int64):
        q = np.concatenate([np.zeros((8, 1), np.int64), o[1:] * 2 + d], axis=1)
        hit |= {int(i) for i in idx.find(q) if i >= 0}
    assert {int(coords[i, 1]) for i in hit} == {0, 1, 4, 5}


def test_dense_neighbour_table_symmetry():
    coords = synth.random_cloud(seed=5, n=600, extent=10)
    km = orc.kernel_map(coords, (3, 3, 3))
    nbr = orc.dense_neighbour_table(km)
    # pair (i,o,kp) <=> pair (o,i,kv-1-kp) for a submanifold map
    assert np.array_equal((nbr >= 0).sum(1), (nbr[::-1] >= 0).sum(1))
    kp, o = np.nonzero(nbr >= 0)
    assert np.array_equal(nbr[26 - kp, nbr[kp, o]], o)


def test_sparse_quantize_pinned_by_lexicographic_unique_and_brute_force():
    """The ravelled-code order is the lexicographic (x,y,z) order; first-occurrence and inverse are
    checked against a dictionary walk over the points."""
    rng = np.random.default_rng(3)
    pts = rng.uniform(-3.0, 5.0, size=(4000, 3))
    pts[0:3997:7] = pts[3:4000:7]                         # exact duplicates of other points
    for voxel in [(0.5, 0.5, 0.5), (0.3, 1.1, 0.25)]:
        coords, index, inverse = orc.sparse_quantize(pts, voxel)
        q = np.floor(pts / np.array(voxel)).astype(np.int64)
        want = np.unique(q, axis=0)                       # rows in lexicographic order
        assert np.array_equal(coords, want)
        first = {}
        for i, row in enumerate(map(tuple, q)):
            first.setdefault(row, i)
        assert [first[tuple(r)] for r in want] == index.tolist()
        assert np.array_equal(coords[inverse], q)
    # hand example: voxel 1, points in cells (0,0,0), (-1,0,2), (0,0,0), (-1,0,1)
    c, idx, inv = orc.sparse_quantize(np.array([[0.5, 0.2, 0.9], [-0.1, 0.0, 2.0], [0.0, 0.99, 0.0], [-1.0, 0.5, 1.5]]), (1, 1, 1))
    assert c.tolist() == [[-1, 0, 1], [-1, 0, 2], [0, 0, 0]] and idx.tolist() == [3, 1, 0] and inv.tolist() == [2, 1, 2, 0]


def test_front_end_sparse_quantize_on_numpy_matches_oracle():
    from pcengine_amd import utils
    rng = np.random.default_rng(4)
    pts = rng.uniform(0, 10, size=(3000, 3))
    c, idx, inv = utils.sparse_quantize(pts, 0.4, return_index=True, return_inverse=True)
    oc, oi, ov = orc.sparse_quantize(pts, (0.4, 0.4, 0.4))
    assert np.array_equal(c, oc) and np.array_equal(idx, oi) and np.array_equal(inv, ov)


@pytest.mark.parametrize("ks,stride,pad", [((3, 3, 3), (1, 1, 1), (0, 0, 0)), ((2, 2, 2), (2, 2, 2), (0, 0, 0)),
                                           ((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((3, 1, 3), (1, 1, 1), (0, 0, 0))])
def test_backward_vs_autograd_through_dense_conv3d(ks, stride, pad):
    """grad_feats and grad_W of the oracle against torch.autograd on the densified convolution
    (and on conv_transpose3d for the transposed layer), loss = sum(out * G) at the active sites."""
    ext = 9
    subm = tuple(stride) == (1, 1, 1)
    coords = synth.random_cloud(seed=23, n=260, extent=ext, batches=2)
    coords = np.unique(np.concatenate([coords, np.array([[0, ext - 1, ext - 1, ext - 1]], np.int32)]), axis=0)
    ci, co = 4, 6
    kv = ks[0] * ks[1] * ks[2]
    f = synth.features(3, len(coords), ci, np.float64)
    w = synth.weights(3, kv, ci, co, np.float64)
    km = orc.kernel_map(coords, ks, stride, pad)
    g = np.random.default_rng(3).standard_normal((km.n_out, co))
    gf, gw = orc.conv_backward(f, w, km, ks, g)
    ft = torch.as_tensor(f).requires_grad_(True)
    wt = torch.as_tensor(w).requires_grad_(True)
    c = torch.as_tensor(coords.astype(np.int64))
    dense = torch.zeros((2, ext, ext, ext, ci), dtype=torch.float64).index_put((c[:, 0], c[:, 1], c[:, 2], c[:, 3]), ft).permute(0, 4, 1, 2, 3)
    wd = wt.reshape(ks[0], ks[1], ks[2], ci, co).permute(4, 3, 0, 1, 2)
    ref = F.conv3d(dense, wd, stride=stride, padding=[(k - 1) // 2 for k in ks] if subm else pad)
    oc = torch.as_tensor(km.out_coords.astype(np.int64))
    (ref[oc[:, 0], :, oc[:, 1], oc[:, 2], oc[:, 3]] * torch.as_tensor(g)).sum().backward()
    assert orc.rel_l2(gf, ft.grad.numpy()) < 1e-12 and orc.rel_l2(gw, wt.grad.numpy()) < 1e-12
    if not subm:
        # transposed layer: features live on the output coordinates, gradients flow back to them
        fo = synth.features(4, km.n_out, co, np.float64)
        wT = synth.weights(4, kv, co, ci, np.float64)
        gi = np.random.default_rng(4).standard_normal((len(coords), ci))
        gfo, gwT = orc.conv_backward(fo, wT, km, ks, gi, transposed=True)
        fot = torch.as_tensor(fo).requires_grad_(True)
        wTt = torch.as_tensor(wT).requires_grad_(True)
        dense_o = torch.zeros((2,) + tuple(ref.shape[2:]) + (co,), dtype=torch.float64).index_put(
            (oc[:, 0], oc[:, 1], oc[:, 2], oc[:, 3]), fot).permute(0, 4, 1, 2, 3)
        wdt = wTt.reshape(ks[0], ks[1], ks[2], co, ci).permute(3, 4, 0, 1, 2)
        opad = [(ext + 2 * pad[a] - ks[a]) % stride[a] for a in range(3)]
        up = F.conv_transpose3d(dense_o, wdt, stride=stride, padding=pad, output_padding=opad)
        (up[c[:, 0], :, c[:, 1], c[:, 2], c[:, 3]] * torch.as_tensor(gi)).sum().backward()
        assert orc.rel_l2(gfo, fot.grad.numpy()) < 1e-12 and orc.rel_l2(gwT, wTt.grad.numpy()) < 1e-12


def _load_make_manifest():
    import importlib.util
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_manifest.py")
    spec = importlib.util.spec_from_file_location("make_manifest", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg4", "cfg5"])
def test_manifest_of_benchmark_inputs_is_reproduced(name):
    """tests/golden/manifest.json freezes the voxel counts, pair counts and digests of the benchmark clouds and of
    their kernel maps: the seeded generators and the oracle reproduce it bit for bit."""
    import json
    mm = _load_make_manifest()
    with open(mm.PATH) as f:
        frozen = json.load(f)
    assert set(frozen) == set(mm.CONFIGS)
    assert mm.config_entry(name) == frozen[name]
    # what the frozen numbers must satisfy whatever the generator: pair symmetry of submanifold maps
    sub = frozen[name]["layers"]["k333_s111_p000"]
    assert sub["knnz"] == sub["knnz"][::-1] and sub["knnz"][13] == 0 and sum(sub["knnz"]) == sub["pairs"]
    assert sub["n_out"] == frozen[name]["voxels"]
    down = frozen[name]["layers"].get("k222_s222_p000")
    if down:
        assert down["pairs"] <= frozen[name]["voxels"] and down["n_out"] <= down["pairs"]


@pytest.mark.parametrize("ks,stride,pad", [((3, 3, 3), (1, 1, 1), (0, 0, 0)), ((2, 2, 2), (2, 2, 2), (0, 0, 0)),
                                           ((3, 3, 3), (2, 2, 2), (1, 1, 1))])
def test_timed_cpu_path_computes_what_the_oracle_computes(ks, stride, pad):
    """oracle/cpu_path.py is the torch form bench.py times as the CPU baseline; its values must be the
    float64 oracle's (which the dense conv3d tests above pin) to fp32 rounding."""
    from oracle import cpu_path
    coords = synth.random_cloud(seed=77, n=3000, extent=16, batches=2)
    kv = ks[0] * ks[1] * ks[2]
    f = synth.features(7, len(coords), 24).astype(np.float32)
    w = synth.weights(7, kv, 24, 40).astype(np.float32)
    km = orc.kernel_map(coords, ks, stride, pad)
    want = orc.conv_forward(f.astype(np.float64), w.astype(np.float64), km, ks)
    got = cpu_path.conv_forward_torch(torch.as_tensor(f), torch.as_tensor(w), km, ks).numpy()
    assert got.shape == want.shape and orc.rel_l2(got.astype(np.float64), want) <= 1e-6
    if stride == (1, 1, 1):
        m_ms, c_ms, out, km2 = cpu_path.time_layer(coords, f, w, ks, warmup=0, runs=1)
        assert m_ms > 0 and c_ms > 0 and np.array_equal(km2.imap, km.imap) and np.array_equal(out, got)
