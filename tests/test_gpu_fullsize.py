"""Configurations 3 and 5 at their full sizes: parity with the oracle where it finishes in seconds, and
properties that hold at any size (every dataflow computes the same sums; map symmetries; sortedness)."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from pcengine_amd import backend, synth
from pcengine_amd.backend import DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS
from tests.util import DEV, assert_map_equal, dev_coords, gpu_map, rounded

pytestmark = pytest.mark.gpu

FLOWS = [DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS]


def test_config3_down_then_transposed_up_full_size():
    """k2s2 64->128 on the 150 k-voxel LiDAR cloud, then the transposed layer 128->64 back onto the input
    coordinates over the same map (script/spconv.py:306-329)."""
    coords = synth.lidar_cloud()
    ks, st, pad = (2, 2, 2), (2, 2, 2), (0, 0, 0)
    ref = orc.kernel_map(coords, ks, st, pad)
    km = gpu_map(coords, ks, st, pad, want_csr=True, want_nbr_in=True, batchsize=1)
    assert_map_equal(km, ref, csr=True)
    f = synth.features(3, len(coords), 64)
    w_down = synth.weights(3, 8, 64, 128)
    w_up = synth.weights(4, 8, 128, 64)
    dt = torch.float16
    mid_want = orc.conv_forward(rounded(f, dt), rounded(w_down, dt), ref, ks)
    fd = torch.as_tensor(f, device=DEV).to(dt)
    wd, wu = (torch.as_tensor(w, device=DEV).to(dt) for w in (w_down, w_up))
    # the selector's picks (the K-stepped ordered form for the down layer) run beside the forced dataflows
    picked_down = backend.select_dataflow(km, 64, 128, dt)
    picked_up = backend.select_dataflow(km, 128, 64, dt, transposed=True)
    assert picked_down == backend.DATAFLOW_OSO
    for flow in FLOWS + [backend.DATAFLOW_OSO]:
        mid = backend.conv_forward(fd, wd, km, flow)
        assert orc.rel_l2(mid.double().cpu().numpy(), mid_want) <= 1e-3, flow
        if flow == backend.DATAFLOW_OSO:
            flow = picked_up        # the ordered form has no transposed layer: the selector's pick runs instead
        # the transposed layer sees the fp16 rows the down layer stored
        up_want = orc.conv_forward(mid.double().cpu().numpy(), rounded(w_up, dt), ref, ks, transposed=True)
        up = backend.conv_forward(mid, wu, km, flow, transposed=True)
        assert up.shape == (len(coords), 64)
        assert orc.rel_l2(up.double().cpu().numpy(), up_want) <= 1e-3, flow


def test_config5_indoor_batch_full_size():
    """Eight indoor scenes, ~954 k voxels: the submanifold map against the oracle, its symmetry, and the
    four dataflows against each other and against linearity on a C 64 layer."""
    coords = synth.indoor_batch()
    n = len(coords)
    assert 900_000 < n < 1_000_000 and coords[:, 0].max() == 7
    km = gpu_map(coords, (3, 3, 3), want_csr=True)
    ref = orc.kernel_map(coords, (3, 3, 3))
    assert_map_equal(km, ref, csr=True)
    # pair (i, o, kp) <=> pair (o, i, kv-1-kp): the mirrored pair list is the same set
    kp_of = torch.repeat_interleave(torch.arange(27, device=DEV), km.knnz.long())
    fwd = (kp_of * n + km.imap.long()) * n + km.omap.long()
    mir = ((26 - kp_of) * n + km.omap.long()) * n + km.imap.long()
    assert torch.equal(torch.sort(fwd).values, torch.sort(mir).values)
    # strided level: sorted unique output coordinates; an input is in at most one k2s2 pair (inputs on the
    # far walls fall outside the reference's output bound, script/spconv.py:358-360, and have none)
    k2 = gpu_map(coords, (2, 2, 2), (2, 2, 2), batchsize=8)
    assert_map_equal(k2, orc.kernel_map(coords, (2, 2, 2), (2, 2, 2)))
    oc = k2.out_coords.cpu().numpy().astype(np.int64)
    code = ((oc[:, 0] * 3259 + oc[:, 1]) * 3259 + oc[:, 2]) * 3259 + oc[:, 3]
    assert (np.diff(code) > 0).all()
    assert torch.unique(k2.imap).numel() == k2.M and k2.M < n
    f = synth.features(5, n, 64)
    w = synth.weights(5, 27, 64, 64)
    fd = torch.as_tensor(f, device=DEV).half()
    wd = torch.as_tensor(w, device=DEV).half()
    want = orc.conv_forward(rounded(f, torch.float16), rounded(w, torch.float16), ref, (3, 3, 3))
    packed = backend.pack_weights(wd)
    outs = {flow: backend.conv_forward(fd, wd, km, flow, packed=packed) for flow in FLOWS}
    for flow, out in outs.items():
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3, flow
    # linearity: conv(2x) == 2 conv(x).  Doubling is exact in fp16 and fp32 except for values stored in the
    # fp16 subnormal range (spacing 2^-24): the output itself and each of the up to 26 partial rows of a
    # row.  Such a difference in a partial row (< 1e-7) can also tip the final rounding of the row's sum:
    # one ulp, on a few elements in a million (none with the output-stationary dataflow, which stores no
    # partial rows).  A dropped or doubled pair would change an element by ~0.2.
    for flow in (DATAFLOW_FDS, DATAFLOW_OS):
        twice = backend.conv_forward(fd * 2, wd, km, flow, packed=packed).float()
        ref2 = outs[flow].float() * 2
        diff = (twice - ref2).abs()
        assert bool((diff <= 2.0 ** -10 * ref2.abs() + 27 * 2.0 ** -23).all()), flow
        tipped = int((diff > 27 * 2.0 ** -23).sum())
        assert tipped <= (0 if flow == DATAFLOW_OS else diff.numel() // 100_000), (flow, tipped)


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg4", "cfg5"])
def test_full_size_maps_match_the_frozen_manifest(name):
    """Every benchmark cloud at its full size: the GPU's output coordinates, per-offset counts and pair lists
    against the digests that tests/golden/manifest.json holds (written by the CPU oracle, reproduced by it in
    the CPU suite), submanifold and k2s2 layer, bit for bit."""
    import hashlib
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "manifest.json")) as f:
        frozen = json.load(f)[name]
    gen = {"cfg1": synth.sphere_plane_cloud, "cfg2": synth.lidar_cloud, "cfg4": synth.lidar_cloud_100k,
           "cfg5": synth.indoor_batch}[name]
    coords = gen()

    def digest(*tensors):
        h = hashlib.sha256()
        for t in tensors:
            h.update(np.ascontiguousarray(t.cpu().numpy(), dtype="<i4").tobytes())
        return h.hexdigest()
    assert len(coords) == frozen["voxels"] and digest(torch.as_tensor(coords)) == frozen["coords_sha256"]
    for key, want in frozen["layers"].items():
        ks = tuple(int(c) for c in key[1:4])
        stride = tuple(int(c) for c in key[6:9])
        kw = {} if stride == (1, 1, 1) else {"batchsize": frozen["batches"]}
        km = gpu_map(coords, ks, stride, (0, 0, 0), **kw)
        assert (km.n_out, km.M, km.qsum) == (want["n_out"], want["pairs"], want["qsum"]), key
        assert km.knnz.cpu().tolist() == want["knnz"], key
        assert digest(km.out_coords) == want["out_coords_sha256"], key
        assert digest(km.imap[:km.M], km.omap[:km.M]) == want["pairs_sha256"], key


@pytest.mark.parametrize("name", ["cfg4", "cfg5"])
def test_every_map_of_the_network_pyramid_matches_the_frozen_manifest(name):
    """The nine maps a MinkUNet-style forward builds on a benchmark cloud (five submanifold 3x3x3 maps, four
    k2s2 maps between the levels, script/spconv.py:330-372 once per layer geometry): each level's coordinates,
    per-offset counts and pair lists against the digests of tests/golden/manifest.json, bit for bit.  Every
    level is built from the coordinates the GPU produced for the level before, with the coordinate bound the
    front end carries along (script/spconv.py:358-360)."""
    import hashlib
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "manifest.json")) as f:
        frozen = json.load(f)[name]
    coords = {"cfg4": synth.lidar_cloud_100k, "cfg5": synth.indoor_batch}[name]()

    def digest(*tensors):
        h = hashlib.sha256()
        for t in tensors:
            h.update(np.ascontiguousarray(t.cpu().numpy(), dtype="<i4").tobytes())
        return h.hexdigest()

    def check(km, want, key):
        assert (km.n_out, km.M, km.qsum) == (want["n_out"], want["pairs"], want["qsum"]), key
        assert km.knnz.cpu().tolist() == want["knnz"], key
        assert digest(km.out_coords) == want["out_coords_sha256"], key
        assert digest(km.imap[:km.M], km.omap[:km.M]) == want["pairs_sha256"], key

    cd = dev_coords(coords)
    cmax = coords[:, 1:].max(axis=0).tolist()
    assert len(frozen["pyramid"]) == 5
    for lv in frozen["pyramid"]:
        key = (name, lv["level"])
        assert cd.shape[0] == lv["voxels"] and cmax == lv["coords_max"] and digest(cd) == lv["coords_sha256"], key
        # batch count stated: the column grid (the front end's route); test_full_size_maps_match_the_frozen_manifest
        # builds the level-0 maps through the hash table
        sub = backend.build_kernel_map(cd, (3, 3, 3), (1, 1, 1), (0, 0, 0), [0, 0, 0], cmax, True, want_csr=True,
                                       batchsize=frozen["batches"])
        check(sub, lv["layers"]["k333_s111_p000"], key)
        if "k222_s222_p000" in lv["layers"]:
            cmax = backend.strided_coords_max(cmax, (2, 2, 2), (2, 2, 2), (0, 0, 0))
            down = backend.build_kernel_map(cd, (2, 2, 2), (2, 2, 2), (0, 0, 0), [0, 0, 0], cmax, False, want_csr=True,
                                            batchsize=frozen["batches"])
            check(down, lv["layers"]["k222_s222_p000"], key)
            cd = down.out_coords
