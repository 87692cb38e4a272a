"""The native planner of a network's kernel maps (pce_pyramid_plan / pce_pyramid_build: one allocation, two
library calls) and the forward arena: the same maps bit for bit as the map-by-map builds and as the oracle, the
same network output, and no device allocation in a forward once the plan exists."""
import numpy as np
import pytest
import torch

import pcengine_amd as pe
from oracle import oracle as orc
from pcengine_amd import _lib, backend, nets, synth
from pcengine_amd.spconv import MapPlanner, prebuild_maps
from tests.util import DEV, dev_coords

pytestmark = pytest.mark.gpu

FIELDS = ("imap", "omap", "knnz", "kpos", "qkpos", "out_coords", "nbr_out", "nbr_in", "icsr", "ocsr", "icode", "ocode", "islot", "oslot")


def _tensor(coords, batches, c=4):
    f = torch.as_tensor(synth.features(4, len(coords), c), device=DEV).half()
    return pe.spTensor(f, dev_coords(coords), None, [0, 0, 0], coords[:, 1:].max(0).tolist(), batchsize=batches)


def _assert_same_maps(a, b):
    assert set(a.kmaps) == set(b.kmaps)
    for key, ka in a.kmaps.items():
        kb = b.kmaps[key]
        assert (ka.n_in, ka.n_out, ka.M, ka.qsum, ka.order_heavy, ka.order_nonzero, ka.order_single) == \
               (kb.n_in, kb.n_out, kb.M, kb.qsum, kb.order_heavy, kb.order_nonzero, kb.order_single), key
        for name in FIELDS:
            ta, tb = getattr(ka, name), getattr(kb, name)
            assert (ta is None) == (tb is None), (key, name)
            if ta is not None:
                assert torch.equal(ta, tb), (key, name)
        assert (ka.order is None) == (kb.order is None), key
        if ka.order is not None:
            n = ka.n_out
            assert torch.equal(ka.order[n:2 * n], kb.order[n:2 * n])      # masks (positions of equal keys depend on the run)
    assert set(a.cbook) == set(b.cbook) and all(torch.equal(a.cbook[k], b.cbook[k]) for k in a.cbook)


@pytest.mark.parametrize("cloud", ["lidar", "indoor"])
def test_planned_maps_equal_the_map_by_map_builds_and_the_oracle(cloud):
    if cloud == "lidar":
        coords, batches = synth.lidar_cloud_100k()[::2].copy(), 1
    else:
        coords, batches = synth.random_cloud(seed=71, n=30000, extent=48, batches=3), 3
    layers = [(3, 1, 0), (2, 2, 0), (3, 1, 0), (2, 2, 0), (3, 1, 0), (2, 2, 0), (3, 1, 0)]
    plain, planned = _tensor(coords, batches), _tensor(coords, batches)
    prebuild_maps(plain, layers)
    planner = MapPlanner()
    prebuild_maps(planned, layers, planner)
    assert len(planner.plans) == 1
    _assert_same_maps(plain, planned)
    # the oracle, level by level
    c = coords
    for lv in range(3):
        ref = orc.kernel_map(c, (3, 3, 3))
        code = 94273 * 2 ** lv + 311 * 2 ** lv + 2 ** lv
        km = planned.kmaps[(94273 * 3 + 311 * 3 + 3, code, 94585)]
        assert np.array_equal(km.imap.cpu().numpy(), ref.imap) and np.array_equal(km.omap.cpu().numpy(), ref.omap)
        down = orc.kernel_map(c, (2, 2, 2), (2, 2, 2))
        kd = planned.kmaps[(94273 * 2 + 311 * 2 + 2, code, 94273 * 2 + 311 * 2 + 2)]
        assert np.array_equal(kd.out_coords.cpu().numpy(), down.out_coords)
        assert np.array_equal(kd.imap.cpu().numpy(), down.imap) and np.array_equal(kd.omap.cpu().numpy(), down.omap)
        c = down.out_coords
    # a smaller cloud inside the same box reuses the plan and its allocation; a larger one replaces it
    plan = next(iter(planner.plans.values()))
    arena_ptr = plan.arena.data_ptr()
    small = coords[: len(coords) // 2]
    small = np.concatenate([small, coords[-1:]], 0)        # keeps the box (the last row holds the largest batch index)
    a, b = _tensor(small, batches), _tensor(small, batches)
    a.coords_max = b.coords_max = coords[:, 1:].max(0).tolist()
    prebuild_maps(a, layers)
    prebuild_maps(b, layers, planner)
    assert len(planner.plans) == 1 and next(iter(planner.plans.values())).arena.data_ptr() == arena_ptr
    _assert_same_maps(a, b)


def test_planner_falls_back_where_it_does_not_apply():
    coords = synth.random_cloud(seed=72, n=6000, extent=24, batches=2)
    planner = MapPlanner()
    # unsorted rows: the plan is made, the build reports the cloud, the maps come from the map-by-map path
    perm = np.random.default_rng(0).permutation(len(coords))
    x, y = _tensor(coords[perm].copy(), 2), _tensor(coords[perm].copy(), 2)
    layers = [(3, 1, 0), (2, 2, 0), (3, 1, 0)]
    prebuild_maps(x, layers)
    prebuild_maps(y, layers, planner)
    _assert_same_maps(x, y)
    # a padded strided layer (kernel 3, stride 2) is no bitmap chain: no plan at all
    z = _tensor(coords, 2)
    prebuild_maps(z, [(3, 1, 0), (3, 2, 1), (3, 1, 0)], planner)
    w = _tensor(coords, 2)
    prebuild_maps(w, [(3, 1, 0), (3, 2, 1), (3, 1, 0)])
    _assert_same_maps(w, z)
    # C ABI: sizes and argument checks
    lib = _lib.load()
    assert lib.pce_pyramid_plan_sizeof() == _lib.ctypes.sizeof(_lib.PyrPlan)
    plan = _lib.PyrPlan()
    req = (_lib.PyrRequest * 1)()
    req[0].level_in, req[0].level_out = 0, 1
    req[0].geom = backend.Geom.make((3, 3, 3), (1, 1, 1), (0, 0, 0), [0, 0, 0], [9, 9, 9], True)     # submanifold across levels
    assert lib.pce_pyramid_plan(1000, 0, None, 1, req, 1, plan) == _lib.PCE_EINVAL
    req[0].level_out = 0
    assert lib.pce_pyramid_plan(1000, 0, None, 1, req, 1, plan) == _lib.PCE_OK and plan.arena_bytes > 0
    buf = torch.empty(plan.arena_bytes, dtype=torch.uint8, device=DEV)
    c = dev_coords(synth.random_cloud(seed=73, n=900, extent=9))
    s = torch.cuda.current_stream().cuda_stream
    n = c.shape[0]
    assert 0 < n <= 1000 and int(c[:, 1:].max()) <= 9
    assert lib.pce_pyramid_build(plan, c.data_ptr(), 2000, buf.data_ptr(), buf.numel(), s) == _lib.PCE_ECAPACITY
    assert lib.pce_pyramid_build(plan, c.data_ptr(), n, buf.data_ptr(), buf.numel() - 256, s) == _lib.PCE_EWORKSPACE
    assert lib.pce_pyramid_build(plan, c.data_ptr(), n, buf.data_ptr(), buf.numel(), s) == _lib.PCE_OK, lib.pce_last_error()
    assert plan.map[0].n_in == n and plan.map[0].n_pairs == orc.kernel_map(c.cpu().numpy(), (3, 3, 3)).M


def test_planned_forward_allocates_nothing_and_matches_the_plain_forward():
    """The U-Net with the planner on: bit-identical to the plain forward; from the third forward over a cloud on
    (the first measures the arena, the second allocates it) no device memory is allocated during a forward."""
    coords = synth.lidar_cloud_100k()[::3].copy()
    f = torch.as_tensor(synth.features(4, len(coords), 4), device=DEV).half()
    cd = dev_coords(coords)
    cmax = coords[:, 1:].max(0).tolist()
    torch.manual_seed(4)
    model = nets.SparseResUNet(4, 20).to(DEV).eval().fuse_bn().half()
    mk = lambda: pe.spTensor(f, cd, None, [0, 0, 0], cmax)
    with torch.no_grad():
        want = model(mk()).feats.clone()
        model.use_planner()
        for _ in range(3):
            got = model(mk()).feats
            assert torch.equal(got, want)
        torch.cuda.synchronize()
        before, count = torch.cuda.memory_allocated(), torch.cuda.memory_stats()["allocation.all.allocated"]
        got = model(mk()).feats
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == count
        assert torch.equal(got, want)
        # a larger cloud: the plan and the arena grow, the result is the plain forward's
        big = synth.lidar_cloud_100k()[::2].copy()
        fb = torch.as_tensor(synth.features(5, len(big), 4), device=DEV).half()
        xb = lambda: pe.spTensor(fb, dev_coords(big), None, [0, 0, 0], big[:, 1:].max(0).tolist())
        got_big = model(xb()).feats.clone()
        model.use_planner(False)
        assert torch.equal(got_big, model(xb()).feats)


@pytest.mark.parametrize("planned", [False, True])
def test_network_builds_maps_without_pair_lists_where_its_layers_read_the_table_only(planned, monkeypatch):
    """The U-Net marks the 3x3x3 map of a level table-only when every layer of the level has a width the ordered
    dataflow takes (an fp16 inference forward of the default network: its two upper levels): those maps come without
    pair lists, the others with them, and the forward is bit-identical to one whose maps were all built in full."""
    coords = synth.lidar_cloud_100k()[::3].copy()
    f = torch.as_tensor(synth.features(4, len(coords), 4), device=DEV).half()
    cd = dev_coords(coords)
    cmax = coords[:, 1:].max(0).tolist()
    torch.manual_seed(4)
    model = nets.SparseResUNet(4, 20).to(DEV).eval().fuse_bn().half()
    plan = model.map_plan(torch.float16)
    assert [e[3] for e in plan if len(e) == 4] == [True, True, False, False, False]
    assert not any(e[3] for e in model.map_plan() if len(e) == 4) and not any(e[3] for e in model.map_plan(torch.float32) if len(e) == 4)
    if planned:
        model.use_planner()
    mk = lambda: pe.spTensor(f, cd, None, [0, 0, 0], cmax, batchsize=1)
    with torch.no_grad():
        x = mk()
        lean = model(x).feats.clone()
        subm = sorted((km.n_out, km.has_pairs) for key, km in x.kmaps.items() if km.subm)
        assert [h for _, h in subm] == [True, True, True, False, False]          # by rows: the two largest levels are lean
        assert all(km.has_pairs for km in x.kmaps.values() if not km.subm)
        monkeypatch.setattr(model, "map_plan", lambda dtype=None: [e[:3] for e in plan])
        y = mk()
        full = model(y).feats.clone()
        assert all(km.has_pairs for km in y.kmaps.values())
    assert torch.equal(lean, full)
    # a forced dataflow that reads pair lists on a lean map builds them then
    km = max((km for km in x.kmaps.values() if km.subm), key=lambda k: k.n_out)
    w = torch.as_tensor(synth.weights(2, 27, 32, 32), device=DEV).half()
    g = torch.as_tensor(synth.features(3, km.n_out, 32), device=DEV).half()
    a = backend.conv_forward(g, w, km, backend.DATAFLOW_FDS)
    assert km.has_pairs
    b = backend.conv_forward(g, w, km, backend.DATAFLOW_OSO)
    assert float((a.float() - b.float()).norm() / b.float().norm()) <= 2e-3
