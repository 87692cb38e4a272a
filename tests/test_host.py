"""CPU-side checks: the C-ABI library loads and exports what include/pcengine_amd.h declares,
the host logic of the front end, and the loud failure without a GPU.  No compute calls."""
import os
import re

import numpy as np
import pytest
import torch

import pcengine_amd as pe
from pcengine_amd import _lib, backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "pcengine_amd.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(pce_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = _lib.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared but not exported"
    assert declared == set(_lib.exported_names())
    assert lib.pce_version() >= 100
    # the stage mask of the measurement build is no part of the product library
    assert not hasattr(lib, "pce_set_stage_mask")
    extra = open(os.path.join(ROOT, "include", "pcengine_amd_measure.h")).read()
    extra = re.sub(r"/\*.*?\*/", "", extra, flags=re.S)
    assert set(re.findall(r"\b(pce_[a-z0-9_]+)\s*\(", extra)) == {"pce_set_stage_mask"}
    with _lib.measurement_build() as mlib:
        assert _lib.load() is mlib
        for name in sorted(declared) + ["pce_set_stage_mask"]:
            assert hasattr(mlib, name), f"{name} is missing from the measurement build"
    assert _lib.load() is lib


def test_pure_host_entry_points():
    lib = _lib.load()
    assert lib.pce_hash_slots(1) == 8 and lib.pce_hash_slots(20000) == 65536 and lib.pce_hash_slots(150000) == 524288
    assert lib.pce_hash_table_bytes(150000) == 524288 * 16
    g = _lib.Geom.make((2, 2, 2), (2, 2, 2), (0, 0, 0), (0, 0, 0), (10, 10, 10), False)
    assert lib.pce_outcoords_workspace_bytes(1000, g, 0) > 0
    bad = _lib.Geom.make((0, 2, 2), (2, 2, 2), (0, 0, 0), (0, 0, 0), (10, 10, 10), False)
    assert lib.pce_outcoords_workspace_bytes(1000, bad, 0) == -1
    assert lib.pce_kmap_workspace_bytes(1000, 1000, 27, 1) > lib.pce_kmap_workspace_bytes(1000, 1000, 27, 0)
    assert lib.pce_conv_fod_workspace_bytes(1000, 64, _lib.PCE_F16) == 1000 * 64 * 4
    assert lib.pce_conv_fod_workspace_bytes(1000, 64, _lib.PCE_F32) == 0


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    assert lib.pce_conv_fwd_fod(None, None, None, None, 0, 1, 1, 1, 1, 1, -1, None, None, None, None, 0, None, 0, None, None) == _lib.PCE_EINVAL
    with pytest.raises(ValueError):
        _lib.check(_lib.PCE_EINVAL)
    one = 1
    fod = lambda n_in, n_out, qsum, ws: lib.pce_conv_fwd_fod(one, one, None, one, 0, n_in, n_out, 4, 4, 27, 13, one, one, one, one, qsum, one, ws, None, None)
    assert fod(10, 10, 100, 1 << 20) == _lib.PCE_EINVAL        # qsum % 128
    assert fod(10, 12, 128, 1 << 20) == _lib.PCE_EINVAL        # a centre offset needs n_in == n_out
    assert fod(10, 10, 128, 16) == _lib.PCE_EWORKSPACE
    assert lib.pce_conv_fwd_gms(one, one, None, one, 0, 10, 10, 4, 4, 27, 13, one, one, one, one, one, one, 128, one, 10, None, None) == _lib.PCE_EWORKSPACE
    assert lib.pce_conv_fwd_fds(one, one, None, one, 0, 10, 10, 4, 4, 27, 13, one, one, one, one, one, None, None, one, None, 100, 128, one, 10, None, None) == _lib.PCE_EWORKSPACE
    assert lib.pce_conv_fwd_os(one, one, None, one, 7, 10, 10, 4, 4, 27, one, None, None) == _lib.PCE_EINVAL      # dtype
    epi = _lib.Epilogue()
    epi.act = 9
    assert lib.pce_conv_fwd_os(one, one, None, one, 0, 10, 10, 4, 4, 27, one, epi, None) == _lib.PCE_EINVAL     # activation
    epi.act, epi.residual = _lib.ACT_RELU, one
    assert lib.pce_conv_fwd_os(one, one, None, one, 0, 10, 10, 4, 4, 27, one, epi, None) == _lib.PCE_EINVAL     # residual aliases out
    assert b"alias" in lib.pce_last_error()
    assert lib.pce_packed_weight_bytes(_lib.PCE_F16, 27, 64, 64) == 27 * 8 * 64 * 16
    assert lib.pce_packed_weight_bytes(_lib.PCE_F16, 27, 4, 20) == 27 * 1 * 32 * 16
    assert lib.pce_packed_weight_bytes(_lib.PCE_F32, 27, 64, 64) == 0


def test_selector_is_monotone_in_density():
    lib = _lib.load()
    n = 100000
    picks = [lib.pce_select_dataflow(n, n, int(rho * n), 64, 64, 27, 13, 0, 0) for rho in (0.1, 0.5, 1.0, 3.0, 8.0, 20.0)]
    assert picks[0] == _lib.DATAFLOW_OSO and picks[-1] == _lib.DATAFLOW_OS
    order = {_lib.DATAFLOW_OSO: 0, _lib.DATAFLOW_FDS: 0, _lib.DATAFLOW_FOD: 0, _lib.DATAFLOW_GMS: 1, _lib.DATAFLOW_OS: 2}
    ranks = [order[p] for p in picks]
    assert ranks == sorted(ranks)


def test_selector_on_measured_layers():
    """Layers whose four dataflows were timed on the GPU: the selector picks the fastest (or one within 2 % of it)."""
    lib = _lib.load()
    FDS, OS, OSO = _lib.DATAFLOW_FDS, _lib.DATAFLOW_OS, _lib.DATAFLOW_OSO
    cases = [  # n_in, n_out, pairs, c_in, c_out, kv, expected
        (149866, 149866, 30620, 64, 64, 27, OSO),      # the headline layer
        (97941, 97941, 80234, 32, 32, 27, OSO),        # narrow layers of a LiDAR network: rho 0.8 and 3.0
        (89469, 89469, 271786, 64, 64, 27, OSO),
        (541185, 541185, 2852000, 64, 64, 27, OSO),    # indoor batch, rho 5.3: equal to output-stationary, 0.6 of deferred scatter
        (99692, 99692, 13406, 96, 96, 27, OSO),        # hardly any pairs: 18-20 vs 20-22 us for deferred scatter
        (97941, 97941, 80234, 96, 96, 27, OSO),        # the K-stepped ordered kernel: 28 vs 32 us
        (97941, 97941, 80234, 128, 96, 27, OSO),       # 31 vs 34 us
        (89469, 89469, 271786, 128, 128, 27, FDS),     # wider than the ordered kernels take: 64 vs 67 us
        (89469, 89469, 271786, 192, 128, 27, FDS),
        (65807, 65807, 586656, 64, 64, 27, OS),        # rho 8.9: the dense tiles
        (149866, 146018, 149866, 64, 128, 8, OSO),     # k2s2 on a LiDAR cloud, one pair for nearly every row: 21.3 vs 24.5 us (FDS)
        (149866, 146018, 149866, 128, 128, 8, FDS),    # ... wider than the ordered kernels take: routed deferred scatter
        (541185, 216268, 539306, 128, 96, 8, OSO),     # indoor batch, 2.5 pairs per row: 60 vs 65 us (OS)
        (216268, 53439, 215000, 128, 128, 8, OS),      # k2s2 on an indoor batch, four pairs per row
        (65807, 25916, 64194, 128, 128, 8, OS),
        (53439, 53439, 550000, 128, 256, 27, OS),      # rho = 10.3
        (53439, 53439, 550000, 256, 256, 27, FDS),
        (25916, 25916, 506646, 256, 256, 27, OS),      # rho = 19.5
        (12063, 12063, 140000, 512, 512, 27, FDS),
        (65807, 65807, 586656, 64, 128, 27, OSO),      # 56 vs 63 us for the dense tiles
        (25916, 25916, 506646, 64, 128, 27, OS),       # rho = 19.5: 33 vs 37 us
    ]
    mid_of = lambda kv: kv // 2 if kv == 27 else -1
    for n_in, n_out, pairs, ci, co, kv, want in cases:
        assert lib.pce_select_dataflow(n_in, n_out, pairs, ci, co, kv, mid_of(kv), 0, _lib.PCE_F16) == want, (n_in, n_out, ci, co, kv)
    sel = lambda n_in, n_out, pairs, ci, co, kv, dt, transposed=0: lib.pce_select_dataflow(n_in, n_out, pairs, ci, co, kv, mid_of(kv), transposed, dt)
    # fp32: the ordered dataflow up to 32 channels (configuration 1), deferred scatter beyond
    assert sel(20804, 20804, 98238, 16, 16, 27, _lib.PCE_F32) == OSO
    assert sel(20804, 20804, 98238, 64, 64, 27, _lib.PCE_F32) == FDS
    assert sel(20804, 20804, 98238, 32, 32, 27, _lib.PCE_F32) == FDS      # 32 channels: only on sparse clouds
    assert sel(149866, 149866, 30620, 32, 32, 27, _lib.PCE_F32) == OSO
    # narrow 2x2x2 stride-2 layers in fp16: the ordered rows up to two pairs per output row, the dense tiles beyond;
    # never in fp32, never for the transposed layer
    assert sel(149866, 146018, 149866, 32, 32, 8, _lib.PCE_F16) == OSO
    assert sel(99692, 97941, 99692, 32, 32, 8, _lib.PCE_F16) == OSO
    assert sel(89469, 65807, 89469, 64, 64, 8, _lib.PCE_F16) == OSO       # 1.36 pairs per row
    assert sel(679728, 276205, 679728, 64, 64, 8, _lib.PCE_F16) == OS     # 2.46 on an indoor batch
    assert sel(149866, 146018, 149866, 32, 32, 8, _lib.PCE_F32) != OSO
    assert sel(146018, 149866, 149866, 32, 32, 8, _lib.PCE_F16, 1) != OSO
    # The ordered dataflow is answered only for layers its entry point takes: over a grid of widths, kernel volumes,
    # centre offsets, dtypes and densities every OSO answer is a layer pce_conv_oso_takes accepts, never a transposed
    # one; an fp32 layer without a centre offset and equal row counts (a strided layer that lost no rows) is not one.
    for dt in (_lib.PCE_F16, _lib.PCE_F32):
        for kv, mid in ((27, 13), (27, -1), (8, -1), (125, 62), (31, 15), (33, 16), (9, 4)):
            for ci in (4, 8, 16, 24, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256):
                for co in (8, 16, 20, 32, 48, 64, 72, 80, 96, 128, 160, 192, 256):
                    for n_in, n_out, pairs in ((50000, 50000, 5000), (50000, 50000, 100000), (50000, 50000, 600000), (50000, 40000, 50000)):
                        for tr in (0, 1):
                            if lib.pce_select_dataflow(n_in, n_out, pairs, ci, co, kv, mid, tr, dt) == OSO:
                                assert tr == 0 and lib.pce_conv_oso_takes(dt, ci, co, kv, mid) == 1, (dt, kv, mid, ci, co, n_in, n_out)
    assert lib.pce_select_dataflow(50000, 50000, 50000, 16, 16, 27, -1, 0, _lib.PCE_F32) != OSO
    assert lib.pce_conv_oso_takes(_lib.PCE_F16, 80, 96, 27, 13) == 1 and lib.pce_conv_oso_takes(_lib.PCE_F16, 112, 96, 27, 13) == 1
    assert lib.pce_conv_oso_takes(_lib.PCE_F16, 128, 128, 27, 13) == 0 and lib.pce_conv_oso_takes(_lib.PCE_F16, 112, 128, 27, 13) == 0
    assert lib.pce_conv_oso_takes(_lib.PCE_F16, 64, 64, 33, 16) == 0


def test_network_map_plan_marks_levels_whose_layers_read_the_table_only():
    """`SparseResUNet.map_plan(dtype)`: a level is table-only when all of its 3x3x3 layers have widths
    `pce_conv_oso_takes` accepts in that dtype -- the two upper levels of the default network in fp16, none in fp32
    (96 channels), none without a dtype (training), none when a dataflow is forced."""
    import torch
    from pcengine_amd import nets
    marks = lambda plan: [e[3] for e in plan if len(e) == 4]
    m = nets.SparseResUNet(4, 20)
    assert marks(m.map_plan(torch.float16)) == [True, True, False, False, False]
    assert marks(m.map_plan(torch.float32)) == [False] * 5 and marks(m.map_plan()) == [False] * 5
    assert [e[:3] for e in m.map_plan()] == [(3, 1, 0), (2, 2, 0), (3, 1, 0), (2, 2, 0), (3, 1, 0), (2, 2, 0), (3, 1, 0), (2, 2, 0), (3, 1, 0)]
    narrow = nets.SparseResUNet(4, 20, stem=16, enc=(16, 32, 32, 64), dec=(64, 32, 32, 16))
    assert marks(narrow.map_plan(torch.float16)) == [True, True, True, False, True]      # the fourth level has a 96 -> 64 layer: no ordered width
    assert marks(nets.SparseResUNet(4, 20, dataflow="fds").map_plan(torch.float16)) == [False] * 5


def test_codes_and_strides():
    assert pe.conv_info_encoder([1, 1, 1]) == 94585
    for v in [(1, 1, 1), (2, 2, 2), (3, 1, 5), (8, 8, 8)]:
        assert pe.conv_info_decoder(pe.conv_info_encoder(list(v))) == v
        assert backend.decode3(pe.conv_info_encoder(list(v))) == v
    assert pe.output_stride_compute(pe.conv_info_encoder([2, 2, 2]), pe.conv_info_encoder([2, 2, 2])) == pe.conv_info_encoder([4, 4, 4])
    assert pe.output_stride_compute(pe.conv_info_encoder([2, 2, 2]), pe.conv_info_encoder([4, 4, 4]), True) == pe.conv_info_encoder([2, 2, 2])


def test_quantize_and_collate():
    rng = np.random.default_rng(0)
    pts = rng.uniform(0, 1, size=(2000, 3))
    q, idx, inv = pe.sparse_quantize(pts, 0.1, return_index=True, return_inverse=True)
    assert q.dtype == np.int32 and len(np.unique(q, axis=0)) == len(q)
    assert np.array_equal(q[inv], np.floor(pts / 0.1).astype(np.int32))
    assert np.array_equal(np.floor(pts[idx] / 0.1).astype(np.int32), q)
    assert (np.diff(pe.ravel_hash(q).astype(np.int64)) > 0).all()     # sorted by the mixed-radix code
    a = pe.spTensor(torch.ones(len(q), 3), torch.as_tensor(q), None, [0, 0, 0], q.max(0).tolist())
    b = pe.spTensor(torch.ones(5, 3), torch.as_tensor(q[:5]), None, [0, 0, 0], q.max(0).tolist())
    x = pe.sparse_collate([a, b])
    assert x.coords.shape == (len(q) + 5, 4) and x.coords.dtype == torch.int32 and x.batchsize == 2
    assert x.coords[-1, 0] == 1 and x.coords_min == [0, 0, 0] and x.coords_max == q.max(0).tolist()
    y = pe.cat([x, x])
    assert y.feats.shape[1] == 6 and y.kmaps is x.kmaps and y.cbook is x.cbook
    z = x + x
    assert torch.equal(z.feats, x.feats * 2) and z.kmaps is x.kmaps
    assert x.F is x.feats and x.C is x.coords and x.stride == 94585
    # rows keep their order, sample k carries k in column 0, numpy members are converted
    assert torch.equal(x.coords[:len(q), 1:], torch.as_tensor(q)) and int(x.coords[:len(q), 0].max()) == 0
    assert torch.equal(x.coords[len(q):, 1:], torch.as_tensor(q[:5])) and int(x.coords[len(q):, 0].min()) == 1
    n1 = pe.spTensor(np.ones((4, 2), np.float32), q[:4].copy(), None, [0, 0, 0], [9, 9, 9])
    n2 = pe.spTensor(np.ones((3, 2), np.float32), q[:3].copy(), None, [0, 0, 0], [9, 9, 9])
    xn = pe.sparse_collate([n1, n2])
    assert isinstance(n1.coords, torch.Tensor) and xn.feats.shape == (7, 2) and xn.coords[:, 0].tolist() == [0] * 4 + [1] * 3
    odd = pe.spTensor(torch.ones(2, 3), torch.as_tensor(q[:2]), None, [0, 0, 0], [9, 9, 9], stride=94273 * 2 + 311 * 2 + 2)
    with pytest.raises(AssertionError):
        pe.sparse_collate([a, odd])


def test_collate_fn_and_ntuple():
    from pcengine_amd.utils import make_ntuple, sparse_collate_fn
    q = np.arange(12, dtype=np.int32).reshape(4, 3)
    mk = lambda k: pe.spTensor(torch.full((k, 2), float(k)), torch.as_tensor(q[:k]), None, [0, 0, 0], [11, 11, 11])
    samples = [{"pc": mk(2), "label": np.array([1, 2]), "t": torch.zeros(2), "name": "a", "nest": {"v": np.array([5])}},
               {"pc": mk(3), "label": np.array([3, 4, 5]), "t": torch.ones(3), "name": "b", "nest": {"v": np.array([6])}}]
    out = sparse_collate_fn(samples)
    assert isinstance(out["pc"], pe.spTensor) and out["pc"].coords.shape == (5, 4) and out["pc"].batchsize == 2
    assert out["label"].tolist() == [1, 2, 3, 4, 5] and out["t"].tolist() == [0, 0, 1, 1, 1]
    assert out["name"] == ["a", "b"] and out["nest"]["v"].tolist() == [5, 6]
    assert sparse_collate_fn([1, 2]) == [1, 2]
    assert make_ntuple(3, 3) == (3, 3, 3) and make_ntuple([1, 2, 3], 3) == (1, 2, 3)
    assert make_ntuple(torch.tensor([[2, 2, 2]]), 3) == (2, 2, 2) and make_ntuple((4, 5), 2) == (4, 5)
    with pytest.raises(AssertionError):
        make_ntuple([1, 2], 3)


def test_module_construction_and_errors():
    c = pe.conv3d(4, 8, 3)
    assert tuple(c.kernel.shape) == (27, 4, 8) and c.bias is None
    bound = 1 / np.sqrt(8 * 27)
    assert float(c.kernel.abs().max()) <= bound
    assert tuple(pe.conv3d(4, 8, 1).kernel.shape) == (4, 8)
    assert "stride=[2, 2, 2]" in repr(pe.conv3d(4, 8, 2, 2, transposed=True)) and "transposed=True" in repr(pe.conv3d(4, 8, 2, 2, transposed=True))
    assert set(pe.conv3d(4, 8, 3, bias=True).state_dict()) == {"kernel", "bias"}
    for kw in ({"kernel_size": (3, 3, 3)}, {"stride": 1.5}, {"padding": "same"}):
        with pytest.raises(NotImplementedError):
            pe.conv3d(4, 8, **kw)
    with pytest.raises(NotImplementedError):
        pe.conv3d(4, 8, dataflow="magic")


def test_sparse_tensor_container_and_activations_on_cpu():
    """Fields, aliases, in-place movement and shared caches of spTensor (script/sptensor.py:4-91); ReLU and
    LeakyReLU act on the features only (script/activation.py:6-15) and name their fused-epilogue form."""
    feats = torch.tensor([[-1.0, 2.0], [3.0, -4.0], [0.0, 0.5]])
    coords = torch.tensor([[0, 1, 2, 3], [0, 4, 5, 6], [1, 7, 8, 9]], dtype=torch.int32)
    x = pe.spTensor(feats, coords)
    assert x.coords_min == [0, 0, 0] and x.coords_max == [7, 8, 9] and x.init_tag == ["end"] and x.batchsize == 1
    assert x.F is x.feats and x.C is x.coords and len(x) == 3 and "N=3" in repr(x)
    x.F = feats * 2
    assert torch.equal(x.feats, feats * 2)
    x.F = feats
    y = pe.ReLU()(x)
    assert torch.equal(y.feats, feats.clamp(min=0)) and y.coords is x.coords and y.kmaps is x.kmaps and y.cbook is x.cbook
    z = pe.LeakyReLU(0.25)(x)
    assert torch.equal(z.feats, torch.where(feats > 0, feats, feats * 0.25))
    assert pe.ReLU().as_epilogue() == "relu" and pe.LeakyReLU(0.25).as_epilogue() == ("leaky_relu", 0.25)
    assert torch.equal((x + y).feats, feats + feats.clamp(min=0)) and (x + y).kmaps is x.kmaps
    assert x.detach() is x and x.cpu() is x and x.to("cpu") is x
    x.build_buffer({"kernel": [3, 2], "in": [4, 16], "out": [8, 32]}, "cpu")
    assert x.buffer.numel() == (16 + 32) * 3 * 16 and x.buffer.dtype == torch.float32
    inplace = pe.ReLU(True)(x)
    assert inplace.feats.data_ptr() == x.feats.data_ptr() and float(x.feats.min()) == 0.0


def test_no_cpu_compute_path():
    x = pe.spTensor(torch.zeros(3, 4), torch.zeros(3, 4, dtype=torch.int32), None, [0, 0, 0], [0, 0, 0])
    with pytest.raises(RuntimeError, match="no CPU compute path"):
        pe.conv3d(4, 8, 3)(x)
    with pytest.raises(RuntimeError, match="no CPU compute path"):
        pe.conv3d(4, 8, 1)(x)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libpcengine_amd.so")
    with pytest.raises(_lib.PCEError, match="no other compute path"):
        _lib.load()


def test_scheduler_hint_and_buffer_size():
    assert pe.init_layer_scheduler({"stride": [1, 1, 2], "in": [4, 32, 32], "out": [32, 32, 64]}) == "simple"
    assert pe.init_layer_scheduler({"stride": [1, 1, 2], "in": [4, 64, 64], "out": [64, 64, 64]}) == "whole"
    buf = pe.build_conv_buffer({"in": [4, 8], "out": [8, 16], "kernel": [3, 2]}, 10, torch.float16, "cpu")
    assert buf.numel() == (8 + 16) * 10 * 16 and buf.dtype == torch.float16



# mangled-name prefixes: wave_os_kernel<2,4>, wave_gemm_kernel<2,4>, tile_gemm_kernel<half,4|3,FAST,MODE_OS,EPI_ROWS>, pipe_gemm_kernel<*>
_VGPR_CEILINGS = [("_Z14wave_os_kernelILi2ELi4E", 128), ("_Z16wave_gemm_kernelILi2ELi4E", 72),
                  ("_Z16tile_gemm_kernelIDF16_Li4ELb1ELi3ELi1E", 96), ("_Z16tile_gemm_kernelIDF16_Li3ELb1ELi3ELi1E", 80),
                  ("_Z16pipe_gemm_kernelILi", 128),
                  ("_Z15wave_osw_kernelILi", 168)]      # three wavefronts per SIMD for every shape of the K-stepped ordered kernel

def test_no_kernel_uses_scratch_memory(tmp_path):
    """Register spills turn a memory-bound kernel into a several times slower one without changing a
    single result: compile the device code with resource remarks and require zero scratch bytes."""
    import subprocess
    from pcengine_amd import build as pb
    procs = []
    for src in pb.SOURCES:
        cmd = [pb._hipcc(), *pb.HIPCC_FLAGS, "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage",
               "-I", os.path.join(ROOT, "include"), "-I", pb.CSRC, "-c", os.path.join(pb.CSRC, src),
               "-o", str(tmp_path / (src + ".o"))]
        procs.append(subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
    seen, ceilings_seen = 0, set()
    for p in procs:
        out, _ = p.communicate()
        assert p.returncode == 0, out[-2000:]
        name = None
        for line in out.splitlines():
            m = re.search(r"Function Name: (\S+)", line)
            if m:
                name = m.group(1)
            m = re.search(r"VGPRs Spill: (\d+)", line)
            if m:
                assert int(m.group(1)) == 0, f"{name} spills {m.group(1)} vector registers"
            m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
            if m:
                seen += 1
                assert int(m.group(1)) == 0, f"{name} spills {m.group(1)} bytes per lane"
            m = re.search(r" VGPRs: (\d+)", line)
            if m:
                # register ceilings of the kernels whose residency the measured figures rest on (a helper shared by
                # all tile kernels once took the output-stationary tiles from 86 to 134 registers: a tenth of a forward)
                for prefix, limit in _VGPR_CEILINGS:
                    if name.startswith(prefix):
                        assert int(m.group(1)) <= limit, f"{name} holds {m.group(1)} vector registers, limit {limit}"
                        ceilings_seen.add(prefix)
    assert seen > 20 and ceilings_seen == {p for p, _ in _VGPR_CEILINGS}


def _function_bodies(src):
    """(name, is_kernel, body) of every __global__ / __device__ function of a HIP source, by brace matching."""
    def closing(text, i, open_ch, close_ch):
        depth = 0
        while True:
            depth += {open_ch: 1, close_ch: -1}.get(text[i], 0)
            if depth == 0:
                return i
            i += 1
    out = []
    for m in re.finditer(r"__global__\s+void\s+|__device__\s+(?:__forceinline__\s+)?[\w:<>,\s\*&]*?(?=\b\w+\s*\()", src):
        i = m.end()
        if src.startswith("__launch_bounds__", i):
            i = closing(src, src.index("(", i), "(", ")") + 1
        nm = re.match(r"\s*(\w+)\s*\(", src[i:])
        if not nm:
            continue
        args_end = closing(src, i + nm.end() - 1, "(", ")")
        rest = src[args_end + 1:]
        if not rest.lstrip().startswith("{"):
            continue
        start = args_end + 1 + rest.index("{")
        out.append((nm.group(1), src[m.start():m.start() + 10] == "__global__", src[start:closing(src, start, "{", "}") + 1]))
    return out


def test_every_global_to_lds_copy_is_followed_by_a_hand_written_wait():
    """The compiler neither tracks nor reliably waits for global -> LDS copies (`global_load_lds`): a read of the
    copied region must stand behind a hand-written `s_waitcnt vmcnt`.  Checked on the text: in a kernel that
    issues such a copy itself, the next mention of the destination array after the copy comes after a wait; a
    helper that issues copies is only called from kernels that also call one of the waiting helpers."""
    src = open(os.path.join(ROOT, "pcengine_amd", "csrc", "pce_conv.hip")).read()
    src = re.sub(r"//[^\n]*", "", src)
    bodies = _function_bodies(src)
    copy = "__builtin_amdgcn_global_load_lds"
    wait = re.compile(r"s_waitcnt vmcnt\(")
    waiting_helpers = [n for n, k, b in bodies if not k and wait.search(b)]
    assert "pipe_wait_copy" in waiting_helpers
    grew = True
    while grew:       # helpers that wait through another helper
        more = [n for n, k, b in bodies if not k and n not in waiting_helpers
                and any(re.search(r"\b" + h + r"\b", b) for h in waiting_helpers)]
        waiting_helpers += more
        grew = bool(more)
    copying_helpers = [n for n, k, b in bodies if not k and copy in b]
    sites = 0
    for name, is_kernel, body in bodies:
        if not is_kernel:
            continue
        if copy in body:
            for m in re.finditer(re.escape(copy) + r"\(", body):
                depth, j = 1, m.end()
                while depth:
                    depth += {"(": 1, ")": -1}.get(body[j], 0)
                    j += 1
                dest = re.search(r"&\s*(\w+)\s*\[", body[m.end():j])
                assert dest, f"{name}: no LDS destination found in a global -> LDS copy"
                sites += 1
                rest = body[j:]
                # skip further copies into the same array (their destination operand is a mention too)
                use = None
                for u in re.finditer(r"\b" + dest.group(1) + r"\s*\[", rest):
                    before = rest[:u.start()]
                    open_copy = before.rfind(copy)
                    if open_copy >= 0 and before.count("(", open_copy) > before.count(")", open_copy):
                        continue
                    use = u
                    break
                if use is not None:
                    assert wait.search(rest[:use.start()]), \
                        f"{name}: {dest.group(1)} is read after a global -> LDS copy with no s_waitcnt vmcnt in between"
        called = [h for h in copying_helpers if re.search(r"\b" + h + r"\s*(<[^;]*?>)?\s*\(", body)]
        if called:
            sites += 1
            assert wait.search(body) or any(re.search(r"\b" + h + r"\b", body) for h in waiting_helpers), \
                f"{name} copies global -> LDS through {called} and never waits by hand"
    assert sites >= 6
