"""Configurations 4 and 5 at their real shapes: every distinct layer shape of the two networks against the
float64 oracle on a small cloud, every layer of the real full-size forwards against the oracle on sampled
output rows, the whole configuration-4 forward against the oracle's float64 forward, and the forced
dataflows against the selector's choice.  Bars: rel-L2 <= 1e-3 per fp16 layer (the parity contract); a whole
network of ~45 fp16 layers accumulates storage rounding and is held to the bar stated at each test."""
import numpy as np
import pytest
import torch

import pcengine_amd as pe
from oracle import oracle as orc
from pcengine_amd import backend, nets, synth
from pcengine_amd.backend import DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS
from tests import netref
from tests.util import DEV, dev_coords, rounded

pytestmark = pytest.mark.gpu

FLOWS = [DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS]
NETS = {
    "cfg4": dict(stem=32, enc=(32, 64, 128, 256), dec=(256, 128, 96, 96)),
    "cfg5": dict(stem=64, enc=(64, 128, 256, 512), dec=(512, 256, 192, 192)),
}
CLOUDS = {"cfg4": synth.lidar_cloud_100k, "cfg5": synth.indoor_batch}


def _layer_shapes():
    """Distinct (kind, c_in, c_out) of the convolutions of both networks, read off the module trees."""
    shapes = set()
    for kw in NETS.values():
        with torch.device("meta"):      # shapes only: no parameter memory
            model = nets.SparseResUNet(4, 20, **kw)
        for m in model.modules():
            if isinstance(m, pe.conv3d):
                ks, st = tuple(m.kernel_size), tuple(m.stride)
                kind = "1x1" if ks == (1, 1, 1) else ("up" if m.transposed else ("down" if st == (2, 2, 2) else "subm3"))
                shapes.add((kind, m.in_channels, m.out_channels))
    return sorted(shapes)


SHAPES = _layer_shapes()


def test_the_layer_shapes_cover_both_networks():
    assert ("subm3", 768, 512) in SHAPES and ("subm3", 512, 512) in SHAPES and ("1x1", 768, 512) in SHAPES
    assert ("down", 256, 256) in SHAPES and ("up", 512, 512) in SHAPES and ("up", 512, 256) in SHAPES
    assert ("subm3", 384, 256) in SHAPES and ("subm3", 128, 96) in SHAPES and ("subm3", 4, 32) in SHAPES
    assert ("1x1", 192, 20) in SHAPES and ("1x1", 96, 20) in SHAPES


@pytest.mark.parametrize("kind,c_in,c_out", SHAPES)
def test_network_layer_shapes_against_the_oracle(kind, c_in, c_out):
    """Every distinct layer shape of the configuration-4 and configuration-5 networks (32..256 with a 96-wide
    decoder; 64..512 with 768 -> 512, 512 -> 512, the 1x1 768 -> 512 shortcut and the 512-wide k2s2 layers), fp16
    with the folded-norm epilogue (bias, ReLU), through the selector's dataflow and each of the four forced
    ones, against the float64 oracle on a cloud small enough for it."""
    dt = torch.float16
    coords = synth.random_cloud(seed=71, n=3500, extent=14, batches=2)
    rng = np.random.default_rng(c_in * 1000 + c_out)
    kv = {"subm3": 27, "down": 8, "up": 8, "1x1": 1}[kind]
    w = synth.weights(c_in + c_out, kv, c_in, c_out)
    bias = rng.standard_normal(c_out) * 0.1
    wd = torch.as_tensor(w, device=DEV).to(dt)
    bd = torch.as_tensor(bias, device=DEV).to(dt)
    packed = backend.pack_weights(wd)
    if kind == "1x1":
        f = synth.features(3, len(coords), c_in)
        fd = torch.as_tensor(f, device=DEV).to(dt)
        want = np.maximum(rounded(f, dt) @ rounded(w[0], dt) + rounded(bias, dt), 0)
        out = backend.dense_forward(fd, wd[0].contiguous(), backend.pack_weights(wd[0].contiguous()), bias=bd, act="relu")
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3
        return
    if kind == "subm3":
        ref = orc.kernel_map(coords, netref.K3)
        km = backend.build_kernel_map(dev_coords(coords), netref.K3, netref.S1, netref.P0, [0, 0, 0],
                                      coords[:, 1:].max(0).tolist(), True, want_csr=True)
        n_src, transposed = len(coords), False
    else:
        cmax = coords[:, 1:].max(0).tolist()
        ref = orc.kernel_map(coords, netref.K2, netref.S2, netref.P0, cmax=cmax)
        km = backend.build_kernel_map(dev_coords(coords), netref.K2, netref.S2, netref.P0, [0, 0, 0],
                                      orc.strided_coords_max(cmax, netref.K2, netref.S2, netref.P0), False, want_csr=True,
                                      want_nbr_in=True, batchsize=2)
        transposed = kind == "up"
        n_src = ref.n_out if transposed else len(coords)
    assert km.M == ref.M and np.array_equal(km.imap.cpu().numpy(), ref.imap) and np.array_equal(km.omap.cpu().numpy(), ref.omap)
    f = synth.features(3, n_src, c_in)
    fd = torch.as_tensor(f, device=DEV).to(dt)
    if c_in < 16:    # the front end pads a 3- or 4-channel input layer to 16 channels (zero rows in the kernel)
        fd = torch.nn.functional.pad(fd, (0, 16 - c_in))
        wd = torch.nn.functional.pad(wd, (0, 0, 0, 16 - c_in)).contiguous()
        packed = backend.pack_weights(wd)
    want = orc.conv_forward(rounded(f, dt), rounded(w, dt), ref, km.ks, transposed=transposed, bias=rounded(bias, dt))
    want = np.maximum(want, 0)
    picked = backend.select_dataflow(km, c_in, c_out, dt, transposed)
    for flow in [picked] + FLOWS:
        out = backend.conv_forward(fd, wd, km, flow, transposed=transposed, packed=packed, bias=bd, act="relu")
        err = orc.rel_l2(out.double().cpu().numpy(), want)
        assert err <= 1e-3, (kind, c_in, c_out, flow, err)


def _real_model(name):
    torch.manual_seed(4 if name == "cfg4" else 5)
    model = nets.SparseResUNet(4, 20, **NETS[name])
    # norms with statistics away from the identity, so that folding them is visible in the weights
    g = torch.Generator().manual_seed(11)
    for mod in model.modules():
        if isinstance(mod, pe.BatchNorm):
            with torch.no_grad():
                mod.running_mean.uniform_(-0.1, 0.1, generator=g)
                mod.running_var.uniform_(0.6, 1.4, generator=g)
                mod.weight.uniform_(0.8, 1.2, generator=g)
                mod.bias.uniform_(-0.1, 0.1, generator=g)
    return model.to(DEV).eval().fuse_bn().half()


def _input(name, coords):
    f = torch.as_tensor(synth.features(4, len(coords), 4), device=DEV).half()
    batches = int(coords[:, 0].max()) + 1
    return lambda: pe.spTensor(f, dev_coords(coords), None, [0, 0, 0], coords[:, 1:].max(0).tolist(), batchsize=batches)


@pytest.mark.parametrize("name", ["cfg4", "cfg5"])
def test_every_layer_of_the_real_network_against_the_oracle(name, monkeypatch):
    """The real network of the configuration (fp16, norms folded, selector on) on its full-size cloud
    (99 692 LiDAR voxels; 954 111 voxels in eight indoor scenes).  After every convolution the forward executes,
    128 sampled output rows are recomputed in float64 from the layer's own inputs over the oracle's map of that
    level, epilogue included: the per-layer bar of the parity contract, at the real shapes and sizes."""
    coords = CLOUDS[name]()
    model = _real_model(name)
    checker = netref.LayerChecker(backend, netref.oracle_pyramid(coords), rows=128, seed=3)
    checker.install(monkeypatch)
    with torch.no_grad():
        y = model(_input(name, coords)())
    assert y.feats.shape == (len(coords), 20) and bool(torch.isfinite(y.feats).all())
    n_convs = sum(isinstance(m, pe.conv3d) for m in model.modules())
    assert len(checker.records) == n_convs >= 45
    kinds = {r[0] for r in checker.records}
    assert kinds == {"subm3", "k2s2", "Tk2s2", "1x1"}
    worst = max(checker.records, key=lambda r: r[-1])
    assert worst[-1] <= 1e-3, worst
    assert {DATAFLOW_OS, DATAFLOW_FDS} <= {r[5] for r in checker.records}     # the selector used both of its dataflows
    widest = max(r[3] for r in checker.records)
    assert widest == (384 if name == "cfg4" else 768)


def test_config4_network_against_the_float64_oracle_forward():
    """The whole configuration-4 forward (fp16 storage, fp32 accumulate, 46 layers) against the oracle's float64
    forward with the same (fp16-rounded) weights and inputs.  Per layer the bar is 1e-3; end to end the storage
    roundings of 46 layers add up (about sqrt(46) x 2.4e-4 if independent), so the whole network is held to
    5e-3, and to the same coordinates exactly."""
    coords = CLOUDS["cfg4"]()
    model = _real_model("cfg4")
    with torch.no_grad():
        y = model(_input("cfg4", coords)())
    ref_model = model.float().cpu()           # the fp16 weights, exactly, for the float64 walk
    f16 = torch.as_tensor(synth.features(4, len(coords), 4)).half().double().numpy()
    want_c, want = netref.oracle_forward(ref_model, coords, f16)
    assert np.array_equal(y.coords.cpu().numpy(), want_c)
    err = orc.rel_l2(y.feats.double().cpu().numpy(), want)
    assert err <= 5e-3, err


@pytest.mark.parametrize("name", ["cfg4", "cfg5"])
def test_forced_dataflows_agree_with_the_selector_on_the_real_network(name, monkeypatch):
    """Full-size forward of the real network with every layer forced to one dataflow (fetch-on-demand, gather-GEMM-
    scatter, output-stationary, deferred scatter) against the forward the selector composes.  All five compute
    the same sums in fp32 and round to fp16 at different places; the difference accumulated over the network
    stays below 5e-3."""
    coords = CLOUDS[name]()
    model = _real_model(name)
    make = _input(name, coords)
    with torch.no_grad():
        auto = model(make()).feats.double()
        for flow in ("fds", "os", "gms", "fod"):
            monkeypatch.setenv("PCENGINE_DATAFLOW", flow)
            out = model(make()).feats.double()
            monkeypatch.delenv("PCENGINE_DATAFLOW")
            err = float((out - auto).norm() / auto.norm())
            assert err <= 5e-3, (flow, err)
            del out
