"""The dataflow selector on layers it was not tuned on: widths 48, 80, 160 and 192 over three synthetic clouds of
different density.  Every dataflow the layer's entry points take is timed (HIP-graph replays, outputs and
staging buffers allocated beforehand); the selector's choice must be accepted by its entry point and cost at
most 1.4 times the fastest (measured: the fastest on all fifteen layers).  A test of timings: it is collected
after the parity tests so that a noisy machine cannot hide them."""
import numpy as np
import pytest
import torch

from pcengine_amd import backend, synth
from pcengine_amd.backend import DATAFLOW_FDS, DATAFLOW_OS, DATAFLOW_OSO
from tests.util import DEV, dev_coords

pytestmark = pytest.mark.gpu

CLOUDS = {
    "lidar": lambda: synth.lidar_cloud_100k()[::2].copy(),                               # 0.1 pairs per row
    "surface": lambda: synth.sphere_plane_cloud(),                                       # 4.7
    "filled": lambda: synth.random_cloud(seed=95, n=30000, extent=40, batches=1),        # about 11
}
NAMES = {DATAFLOW_FDS: "fds", DATAFLOW_OS: "os", DATAFLOW_OSO: "oso"}
_maps = {}


def _map(cloud):
    if cloud not in _maps:
        coords = CLOUDS[cloud]()
        _maps[cloud] = backend.build_kernel_map(dev_coords(coords), (3, 3, 3), (1, 1, 1), (0, 0, 0), [0, 0, 0], coords[:, 1:].max(0).tolist(),
                                                True, want_csr=True, batchsize=int(coords[:, 0].max()) + 1)
    return _maps[cloud]


def _graph_ms(fn, calls=10, replays=7):
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(calls):
            fn()
    g.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(replays):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) / calls)
    return float(np.median(times))


@pytest.mark.parametrize("cloud", sorted(CLOUDS))
@pytest.mark.parametrize("c_in,c_out", [(48, 48), (80, 80), (80, 128), (160, 160), (192, 192)])
def test_selector_regret_on_widths_it_was_not_tuned_on(cloud, c_in, c_out):
    km = _map(cloud)
    n = km.n_out
    f = torch.as_tensor(synth.features(3, n, c_in), device=DEV).half()
    w = torch.as_tensor(synth.weights(4, 27, c_in, c_out), device=DEV).half()
    packed = backend.pack_weights(w)
    out = torch.empty((n, c_out), dtype=torch.float16, device=DEV)
    buffer = torch.empty(max(km.qsum * (c_in + c_out), 1), dtype=torch.float16, device=DEV)
    picked = backend.select_dataflow(km, c_in, c_out, torch.float16)
    flows = [DATAFLOW_FDS, DATAFLOW_OS] + ([DATAFLOW_OSO] if backend.oso_takes(km, c_in, c_out, torch.float16) else [])
    assert picked in flows                      # a dataflow whose entry point takes the layer
    ms, ref = {}, None
    for flow in flows:
        y = backend.conv_forward(f, w, km, flow, buffer=buffer, packed=packed, out=out)
        torch.cuda.synchronize()
        if ref is None:
            ref = y.float().clone()
        else:
            assert float((y.float() - ref).norm() / ref.norm()) <= 2e-3
        ms[flow] = _graph_ms(lambda: backend.conv_forward(f, w, km, flow, buffer=buffer, packed=packed, out=out))
    best = min(ms, key=ms.get)
    line = ", ".join(f"{NAMES[k]} {v * 1e3:.1f} us" for k, v in ms.items())
    print(f"\n{cloud} {c_in}->{c_out} rows {n} pairs/row {km.M / n:.2f}: {line}; picked {NAMES[picked]}, regret {ms[picked] / ms[best]:.3f}")
    assert ms[picked] <= 1.4 * ms[best], (cloud, c_in, c_out, {NAMES[k]: round(v * 1e3, 1) for k, v in ms.items()}, NAMES[picked])
