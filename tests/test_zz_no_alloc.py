"""The entry point that allocates nothing: pce_conv_fwd_fod_static keeps the fp32 accumulator of the fp16
fetch-on-demand dataflow in a static device array inside the library.  Checked through the C ABI against
pce_conv_fwd_fod (same kernels, caller-provided workspace) and against the float64 oracle, on two calls in a
row that share the array, the second on a smaller input; plus its size limit."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from pcengine_amd import _lib, backend, synth
from tests.util import DEV, gpu_map, rounded

pytestmark = pytest.mark.gpu


def _both(lib, coords, ks, stride, c_in, c_out, seed, epilogue):
    """(static entry point, workspace entry point, oracle) outputs of one fp16 layer."""
    dt = torch.float16
    km = gpu_map(coords, ks, stride, (0, 0, 0), **({} if stride == (1, 1, 1) else {"batchsize": int(coords[:, 0].max()) + 1}))
    ref = orc.kernel_map(coords, ks, stride, (0, 0, 0))
    kv = km.kv
    f = synth.features(seed, km.n_in, c_in)
    w = synth.weights(seed, kv, c_in, c_out)
    fd = torch.as_tensor(f, device=DEV).to(dt)
    wd = torch.as_tensor(w, device=DEV).to(dt)
    mid = backend._mid(ks) if km.subm else -1
    s = torch.cuda.current_stream().cuda_stream
    epi, keep, want = None, [], orc.conv_forward(rounded(f, dt), rounded(w, dt), ref, ks)
    if epilogue:
        rng = np.random.default_rng(seed)
        bias, res = rng.standard_normal(c_out) * 0.3, rng.standard_normal((km.n_out, c_out))
        bd, rd = torch.as_tensor(bias, device=DEV).to(dt), torch.as_tensor(res, device=DEV).to(dt)
        epi = _lib.Epilogue()
        epi.bias, epi.residual, epi.act, epi.slope = bd.data_ptr(), rd.data_ptr(), _lib.ACT_RELU, 0.0
        keep = [bd, rd]
        want = np.maximum(want + rounded(bias, dt) + rounded(res, dt), 0)
    out_static = torch.full((km.n_out, c_out), float("nan"), dtype=dt, device=DEV)
    out_ws = torch.full((km.n_out, c_out), float("nan"), dtype=dt, device=DEV)
    args = (fd.data_ptr(), wd.data_ptr(), None)
    tail = (_lib.PCE_F16, km.n_in, km.n_out, c_in, c_out, kv, mid, km.imap.data_ptr(), km.omap.data_ptr(), km.kpos.data_ptr(),
            km.qkpos.data_ptr(), km.qsum)
    ws_bytes = lib.pce_conv_fod_workspace_bytes(km.n_out, c_out, _lib.PCE_F16)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    _lib.check(lib.pce_conv_fwd_fod_static(*args, out_static.data_ptr(), *tail, epi, s))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    _lib.check(lib.pce_conv_fwd_fod(*args, out_ws.data_ptr(), *tail, ws.data_ptr(), ws_bytes, epi, s))
    torch.cuda.synchronize()
    del keep
    return out_static, out_ws, want


def test_static_scratch_entry_point_matches_the_workspace_entry_point():
    lib = _lib.load()
    assert lib.pce_conv_fod_static_capacity_bytes() == 32 << 20
    big = synth.random_cloud(seed=81, n=60000, extent=48, batches=2)      # 60 000 x 64 x 4 B = 15 MB of accumulator
    small = synth.random_cloud(seed=82, n=2500, extent=14, batches=1)     # reuses the front of the same array
    for coords, ks, stride, c_in, c_out, epilogue in [(big, (3, 3, 3), (1, 1, 1), 64, 64, False),
                                                      (small, (3, 3, 3), (1, 1, 1), 32, 96, True),
                                                      (big, (2, 2, 2), (2, 2, 2), 64, 128, True),   # no centre offset: zero fill
                                                      (small, (2, 2, 2), (2, 2, 2), 16, 16, False)]:
        a, b, want = _both(lib, coords, ks, stride, c_in, c_out, seed=7, epilogue=epilogue)
        assert bool(torch.isfinite(a).all())
        # the two entry points run the same kernels; their fp32 atomic additions may land in a different order
        assert orc.rel_l2(a.double().cpu().numpy(), b.double().cpu().numpy()) <= 1e-3
        assert orc.rel_l2(a.double().cpu().numpy(), want) <= 1e-3
        assert orc.rel_l2(b.double().cpu().numpy(), want) <= 1e-3


def test_static_scratch_entry_point_limits_and_fp32():
    lib = _lib.load()
    one = 1
    too_many = (32 << 20) // (64 * 4) + 1
    rc = lib.pce_conv_fwd_fod_static(16, 16, None, 16, _lib.PCE_F16, too_many, too_many, 64, 64, 27, 13, one, one, one, one, 128, None, None)
    assert rc == _lib.PCE_ECAPACITY and b"static" in lib.pce_last_error()
    with pytest.raises(OverflowError):
        _lib.check(rc)
    assert lib.pce_conv_fwd_fod_static(None, None, None, None, 0, 1, 1, 1, 1, 1, -1, None, None, None, None, 0, None, None) == _lib.PCE_EINVAL
    # fp32 accumulates in the output: no scratch, no size limit, same bits as the workspace entry point's rows
    coords = synth.random_cloud(seed=83, n=5000, extent=18, batches=2)
    km = gpu_map(coords, (3, 3, 3))
    ref = orc.kernel_map(coords, (3, 3, 3))
    f, w = synth.features(3, len(coords), 16), synth.weights(3, 27, 16, 16)
    fd, wd = torch.as_tensor(f, device=DEV).float(), torch.as_tensor(w, device=DEV).float()
    out = torch.empty((len(coords), 16), dtype=torch.float32, device=DEV)
    _lib.check(lib.pce_conv_fwd_fod_static(fd.data_ptr(), wd.data_ptr(), None, out.data_ptr(), _lib.PCE_F32, km.n_in, km.n_out, 16, 16, 27,
                                           13, km.imap.data_ptr(), km.omap.data_ptr(), km.kpos.data_ptr(), km.qkpos.data_ptr(), km.qsum,
                                           None, torch.cuda.current_stream().cuda_stream))
    want = orc.conv_forward(rounded(f, torch.float32), rounded(w, torch.float32), ref, (3, 3, 3))
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-5


def test_static_scratch_entry_point_under_graph_capture():
    """Two calls of the static entry point captured into one HIP graph (the second on a smaller layer, both sharing
    the array), after pce_conv_fod_static_init outside the capture: every replay, with eager work and
    synchronisations in between, equals the workspace entry point's result to the bar of the eager test."""
    lib = _lib.load()
    assert lib.pce_conv_fod_static_init() == _lib.PCE_OK
    dt = torch.float16
    layers = []
    for seed, coords, c_in, c_out in [(5, synth.random_cloud(seed=83, n=20000, extent=30, batches=2), 32, 64),
                                      (6, synth.random_cloud(seed=84, n=3000, extent=14), 64, 32)]:
        km = gpu_map(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0))
        fd = torch.as_tensor(synth.features(seed, km.n_in, c_in), device=DEV).to(dt)
        wd = torch.as_tensor(synth.weights(seed, km.kv, c_in, c_out), device=DEV).to(dt)
        out = torch.full((km.n_out, c_out), float("nan"), dtype=dt, device=DEV)
        ws_bytes = lib.pce_conv_fod_workspace_bytes(km.n_out, c_out, _lib.PCE_F16)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
        want = torch.empty_like(out)
        tail = (_lib.PCE_F16, km.n_in, km.n_out, c_in, c_out, km.kv, 13, km.imap.data_ptr(), km.omap.data_ptr(), km.kpos.data_ptr(),
                km.qkpos.data_ptr(), km.qsum)
        _lib.check(lib.pce_conv_fwd_fod(fd.data_ptr(), wd.data_ptr(), None, want.data_ptr(), *tail, ws.data_ptr(), ws_bytes, None,
                                        torch.cuda.current_stream().cuda_stream))
        layers.append((km, fd, wd, out, want, tail))
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        s = torch.cuda.current_stream().cuda_stream
        for km, fd, wd, out, want, tail in layers:
            _lib.check(lib.pce_conv_fwd_fod_static(fd.data_ptr(), wd.data_ptr(), None, out.data_ptr(), *tail, None, s))
    for _ in range(3):
        for km, fd, wd, out, want, tail in layers:
            out.fill_(float("nan"))
        (layers[0][1] * 2).sum().item()          # eager work and a synchronisation between replays
        g.replay()
        torch.cuda.synchronize()
        for km, fd, wd, out, want, tail in layers:
            assert bool(torch.isfinite(out).all())
            assert orc.rel_l2(out.double().cpu().numpy(), want.double().cpu().numpy()) <= 1e-3
