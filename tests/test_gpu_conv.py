"""Forward-value parity of the three HIP dataflows with the float64 oracle, through the C ABI.
Bars: rel-L2 <= 1e-3 for fp16 storage (fp32 accumulate), <= 1e-5 for fp32."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from pcengine_amd import backend, synth
from pcengine_amd.backend import DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS
from tests.util import DEV, TOL, gpu_map, rounded

pytestmark = pytest.mark.gpu

FLOWS = [DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS]
CHANNELS = [(16, 16), (64, 64), (4, 32), (32, 20), (96, 96), (5, 7), (64, 160), (130, 40)]


def _case(coords, ks, stride, pad, c_in, c_out, dtype, seed=0):
    kv = ks[0] * ks[1] * ks[2]
    f = synth.features(seed, len(coords), c_in)
    w = synth.weights(seed, kv, c_in, c_out)
    ref_map = orc.kernel_map(coords, ks, stride, pad)
    want = orc.conv_forward(rounded(f, dtype), rounded(w, dtype), ref_map, ks)
    fd = torch.as_tensor(f, device=DEV).to(dtype)
    wd = torch.as_tensor(w, device=DEV).to(dtype)
    return fd, wd, ref_map, want


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("c_in,c_out", CHANNELS)
def test_submanifold_all_dataflows(c_in, c_out, dtype):
    coords = synth.random_cloud(seed=41, n=9000, extent=22, batches=2)
    fd, wd, ref_map, want = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), c_in, c_out, dtype)
    km = gpu_map(coords, (3, 3, 3), want_csr=True, want_nbr_in=True)
    packed = backend.pack_weights(wd)
    assert (packed is None) == (dtype == torch.float32)
    for flow in FLOWS:
        for pk in (None, packed):
            out = backend.conv_forward(fd, wd, km, flow, packed=pk)
            err = orc.rel_l2(out.double().cpu().numpy(), want)
            assert err <= TOL[dtype], (flow, pk is not None, err)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("ks,stride,pad", [((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
                                           ((2, 3, 1), (2, 1, 1), (0, 1, 0))])
def test_strided_then_transposed_all_dataflows(ks, stride, pad, dtype):
    coords = synth.random_cloud(seed=42, n=7000, extent=20, batches=2)
    c_in, c_out = 64, 128
    fd, wd, ref_map, want = _case(coords, ks, stride, pad, c_in, c_out, dtype)
    km = gpu_map(coords, ks, stride, pad, want_csr=True, want_nbr_in=True)
    kv = km.kv
    wt = synth.weights(9, kv, c_out, c_in)
    wtd = torch.as_tensor(wt, device=DEV).to(dtype)
    pk, pkt = backend.pack_weights(wd), backend.pack_weights(wtd)
    for flow in FLOWS:
        out = backend.conv_forward(fd, wd, km, flow, packed=pk)
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= TOL[dtype], flow
        # transposed layer back onto the input coordinates, fed with the GPU's own output
        back = backend.conv_forward(out, wtd, km, flow, transposed=True, packed=pkt)
        want_t = orc.conv_forward(out.double().cpu().numpy(), rounded(wt, dtype), ref_map, ks, transposed=True)
        assert back.shape == (len(coords), c_in)
        assert orc.rel_l2(back.double().cpu().numpy(), want_t) <= TOL[dtype], flow


@pytest.mark.parametrize("c_in,c_out", [(128, 256), (256, 128), (96, 96), (384, 256), (40, 200)])
def test_wide_channels_dense_map(c_in, c_out):
    """Deep-layer shapes (dense map, wide channels): the pipelined output-stationary kernel and the others."""
    coords = synth.random_cloud(seed=43, n=5000, extent=14, batches=2)       # ~17 neighbours per voxel
    fd, wd, ref_map, want = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), c_in, c_out, torch.float16)
    km = gpu_map(coords, (3, 3, 3), want_csr=True)
    packed = backend.pack_weights(wd)
    for flow in FLOWS:
        out = backend.conv_forward(fd, wd, km, flow, packed=packed)
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3, flow
    # k2s2 down and transposed up at wide channels through the same kernels
    fd2, wd2, ref2, want2 = _case(coords, (2, 2, 2), (2, 2, 2), (0, 0, 0), c_in, c_out, torch.float16)
    km2 = gpu_map(coords, (2, 2, 2), (2, 2, 2), want_csr=True, want_nbr_in=True)
    out2 = backend.conv_forward(fd2, wd2, km2, DATAFLOW_OS, packed=backend.pack_weights(wd2))
    assert orc.rel_l2(out2.double().cpu().numpy(), want2) <= 1e-3
    wt = torch.as_tensor(synth.weights(5, 8, c_out, c_in), device=DEV).half()
    back = backend.conv_forward(out2, wt, km2, DATAFLOW_OS, transposed=True, packed=backend.pack_weights(wt))
    want_t = orc.conv_forward(out2.double().cpu().numpy(), wt.double().cpu().numpy(), ref2, (2, 2, 2), transposed=True)
    assert orc.rel_l2(back.double().cpu().numpy(), want_t) <= 1e-3


@pytest.mark.parametrize("c_in,c_out", [(16, 8), (32, 48), (48, 64), (64, 24), (64, 64), (16, 40)])
def test_narrow_fp16_layers_barrier_free_kernel(c_in, c_out):
    """fp16 rows of at most 64 channels with packed weights take the wavefront-per-chunk kernel in the
    deferred-scatter dataflow: submanifold (pairs + centre in one launch), strided and transposed."""
    from pcengine_amd import _lib
    coords = synth.random_cloud(seed=44, n=12000, extent=30, batches=2)
    fd, wd, ref_map, want = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), c_in, c_out, torch.float16, seed=6)
    km = gpu_map(coords, (3, 3, 3), want_csr=True)
    pk = backend.pack_weights(wd)
    out = backend.conv_forward(fd, wd, km, DATAFLOW_FDS, packed=pk)
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3
    with _lib.measurement_build() as mlib:            # the same layer through the workgroup-tile kernels
        mlib.pce_set_stage_mask(0xFFFFFFFF & ~16)
        old = backend.conv_forward(fd, wd, km, DATAFLOW_FDS, packed=pk)
    assert orc.rel_l2(old.double().cpu().numpy(), want) <= 1e-3
    # rows without neighbours are the centre GEMM alone and agree bit for bit
    lonely = (km.ocsr[1:] == km.ocsr[:-1])
    assert lonely.any() and torch.equal(out[lonely], old[lonely])
    for ks, stride, pad in [((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (1, 1, 1))]:
        fd2, wd2, ref2, want2 = _case(coords, ks, stride, pad, c_in, c_out, torch.float16, seed=7)
        km2 = gpu_map(coords, ks, stride, pad, want_csr=True)
        down = backend.conv_forward(fd2, wd2, km2, DATAFLOW_FDS, packed=backend.pack_weights(wd2))
        assert orc.rel_l2(down.double().cpu().numpy(), want2) <= 1e-3
        if c_out % 16 == 0:
            wt = torch.as_tensor(synth.weights(8, km2.kv, c_out, c_in), device=DEV).half()
            back = backend.conv_forward(down, wt, km2, DATAFLOW_FDS, transposed=True, packed=backend.pack_weights(wt))
            want_t = orc.conv_forward(down.double().cpu().numpy(), wt.double().cpu().numpy(), ref2, ks, transposed=True)
            assert orc.rel_l2(back.double().cpu().numpy(), want_t) <= 1e-3


def _act_np(x, act):
    if act is None:
        return x
    if act == "relu":
        return np.maximum(x, 0.0)
    return np.where(x > 0, x, x * act[1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("c_in,c_out", [(64, 64), (32, 20), (16, 48), (96, 160), (5, 7)])
def test_fused_epilogue_all_dataflows(c_in, c_out, dtype):
    """out = act(conv + bias + residual) inside the kernels, against the same formula in float64:
    every dataflow, packed and unpacked weights, submanifold / strided / transposed / 1x1."""
    coords = synth.random_cloud(seed=45, n=8000, extent=21, batches=2)
    rng = np.random.default_rng(45)
    bias = rng.standard_normal(c_out) * 0.5
    bd = torch.as_tensor(bias, device=DEV).to(dtype)
    fd, wd, ref_map, want = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), c_in, c_out, dtype, seed=3)
    res = rng.standard_normal((len(coords), c_out))
    rd = torch.as_tensor(res, device=DEV).to(dtype)
    km = gpu_map(coords, (3, 3, 3), want_csr=True, want_nbr_in=True)
    packed = backend.pack_weights(wd)
    combos = [(bd, rd, "relu"), (bd, None, None), (None, rd, ("leaky_relu", 0.1)), (None, None, "relu")]
    for flow in FLOWS:
        for pk in ((None, packed) if packed is not None else (None,)):
            for b, r, act in combos:
                out = backend.conv_forward(fd, wd, km, flow, packed=pk, bias=b, residual=r, act=act)
                ref = want + (rounded(bias, dtype) if b is not None else 0) + (rounded(res, dtype) if r is not None else 0)
                ref = _act_np(ref, act)
                err = orc.rel_l2(out.double().cpu().numpy(), ref)
                assert err <= TOL[dtype], (flow, pk is not None, act, err)
                if act == "relu":
                    assert (out >= 0).all()
    # strided down, transposed up, 1x1
    fd2, wd2, ref2, want2 = _case(coords, (2, 2, 2), (2, 2, 2), (0, 0, 0), c_in, c_out, dtype, seed=4)
    km2 = gpu_map(coords, (2, 2, 2), (2, 2, 2), want_csr=True, want_nbr_in=True)
    res2 = rng.standard_normal((km2.n_out, c_out))
    r2 = torch.as_tensor(res2, device=DEV).to(dtype)
    wt = synth.weights(10, 8, c_out, c_in)
    wtd = torch.as_tensor(wt, device=DEV).to(dtype)
    bt = rng.standard_normal(c_in) * 0.5
    btd = torch.as_tensor(bt, device=DEV).to(dtype)
    for flow in FLOWS:
        down = backend.conv_forward(fd2, wd2, km2, flow, packed=backend.pack_weights(wd2), bias=bd, residual=r2, act="relu")
        ref = np.maximum(want2 + rounded(bias, dtype) + rounded(res2, dtype), 0.0)
        assert orc.rel_l2(down.double().cpu().numpy(), ref) <= TOL[dtype], flow
        up = backend.conv_forward(down, wtd, km2, flow, transposed=True, packed=backend.pack_weights(wtd), bias=btd,
                                  residual=fd, act=("leaky_relu", 0.2))
        ref_t = orc.conv_forward(down.double().cpu().numpy(), rounded(wt, dtype), ref2, (2, 2, 2), transposed=True)
        ref_t = _act_np(ref_t + rounded(bt, dtype) + fd.double().cpu().numpy(), ("leaky_relu", 0.2))
        assert orc.rel_l2(up.double().cpu().numpy(), ref_t) <= TOL[dtype], flow
    w1 = wd[0].contiguous()
    one = backend.dense_forward(fd, w1, backend.pack_weights(w1), bias=bd, residual=rd, act="relu")
    ref1 = np.maximum(fd.double().cpu().numpy() @ w1.double().cpu().numpy() + rounded(bias, dtype) + rounded(res, dtype), 0.0)
    assert orc.rel_l2(one.double().cpu().numpy(), ref1) <= TOL[dtype]


def test_fused_epilogue_argument_errors():
    coords = synth.random_cloud(seed=46, n=500, extent=9)
    fd, wd, _, _ = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), 16, 16, torch.float16)
    km = gpu_map(coords, (3, 3, 3))
    with pytest.raises(ValueError):
        backend.conv_forward(fd, wd, km, DATAFLOW_OS, bias=torch.zeros(3, device=DEV))
    with pytest.raises(ValueError):
        backend.conv_forward(fd, wd, km, DATAFLOW_OS, residual=torch.zeros((2, 16), dtype=torch.float16, device=DEV))
    with pytest.raises(ValueError):
        backend.conv_forward(fd, wd, km, DATAFLOW_OS, act="gelu")
    out = torch.empty((len(coords), 16), dtype=torch.float16, device=DEV)
    with pytest.raises(ValueError):      # the residual may not be the output tensor
        backend.conv_forward(fd, wd, km, DATAFLOW_OS, out=out, residual=out)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_dense_1x1(dtype):
    f = synth.features(3, 5001, 96)
    w = synth.weights(3, 1, 96, 20)[0]
    fd, wd = torch.as_tensor(f, device=DEV).to(dtype), torch.as_tensor(w, device=DEV).to(dtype)
    want = rounded(f, dtype) @ rounded(w, dtype)
    for pk in (None, backend.pack_weights(wd)):
        out = backend.dense_forward(fd, wd, pk)
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= TOL[dtype]


@pytest.mark.parametrize("c_in,c_out", [(192, 192), (256, 192), (192, 168)])
def test_dense_wide_many_rows(c_in, c_out):
    """Plain GEMMs of wide fp16 layers on many rows (the centre terms and 1x1 shortcuts of a network's widest levels):
    a row count that is no multiple of the tile height, with and without the epilogue, against float64 on sampled rows
    and bit for bit against the same rows computed in a short matrix."""
    n = 131072 + 4097
    rng = np.random.default_rng(c_in + c_out)
    f = (rng.standard_normal((n, c_in)) * 0.5).astype(np.float32)
    w = (rng.standard_normal((c_in, c_out)) * 0.05).astype(np.float32)
    bias, res = rng.standard_normal(c_out) * 0.3, rng.standard_normal((n, c_out)).astype(np.float32)
    dt = torch.float16
    fd, wd = torch.as_tensor(f, device=DEV).to(dt), torch.as_tensor(w, device=DEV).to(dt)
    bd, rd = torch.as_tensor(bias, device=DEV).to(dt), torch.as_tensor(res, device=DEV).to(dt)
    pk = backend.pack_weights(wd)
    rows = np.concatenate([np.arange(0, 70), rng.integers(0, n, 400), np.arange(n - 70, n)])
    plain = backend.dense_forward(fd, wd, pk)
    want = rounded(f[rows], dt) @ rounded(w, dt)
    assert orc.rel_l2(plain[rows].double().cpu().numpy(), want) <= 1e-3
    fused = backend.dense_forward(fd, wd, pk, bias=bd, residual=rd, act="relu")
    want = np.maximum(want + rounded(bias, dt) + rounded(res[rows], dt), 0)
    assert orc.rel_l2(fused[rows].double().cpu().numpy(), want) <= 1e-3
    assert bool(torch.isfinite(fused).all())
    head = slice(0, 5000)
    assert torch.equal(backend.dense_forward(fd[head].contiguous(), wd, pk, bias=bd, residual=rd[head].contiguous(), act="relu"), fused[head])


def test_config1_fp32_c16():
    coords = synth.sphere_plane_cloud()
    fd, wd, ref_map, want = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), 16, 16, torch.float32, seed=1)
    km = gpu_map(coords, (3, 3, 3), want_csr=True)
    for flow in FLOWS:
        out = backend.conv_forward(fd, wd, km, flow)
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-5, flow
    # the selector's choice for this layer: the ordered dataflow in its fp32 form
    assert backend.select_dataflow(km, 16, 16, torch.float32) == backend.DATAFLOW_OSO
    out = backend.conv_forward(fd, wd, km, backend.DATAFLOW_OSO)
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-5


def test_config2_fp16_c64_full_size():
    coords = synth.lidar_cloud()
    fd, wd, ref_map, want = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), 64, 64, torch.float16, seed=2)
    km = gpu_map(coords, (3, 3, 3), want_csr=True)
    # the selector's pick for this layer (the ordered output-stationary form) is the kernel the benchmark
    # times; it is checked here at the benchmark's size together with the four other dataflows
    picked = backend.select_dataflow(km, 64, 64, torch.float16)
    assert picked == backend.DATAFLOW_OSO
    flows = FLOWS + [backend.DATAFLOW_OSO]
    outs = [backend.conv_forward(fd, wd, km, flow) for flow in flows]
    for flow, out in zip(flows, outs):
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3, flow
    # linearity in the features holds at any size: conv(2x) == 2 conv(x); scaling by two is exact in
    # fp16 except for results in the subnormal range, whose spacing is 2^-24
    # (both runs take the same launch sequence: packed weights select the two-launch form, whose rows
    # with neighbours are rounded twice)
    packed = backend.pack_weights(wd)
    once = backend.conv_forward(fd, wd, km, DATAFLOW_FDS, packed=packed)
    twice = backend.conv_forward(fd * 2, wd, km, DATAFLOW_FDS, packed=packed)
    assert orc.rel_l2(once.double().cpu().numpy(), want) <= 1e-3
    assert torch.allclose(twice.float(), once.float() * 2, rtol=0, atol=2.0 ** -23)


def test_reference_named_entry_points_d2_and_d1():
    """Drive the five pybind names the way the reference front end does (script/spconv.py:343-431)."""
    coords = synth.random_cloud(seed=44, n=6000, extent=18)
    n = len(coords)
    kv, ci, co = 27, 32, 48
    enc = lambda v: 94273 * v[0] + 311 * v[1] + v[2]
    c = torch.as_tensor(coords, device=DEV)
    f = synth.features(4, n, ci)
    w = synth.weights(4, kv, ci, co)
    fd = torch.as_tensor(f, device=DEV).half()
    wd = torch.as_tensor(w, device=DEV).half()
    ref_map = orc.kernel_map(coords, (3, 3, 3))
    want = orc.conv_forward(rounded(f, torch.float16), rounded(w, torch.float16), ref_map, (3, 3, 3))
    cmax = coords[:, 1:].max(0).tolist()
    # fetch-on-demand protocol
    imap = -torch.ones(kv * n, dtype=torch.int, device=DEV)
    knnz = torch.zeros(kv, dtype=torch.int, device=DEV)
    kpos = torch.zeros(kv + 1, dtype=torch.int, device=DEV)
    qkpos = torch.zeros(kv + 1, dtype=torch.int, device=DEV)
    oc = backend.mapping_d2_cuda(c, 1, enc([3, 3, 3]), kv, ci, co, enc([1, 1, 1]), enc([1, 1, 1]), enc([0, 0, 0]),
                                 0, 0, 0, *cmax, imap, knnz, kpos, qkpos, True)
    assert oc is c
    nz = torch.nonzero(imap != -1)
    omap = imap[nz]
    imap2 = (nz % n).int()
    assert np.array_equal(imap2.flatten().cpu().numpy(), ref_map.imap) and np.array_equal(omap.flatten().cpu().numpy(), ref_map.omap)
    qsum = int(qkpos[-1].cpu())
    out = torch.zeros((n, co), dtype=torch.half, device=DEV)
    backend.conv_fwd_d2_cuda(fd, wd, enc([3, 3, 3]), qsum, out, kpos, qkpos, imap2.contiguous(), omap.contiguous(), True, False)
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3
    # gather-GEMM-scatter protocol, with the reference's allocation sizes (kpos has kv entries)
    imap = -torch.ones(n * kv, dtype=torch.int, device=DEV)
    omap = -torch.ones(n * kv * 8, dtype=torch.int, device=DEV)
    knnz = torch.zeros(kv, dtype=torch.int, device=DEV)
    kpos = torch.zeros(kv, dtype=torch.int, device=DEV)
    qkpos = torch.zeros(kv + 1, dtype=torch.int, device=DEV)
    icsr = torch.zeros(n + 2, dtype=torch.int, device=DEV)
    ocsr = torch.zeros((n + 2) * 8, dtype=torch.int, device=DEV)
    backend.mapping_d1_cuda(c, enc([3, 3, 3]), kv, ci, co, enc([1, 1, 1]), enc([1, 1, 1]), enc([0, 0, 0]), 0, 0, 0, *cmax,
                            imap, omap, icsr, ocsr, knnz, kpos, qkpos, True)
    qsum = int(qkpos[-1].cpu())
    buffer = torch.empty(qsum * (ci + co), dtype=torch.half, device=DEV)
    out = torch.zeros((n, co), dtype=torch.half, device=DEV)
    backend.conv_fwd_d1_cuda(fd, wd, enc([3, 3, 3]), qsum, out, kpos, qkpos, imap, omap, icsr, ocsr, buffer, True, 1)
    assert orc.rel_l2(out.double().cpu().numpy(), want) <= 1e-3
    with pytest.raises(ValueError):     # backend/spconv.cu:38-40
        backend.conv_fwd_d2_cuda(fd[:, :16].contiguous(), wd, enc([3, 3, 3]), qsum, out, kpos, qkpos, imap, omap, True, False)
    # backward with the reference's protocol (script/spconv.py:182-198): fp32, caller-allocated gradients
    f32, w32 = fd.float(), wd.float()
    g = np.random.default_rng(4).standard_normal((n, co))
    gd = torch.as_tensor(g, device=DEV).float()
    in_grad = torch.zeros((n, ci), dtype=torch.float, device=DEV)
    w_grad = torch.zeros((kv, ci, co), dtype=torch.float, device=DEV)
    backend.conv_bwd_d1_cuda(gd, f32, w32, enc([3, 3, 3]), qsum, in_grad, w_grad, knnz, kpos, imap, omap, icsr, ocsr, buffer, 1)
    gf, gw = orc.conv_backward(f32.double().cpu().numpy(), w32.double().cpu().numpy(), ref_map, (3, 3, 3), rounded(g, torch.float32))
    assert orc.rel_l2(in_grad.double().cpu().numpy(), gf) <= 1e-5 and orc.rel_l2(w_grad.double().cpu().numpy(), gw) <= 1e-5


def test_deferred_scatter_without_buffer_needs_one_pair_per_row():
    """pce_conv_fwd_fds takes no partial-row buffer only for a layer without centre offset whose pair count
    equals its output rows (a transposed layer with kernel == stride); anything else is an argument error."""
    from pcengine_amd import _lib
    lib = _lib.load()
    coords = synth.random_cloud(seed=47, n=3000, extent=12)
    fd, wd, _, _ = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), 32, 32, torch.float16)
    km = gpu_map(coords, (3, 3, 3), want_csr=True)
    out = torch.empty((km.n_out, 32), dtype=torch.float16, device=DEV)

    def call(mid, n_pairs):
        return lib.pce_conv_fwd_fds(fd.data_ptr(), wd.data_ptr(), None, out.data_ptr(), _lib.PCE_F16, km.n_in, km.n_out, 32, 32,
                                    km.kv, mid, km.imap.data_ptr(), km.omap.data_ptr(), km.oslot.data_ptr(), km.kpos.data_ptr(),
                                    km.qkpos.data_ptr(), None, None, km.ocsr.data_ptr(), None, n_pairs, km.qsum, None, 0, None, None)
    assert call(13, km.M) == _lib.PCE_EINVAL          # centre offset present
    assert call(-1, km.M) == _lib.PCE_EINVAL          # pairs != output rows
    # the transposed 2x2x2 stride-2 layer qualifies: same result with and without the caller's buffer
    km2 = gpu_map(coords, (2, 2, 2), (2, 2, 2), want_csr=True)
    assert km2.M == km2.n_in
    down = torch.as_tensor(synth.features(5, km2.n_out, 48), device=DEV).half()
    wt = torch.as_tensor(synth.weights(5, 8, 48, 32), device=DEV).half()
    direct = backend.conv_forward(down, wt, km2, DATAFLOW_FDS, transposed=True, packed=backend.pack_weights(wt))
    buf = torch.empty(km2.M * 32, dtype=torch.float16, device=DEV)
    back = torch.empty((km2.n_in, 32), dtype=torch.float16, device=DEV)
    rc = lib.pce_conv_fwd_fds(down.data_ptr(), wt.data_ptr(), backend.pack_weights(wt).data_ptr(), back.data_ptr(), _lib.PCE_F16,
                              km2.n_out, km2.n_in, 48, 32, 8, -1, km2.omap.data_ptr(), km2.imap.data_ptr(), km2.islot.data_ptr(),
                              km2.kpos.data_ptr(), km2.qkpos.data_ptr(), None, None, km2.icsr.data_ptr(), None, km2.M, km2.qsum,
                              buf.data_ptr(), buf.numel(), None, None)
    assert rc == _lib.PCE_OK
    torch.cuda.synchronize()
    assert torch.equal(direct, back)


@pytest.mark.parametrize("cloud", ["surface", "random"])
@pytest.mark.parametrize("c_in,c_out", [(64, 128), (128, 256), (96, 104), (64, 64)])
def test_strided_layer_routes_single_pair_rows(cloud, c_in, c_out):
    """A k2s2 layer in the deferred-scatter dataflow: the only pair of an output row stores the finished row,
    the other rows go through partial rows and the row sum.  Without an epilogue the result equals the unrouted
    one bit for bit (a single partial row is rounded to fp16 once either way); with one, both meet the fp16 bar.
    (64, 64) is a shape the routed kernel does not take: the routing array is ignored."""
    from pcengine_amd import _lib
    lib = _lib.load()
    if cloud == "surface":
        coords = synth.sphere_plane_cloud(seed=7, n_sphere=9000, n_plane=3000)       # nearly every coarse voxel has one child
    else:
        coords = synth.random_cloud(seed=48, n=9000, extent=20, batches=2)
    ks = (2, 2, 2)
    fd, wd, ref_map, want = _case(coords, ks, ks, (0, 0, 0), c_in, c_out, torch.float16, seed=6)
    km = gpu_map(coords, ks, ks, want_csr=True)
    pk = backend.pack_weights(wd)
    # the routing array against its definition
    route = backend.pair_route(km).cpu().numpy()
    assert len(route) == lib.pce_pair_route_elems(km.M, km.n_out) == 4 + km.M + km.n_out
    ocsr, omap, oslot = km.ocsr.cpu().numpy(), km.omap.cpu().numpy()[:km.M], km.oslot.cpu().numpy()[:km.M]
    cnt = np.diff(ocsr)
    assert np.array_equal(route[4:4 + km.M], np.where(cnt[omap] == 1, omap, km.n_out + oslot))
    others = np.flatnonzero(cnt != 1)
    assert route[0] == len(others) and not route[1:4].any()
    assert np.array_equal(np.sort(route[4 + km.M:4 + km.M + route[0]]), others)
    singles = int((cnt == 1).sum())
    assert 0 < singles < km.n_out or cloud == "surface"
    plain = backend.conv_forward(fd, wd, km, DATAFLOW_FDS, packed=pk, route_single_pairs=False)
    routed = backend.conv_forward(fd, wd, km, DATAFLOW_FDS, packed=pk)
    assert torch.equal(plain, routed)
    assert orc.rel_l2(routed.double().cpu().numpy(), want) <= 1e-3
    # a second call on the cached routing, into a poisoned output and buffer
    out = torch.full((km.n_out, c_out), float("nan"), dtype=torch.float16, device=DEV)
    buf = torch.full((km.M * c_out,), float("nan"), dtype=torch.float16, device=DEV)
    again = backend.conv_forward(fd, wd, km, DATAFLOW_FDS, packed=pk, out=out, buffer=buf)
    assert torch.equal(again, routed)
    rng = np.random.default_rng(48)
    bias, res = rng.standard_normal(c_out) * 0.5, rng.standard_normal((km.n_out, c_out))
    bd, rd = torch.as_tensor(bias, device=DEV).half(), torch.as_tensor(res, device=DEV).half()
    for b, r, act in [(bd, rd, "relu"), (bd, None, None), (None, rd, ("leaky_relu", 0.1)), (None, None, "relu")]:
        got = backend.conv_forward(fd, wd, km, DATAFLOW_FDS, packed=pk, bias=b, residual=r, act=act)
        ref = want + (rounded(bias, torch.float16) if b is not None else 0) + (rounded(res, torch.float16) if r is not None else 0)
        ref = _act_np(ref, act)
        assert orc.rel_l2(got.double().cpu().numpy(), ref) <= 1e-3, act
    # argument checks of the routing entry point
    one = km.ocsr.data_ptr()
    assert lib.pce_pair_route(None, None, None, 5, 5, None, 100, None) == _lib.PCE_EINVAL
    assert lib.pce_pair_route(one, one, one, 1 << 30, 1 << 30, one, 1 << 40, None) == _lib.PCE_ECAPACITY
    assert lib.pce_pair_route(one, one, one, 5, 5, one, 13, None) == _lib.PCE_EWORKSPACE


@pytest.mark.parametrize("c_in,c_out", [(128, 96), (256, 128)])
def test_transposed_layer_with_clipped_parents_is_routed(c_in, c_out):
    """A transposed k2s2 layer over a map whose coarse bound clipped some parents away: the fine voxels without a
    parent have no pair (their rows are act(bias + residual)), every other row has exactly one, stored by the pair
    tiles; only the rows without a pair are left to the row sum."""
    coords = synth.random_cloud(seed=49, n=9000, extent=21, batches=2)     # coordinates 0..20: x = 20 has no parent
    ks = (2, 2, 2)
    ref_map = orc.kernel_map(coords, ks, ks, (0, 0, 0))
    km = gpu_map(coords, ks, ks, want_csr=True)
    assert 0 < km.M < km.n_in
    route = backend.pair_route(km, transposed=True).cpu().numpy()
    cnt = np.diff(km.icsr.cpu().numpy())
    assert set(np.unique(cnt)) == {0, 1}
    assert route[0] == (cnt == 0).sum()
    assert np.array_equal(np.sort(route[4 + km.M:4 + km.M + route[0]]), np.flatnonzero(cnt == 0))
    assert np.array_equal(route[4:4 + km.M], km.imap.cpu().numpy()[:km.M])
    coarse = synth.features(8, km.n_out, c_in)
    wt = synth.weights(8, 8, c_in, c_out)
    cd, wd = torch.as_tensor(coarse, device=DEV).half(), torch.as_tensor(wt, device=DEV).half()
    pk = backend.pack_weights(wd)
    want = orc.conv_forward(rounded(coarse, torch.float16), rounded(wt, torch.float16), ref_map, ks, transposed=True)
    plain = backend.conv_forward(cd, wd, km, DATAFLOW_FDS, transposed=True, packed=pk, route_single_pairs=False)
    out = torch.full((km.n_in, c_out), float("nan"), dtype=torch.float16, device=DEV)
    routed = backend.conv_forward(cd, wd, km, DATAFLOW_FDS, transposed=True, packed=pk, out=out)
    assert torch.equal(plain, routed)
    assert (routed[torch.as_tensor(cnt == 0, device=DEV)] == 0).all()
    assert orc.rel_l2(routed.double().cpu().numpy(), want) <= 1e-3
    rng = np.random.default_rng(49)
    bias, res = rng.standard_normal(c_out) * 0.5, rng.standard_normal((km.n_in, c_out))
    bd, rd = torch.as_tensor(bias, device=DEV).half(), torch.as_tensor(res, device=DEV).half()
    for b, r, act in [(bd, rd, "relu"), (bd, None, ("leaky_relu", 0.1)), (None, rd, None)]:
        got = backend.conv_forward(cd, wd, km, DATAFLOW_FDS, transposed=True, packed=pk, bias=b, residual=r, act=act)
        ref = want + (rounded(bias, torch.float16) if b is not None else 0) + (rounded(res, torch.float16) if r is not None else 0)
        assert orc.rel_l2(got.double().cpu().numpy(), _act_np(ref, act)) <= 1e-3, act


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("ks,c_in,c_out", [((5, 5, 5), 32, 32), ((5, 5, 5), 64, 128), ((5, 3, 1), 16, 24), ((1, 5, 5), 128, 96),
                                           ((2, 2, 2), 32, 32), ((2, 3, 3), 64, 128), ((2, 2, 2), 128, 128)])
def test_large_and_anisotropic_kernels_forward_and_backward(ks, c_in, c_out, dtype):
    """Kernel volumes beyond what travels in the kernel arguments (5x5x5 = 125 offsets), anisotropic kernels and
    stride-1 layers with even kernel sizes (whose maps have no mirror symmetry: the feature gradient runs the
    transposed layer over the swapped map), every dataflow, forward and both gradients, against the oracle
    (whose offsets follow the reference's rule, backend/hash.cuh:147-149)."""
    coords = synth.random_cloud(seed=48, n=4000, extent=15, batches=2)
    fd, wd, ref_map, want = _case(coords, ks, (1, 1, 1), (0, 0, 0), c_in, c_out, dtype, seed=11)
    km = gpu_map(coords, ks, want_csr=True, want_nbr_in=True)
    assert km.M == ref_map.M and torch.equal(km.imap.cpu(), torch.as_tensor(ref_map.imap)) and torch.equal(km.omap.cpu(), torch.as_tensor(ref_map.omap))
    packed = backend.pack_weights(wd)
    for flow in FLOWS:
        out = backend.conv_forward(fd, wd, km, flow, packed=packed)
        assert orc.rel_l2(out.double().cpu().numpy(), want) <= TOL[dtype], (ks, flow)
    rng = np.random.default_rng(48)
    g = rounded(rng.standard_normal((len(coords), c_out)), dtype)
    gd = torch.as_tensor(g, device=DEV).to(dtype)
    gf, gw = backend.conv_backward(fd, wd, km, gd)
    want_f, want_w = orc.conv_backward(fd.double().cpu().numpy(), wd.double().cpu().numpy(), ref_map, ks, g)
    assert orc.rel_l2(gf.double().cpu().numpy(), want_f) <= TOL[dtype]
    assert orc.rel_l2(gw.double().cpu().numpy(), want_w) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("c_in,c_out", [(32, 32), (128, 128), (5, 7)])
def test_layer_without_pairs_and_single_voxel(c_in, c_out, dtype):
    """Isolated voxels (no neighbour within the kernel) leave only the centre term; a cloud of one voxel is the
    smallest tensor there is.  Forward through every dataflow and both gradients."""
    grid = np.stack(np.meshgrid(np.arange(0, 40, 3), np.arange(0, 40, 3), np.arange(0, 12, 3), indexing="ij"), -1).reshape(-1, 3)
    for coords in (np.concatenate([np.zeros((len(grid), 1), np.int64), grid], 1).astype(np.int32),
                   np.array([[0, 5, 6, 7]], np.int32)):
        fd, wd, ref_map, want = _case(coords, (3, 3, 3), (1, 1, 1), (0, 0, 0), c_in, c_out, dtype, seed=12)
        km = gpu_map(coords, (3, 3, 3), want_csr=True, want_nbr_in=True)
        assert km.M == 0 and ref_map.M == 0
        packed = backend.pack_weights(wd)
        for flow in FLOWS:
            out = backend.conv_forward(fd, wd, km, flow, packed=packed)
            assert orc.rel_l2(out.double().cpu().numpy(), want) <= TOL[dtype], flow
        g = rounded(np.random.default_rng(3).standard_normal((len(coords), c_out)), dtype)
        gf, gw = backend.conv_backward(fd, wd, km, torch.as_tensor(g, device=DEV).to(dtype))
        want_f, want_w = orc.conv_backward(fd.double().cpu().numpy(), wd.double().cpu().numpy(), ref_map, (3, 3, 3), g)
        assert orc.rel_l2(gf.double().cpu().numpy(), want_f) <= TOL[dtype]
        assert orc.rel_l2(gw.double().cpu().numpy(), want_w) <= TOL[dtype]
