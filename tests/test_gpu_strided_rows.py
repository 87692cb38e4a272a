"""Feature matrices that are column slices of wider matrices (the halves of a concatenated skip connection):
read and written in place by the deferred-scatter and output-stationary kernels, bit-identical to the dense run;
copied by the front end for the other dataflows; refused by the C entry points that take dense rows only."""
import numpy as np
import pytest
import torch

import pcengine_amd as pe
from oracle import oracle as orc
from pcengine_amd import _lib, backend, nets, synth
from pcengine_amd.backend import DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS
from tests.util import DEV, dev_coords

pytestmark = pytest.mark.gpu

K3, K2, S1, S2, P0 = (3, 3, 3), (2, 2, 2), (1, 1, 1), (2, 2, 2), (0, 0, 0)


def _slices(n_in, c_in, n_out, c_out, dtype, left_in, left_out, seed):
    """Input rows sitting in columns [left_in, left_in + c_in) of a wider matrix, an output slice likewise; the
    columns around both hold sentinels that must survive."""
    wide_in = torch.full((n_in, left_in + c_in + 8), 7.0, dtype=dtype, device=DEV)
    f = torch.as_tensor(synth.features(seed, n_in, c_in), device=DEV).to(dtype)
    wide_in[:, left_in:left_in + c_in] = f
    wide_out = torch.full((n_out, left_out + c_out + 16), -3.0, dtype=dtype, device=DEV)
    return f, wide_in, wide_in[:, left_in:left_in + c_in], wide_out, wide_out[:, left_out:left_out + c_out]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("c_in,c_out", [(32, 32), (64, 64), (96, 96), (128, 128), (256, 256), (64, 128), (128, 96), (16, 24)])
def test_submanifold_layers_on_column_slices(c_in, c_out, dtype):
    coords = synth.random_cloud(seed=81, n=7000, extent=20, batches=2)
    km = backend.build_kernel_map(dev_coords(coords), K3, S1, P0, [0, 0, 0], coords[:, 1:].max(0).tolist(), True,
                                  want_csr=True, batchsize=2)
    n = len(coords)
    f, wide_in, f_view, wide_out, o_view = _slices(n, c_in, n, c_out, dtype, 40, 64, c_in + c_out)
    w = torch.as_tensor(synth.weights(1, 27, c_in, c_out), device=DEV).to(dtype)
    packed = backend.pack_weights(w)
    bias = torch.as_tensor(np.random.default_rng(1).standard_normal(c_out) * 0.1, device=DEV).to(dtype)
    res = torch.as_tensor(synth.features(9, n, c_out), device=DEV).to(dtype)
    for flow in (DATAFLOW_FDS, DATAFLOW_OS, DATAFLOW_GMS, DATAFLOW_FOD):
        for kw in (dict(), dict(bias=bias, residual=res, act="relu")):
            want = backend.conv_forward(f, w, km, flow, packed=packed, **kw)
            wide_out.fill_(-3.0)
            got = backend.conv_forward(f_view, w, km, flow, packed=packed, out=o_view, **kw)
            assert got.data_ptr() == o_view.data_ptr()
            if flow == DATAFLOW_FOD:      # atomic accumulation: the order of the additions differs run to run
                tol = 2e-3 if dtype == torch.float16 else 1e-5
                assert torch.allclose(o_view.float(), want.float(), rtol=tol, atol=tol)
            else:
                assert torch.equal(o_view, want), (flow, kw.keys())
            assert bool((wide_out[:, :64] == -3.0).all()) and bool((wide_out[:, 64 + c_out:] == -3.0).all())
            assert bool((wide_in[:, :40] == 7.0).all()) and bool((wide_in[:, 40 + c_in:] == 7.0).all())


@pytest.mark.parametrize("cloud", ["surface", "random"])
@pytest.mark.parametrize("c_in,c_out", [(32, 32), (64, 64), (128, 128), (64, 128), (256, 128)])
def test_strided_and_transposed_layers_on_column_slices(c_in, c_out, cloud):
    """The k2s2 layer that reads a kept encoder output, and the transposed layer that writes the left half of the
    concatenated matrix (routed pair tiles, single-pair rows, output-stationary)."""
    dtype = torch.float16
    coords = synth.sphere_plane_cloud() if cloud == "surface" else synth.random_cloud(seed=82, n=9000, extent=26)
    cmax = coords[:, 1:].max(0).tolist()
    km = backend.build_kernel_map(dev_coords(coords), K2, S2, P0, [0, 0, 0], backend.strided_coords_max(cmax, K2, S2, P0), False,
                                  want_csr=True, want_nbr_in=True, batchsize=1)
    w_dn = torch.as_tensor(synth.weights(2, 8, c_in, c_out), device=DEV).to(dtype)
    w_up = torch.as_tensor(synth.weights(3, 8, c_out, c_in), device=DEV).to(dtype)
    bias_dn = torch.as_tensor(np.random.default_rng(2).standard_normal(c_out) * 0.1, device=DEV).to(dtype)
    bias_up = torch.as_tensor(np.random.default_rng(3).standard_normal(c_in) * 0.1, device=DEV).to(dtype)
    f, _, f_view, wide_mid, mid_view = _slices(km.n_in, c_in, km.n_out, c_out, dtype, 24, 32, 5)
    _, _, _, wide_back, back_view = _slices(km.n_out, c_out, km.n_in, c_in, dtype, 0, 0, 6)
    for flow in (DATAFLOW_FDS, DATAFLOW_OS):
        want_dn = backend.conv_forward(f, w_dn, km, flow, packed=backend.pack_weights(w_dn), bias=bias_dn, act="relu")
        wide_mid.fill_(-3.0)
        got_dn = backend.conv_forward(f_view, w_dn, km, flow, packed=backend.pack_weights(w_dn), out=mid_view, bias=bias_dn, act="relu")
        assert torch.equal(got_dn, want_dn)
        assert bool((wide_mid[:, :32] == -3.0).all()) and bool((wide_mid[:, 32 + c_out:] == -3.0).all())
        # back up: reads the slice just written, writes columns [0, c_in) of a wider matrix
        want_up = backend.conv_forward(want_dn, w_up, km, flow, transposed=True, packed=backend.pack_weights(w_up), bias=bias_up, act="relu")
        wide_back.fill_(-3.0)
        got_up = backend.conv_forward(mid_view, w_up, km, flow, transposed=True, packed=backend.pack_weights(w_up), out=back_view,
                                      bias=bias_up, act="relu")
        assert torch.equal(got_up, want_up)
        assert bool((wide_back[:, c_in:] == -3.0).all())


def test_network_concatenates_in_place(monkeypatch):
    """The U-Net's inference forward writes both halves of every skip concatenation in place: no concatenation
    kernel runs, and the output equals, bit for bit, the forward that concatenates with a copy."""
    coords = synth.lidar_cloud_100k()
    f = torch.as_tensor(synth.features(4, len(coords), 4), device=DEV).half()
    cd = dev_coords(coords)
    cmax = coords[:, 1:].max(0).tolist()
    torch.manual_seed(4)
    model = nets.SparseResUNet(4, 20).to(DEV).eval().fuse_bn().half()
    calls = []
    real = backend.concat_cols
    monkeypatch.setattr(backend, "concat_cols", lambda *a, **k: calls.append(1) or real(*a, **k))
    with torch.no_grad():
        y = model(pe.spTensor(f, cd, None, [0, 0, 0], cmax))
    assert calls == []
    monkeypatch.setattr(nets.SparseResUNet, "_skips_in_place", lambda self, x: False)
    with torch.no_grad():
        z = model(pe.spTensor(f, cd, None, [0, 0, 0], cmax))
    assert len(calls) == 4 and torch.equal(y.feats, z.feats)
    # with norms not folded (training form) the network keeps the concatenating forward
    monkeypatch.undo()
    plain = nets.SparseResUNet(4, 20).to(DEV).eval()
    small = synth.random_cloud(seed=83, n=3000, extent=24)
    x = pe.spTensor(torch.as_tensor(synth.features(4, len(small), 4), device=DEV).float(), dev_coords(small), None, [0, 0, 0],
                    small[:, 1:].max(0).tolist())
    assert not plain._skips_in_place(x)


def test_frozen_network_with_input_gradients_keeps_the_copying_forward():
    """Frozen parameters, grad enabled, input features that require grad (an input-saliency pass over a fused model):
    autograd results are fresh tensors, so nothing may be written in place -- the network takes the concatenating
    forward, returns what the plain forward returns and carries the gradient to the input; a layer asked to write
    ``out=`` on that path refuses."""
    coords = synth.random_cloud(seed=85, n=4000, extent=26)
    cd = dev_coords(coords)
    cmax = coords[:, 1:].max(0).tolist()
    torch.manual_seed(6)
    model = nets.SparseResUNet(4, 20, stem=16, enc=(16, 32, 48, 64), dec=(64, 48, 24, 24)).to(DEV).eval().fuse_bn()
    for p in model.parameters():
        p.requires_grad_(False)
    f = torch.as_tensor(synth.features(4, len(coords), 4), device=DEV).float()
    with torch.no_grad():
        x0 = pe.spTensor(f, cd, None, [0, 0, 0], cmax)
        assert model._skips_in_place(x0)
        want = model(x0).feats
    fg = f.clone().requires_grad_(True)
    x = pe.spTensor(fg, cd, None, [0, 0, 0], cmax)
    assert not model._skips_in_place(x)
    y = model(x).feats
    assert orc.rel_l2(y.detach().double().cpu().numpy(), want.double().cpu().numpy()) <= 1e-5
    y.square().sum().backward()
    assert fg.grad is not None and bool(torch.isfinite(fg.grad).all()) and float(fg.grad.abs().max()) > 0
    layer = pe.conv3d(4, 16, 3).to(DEV)
    for p in layer.parameters():
        p.requires_grad_(False)
    with pytest.raises(ValueError, match="out="):
        layer(pe.spTensor(fg, cd, None, [0, 0, 0], cmax), out=torch.empty((len(coords), 16), device=DEV))


def test_row_strides_are_refused_where_rows_must_be_dense():
    lib = _lib.load()
    coords = synth.random_cloud(seed=84, n=2000, extent=14)
    km = backend.build_kernel_map(dev_coords(coords), K3, S1, P0, [0, 0, 0], coords[:, 1:].max(0).tolist(), True, want_csr=True)
    n, c = len(coords), 32
    f = torch.zeros((n, c), dtype=torch.float16, device=DEV)
    w = torch.zeros((27, c, c), dtype=torch.float16, device=DEV)
    out = torch.zeros((n, 2 * c), dtype=torch.float16, device=DEV)
    buf = torch.zeros(km.qsum * 2 * c + 1, dtype=torch.float16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    e = _lib.Epilogue()
    e.ld_out = 2 * c
    rc = lib.pce_conv_fwd_gms(f.data_ptr(), w.data_ptr(), None, out.data_ptr(), _lib.PCE_F16, n, n, c, c, 27, 13, km.icsr.data_ptr(),
                              km.icode.data_ptr(), km.ocsr.data_ptr(), km.ocode.data_ptr(), km.kpos.data_ptr(), km.qkpos.data_ptr(),
                              km.qsum, buf.data_ptr(), buf.numel(), e, s)
    assert rc == _lib.PCE_EINVAL and b"dense" in lib.pce_last_error()
    for bad in (c - 8, c + 4):       # below the channel count, not a multiple of 8
        e = _lib.Epilogue()
        e.ld_out = bad
        rc = lib.pce_conv_fwd_os(f.data_ptr(), w.data_ptr(), None, out.data_ptr(), _lib.PCE_F16, n, n, c, c, 27, km.nbr_out.data_ptr(), e, s)
        assert rc == _lib.PCE_EINVAL and b"row strides" in lib.pce_last_error()
    # a view the kernels cannot take in place (odd column offset) is still served, through a dense copy
    wide = torch.zeros((n, c + 16), dtype=torch.float16, device=DEV)
    wide[:, 4:4 + c] = torch.as_tensor(synth.features(1, n, c), device=DEV).half()
    w = torch.as_tensor(synth.weights(1, 27, c, c), device=DEV).half()
    a = backend.conv_forward(wide[:, 4:4 + c], w, km, DATAFLOW_FDS)
    b = backend.conv_forward(wide[:, 4:4 + c].contiguous(), w, km, DATAFLOW_FDS)
    assert torch.equal(a, b)
