"""The Python front end (conv3d / spTensor / BatchNorm / ReLU / cat) on the GPU against the oracle."""
import numpy as np
import pytest
import torch

import pcengine_amd as pe
from oracle import oracle as orc
from pcengine_amd import synth
from tests.util import DEV, rounded

pytestmark = pytest.mark.gpu


def _tensor(coords, c, dtype, init_tag=None):
    f = synth.features(7, len(coords), c)
    x = pe.spTensor(torch.as_tensor(f, device=DEV).to(dtype), torch.as_tensor(coords, device=DEV), None,
                    [0, 0, 0], coords[:, 1:].max(0).tolist(), init_tag=init_tag)
    return x, rounded(f, dtype)


def _weights(layer, dtype):
    w = layer.kernel.detach().to(dtype).double().cpu().numpy()
    return w


@pytest.mark.parametrize("flow,tags", [("auto", None), ("fod", None), ("gms", None), ("os", None), ("fds", None), ("auto", ["D1", "D2", "end"]),
                                       ("auto", ["D2", "D1", "end"])])
def test_down_up_block_matches_oracle(flow, tags):
    dtype = torch.float16
    coords = synth.random_cloud(seed=51, n=8000, extent=24, batches=2)
    x, f = _tensor(coords, 16, dtype, init_tag=tags)
    torch.manual_seed(0)
    c1 = pe.conv3d(16, 32, 3, dataflow=flow).to(DEV).half()
    down = pe.conv3d(32, 64, 2, 2, dataflow=flow).to(DEV).half()
    c2 = pe.conv3d(64, 64, 3, bias=True, dataflow=flow).to(DEV).half()
    up = pe.conv3d(64, 32, 2, 2, transposed=True, dataflow=flow).to(DEV).half()
    head = pe.conv3d(64, 20, 1, bias=True).to(DEV).half()
    relu = pe.ReLU()
    with torch.no_grad():
        y1 = relu(c1(x))
        y2 = relu(down(y1))
        y3 = relu(c2(y2))
        y4 = up(y3)
        y5 = head(pe.cat([y4, y1]))
    # oracle, carrying the GPU's fp16 activations forward layer by layer
    m1 = orc.kernel_map(coords, (3, 3, 3))
    m2 = orc.kernel_map(coords, (2, 2, 2), (2, 2, 2))
    m3 = orc.kernel_map(m2.out_coords, (3, 3, 3))
    assert np.array_equal(y2.coords.cpu().numpy(), m2.out_coords)
    assert y4.coords is x.coords and y2.stride == pe.conv_info_encoder([2, 2, 2]) and y4.stride == x.stride
    assert y2.coords_max == orc.strided_coords_max(x.coords_max, (2, 2, 2), (2, 2, 2), (0, 0, 0))
    assert len(x.kmaps) == 3 and y5.kmaps is x.kmaps
    g = lambda t: t.feats.double().cpu().numpy()
    want1 = np.maximum(orc.conv_forward(f, _weights(c1, dtype), m1, (3, 3, 3)), 0)
    assert orc.rel_l2(g(y1), want1) <= 1e-3
    want2 = np.maximum(orc.conv_forward(g(y1), _weights(down, dtype), m2, (2, 2, 2)), 0)
    assert orc.rel_l2(g(y2), want2) <= 1e-3
    want3 = np.maximum(orc.conv_forward(g(y2), _weights(c2, dtype), m3, (3, 3, 3), bias=c2.bias.detach().double().cpu().numpy()), 0)
    assert orc.rel_l2(g(y3), want3) <= 1e-3
    want4 = orc.conv_forward(g(y3), _weights(up, dtype), m2, (2, 2, 2), transposed=True)
    assert orc.rel_l2(g(y4), want4) <= 1e-3
    want5 = np.concatenate([g(y4), g(y1)], 1) @ _weights(head, dtype) + head.bias.detach().double().cpu().numpy()
    assert orc.rel_l2(g(y5), want5) <= 1e-3
    if tags:
        assert x.init_tag == tags[1:] and len(tags) == 3     # consumed one per new map; the caller's list is not mutated
        assert y5.init_tag == ["end"]
        first = x.kmaps[(pe.conv_info_encoder([3, 3, 3]), x.stride, pe.conv_info_encoder([1, 1, 1]))]
        assert len(first) == (8 if tags[0] == "D1" else 6)


def test_transposed_without_cached_map_raises():
    coords = synth.random_cloud(seed=52, n=500, extent=10)
    x, _ = _tensor(coords, 8, torch.float32)
    with pytest.raises(KeyError):
        pe.conv3d(8, 8, 2, 2, transposed=True).to(DEV)(x)


def test_batchnorm_and_residual_fp32():
    coords = synth.random_cloud(seed=53, n=3000, extent=16)
    x, f = _tensor(coords, 16, torch.float32)
    conv = pe.conv3d(16, 16, 3).to(DEV)
    bn = pe.BatchNorm(16).to(DEV).eval()
    with torch.no_grad():
        bn.running_mean.uniform_(-0.1, 0.1)
        bn.running_var.uniform_(0.5, 1.5)
        y = pe.ReLU()(bn(conv(x))) + x
    m = orc.kernel_map(coords, (3, 3, 3))
    z = orc.conv_forward(f, conv.kernel.detach().double().cpu().numpy(), m, (3, 3, 3))
    mean, var = bn.running_mean.double().cpu().numpy(), bn.running_var.double().cpu().numpy()
    want = np.maximum((z - mean) / np.sqrt(var + bn.eps), 0) + f
    assert orc.rel_l2(y.feats.double().cpu().numpy(), want) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("n,c_a,c_b", [(1, 8, 8), (5000, 96, 32), (70001, 192, 64), (333, 256, 128), (4097, 12, 20), (100, 5, 7),
                                       (64, 1024, 1032)])
def test_cat_of_two_tensors(n, c_a, c_b, dtype):
    """`cat` of two tensors (the skip concatenation of a U-Net) is bit-identical to torch.cat, whether the
    streaming kernel takes the layout or not, and hands the gradient back in two slices."""
    from pcengine_amd import backend
    g = torch.Generator().manual_seed(n + c_a)
    a = torch.randn(n, c_a, generator=g).to(dtype).to(DEV).requires_grad_(True)
    b = torch.randn(n, c_b, generator=g).to(dtype).to(DEV).requires_grad_(True)
    coords = torch.zeros((n, 4), dtype=torch.int32, device=DEV)
    xa = pe.spTensor(a, coords, None, [0, 0, 0], [1, 1, 1])
    xb = pe.spTensor(b, coords, None, [0, 0, 0], [1, 1, 1])
    y = pe.cat([xa, xb])
    want = torch.cat([a.detach(), b.detach()], dim=1)
    assert y.feats.dtype == dtype and torch.equal(y.feats.detach(), want)
    per = 8 if dtype == torch.float16 else 4
    fits = c_a % per == 0 and c_b % per == 0 and (c_a + c_b) // per <= 256
    assert (backend.concat_cols(a.detach(), b.detach()) is not None) == fits
    go = torch.randn(n, c_a + c_b, generator=g).to(dtype).to(DEV)
    y.feats.backward(go)
    assert torch.equal(a.grad, go[:, :c_a]) and torch.equal(b.grad, go[:, c_a:])
    z = pe.cat([xa, xb, xa])            # more than two inputs: torch's own concatenation
    assert torch.equal(z.feats.detach(), torch.cat([want, a.detach()], dim=1))
