"""Gradients of the sparse convolution (features, kernel, bias) against the float64 oracle, whose
backward is pinned by torch.autograd through a dense conv3d (tests/test_oracle.py)."""
import numpy as np
import pytest
import torch

import pcengine_amd as pe
from oracle import oracle as orc
from pcengine_amd import backend, nets, synth
from tests.util import DEV, TOL, gpu_map, rounded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("c_in,c_out", [(16, 16), (64, 64), (5, 7), (96, 160)])
def test_backward_submanifold_strided_transposed(c_in, c_out, dtype):
    coords = synth.random_cloud(seed=71, n=6000, extent=19, batches=2)
    rng = np.random.default_rng(71)
    for ks, stride, pad in [((3, 3, 3), (1, 1, 1), (0, 0, 0)), ((2, 2, 2), (2, 2, 2), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (1, 1, 1))]:
        kv = ks[0] * ks[1] * ks[2]
        ref = orc.kernel_map(coords, ks, stride, pad)
        km = gpu_map(coords, ks, stride, pad, want_csr=True, want_nbr_in=True)
        f = rounded(synth.features(7, len(coords), c_in), dtype)
        w = rounded(synth.weights(7, kv, c_in, c_out), dtype)
        g = rounded(rng.standard_normal((ref.n_out, c_out)), dtype)
        fd, wd, gd = (torch.as_tensor(a, device=DEV).to(dtype) for a in (f, w, g))
        gf, gw = backend.conv_backward(fd, wd, km, gd)
        want_f, want_w = orc.conv_backward(f, w, ref, ks, g)
        assert gf.dtype == dtype and gw.dtype == dtype and gw.shape == wd.shape
        assert orc.rel_l2(gf.double().cpu().numpy(), want_f) <= TOL[dtype], (ks, "feats")
        assert orc.rel_l2(gw.double().cpu().numpy(), want_w) <= TOL[dtype], (ks, "kernel")
        if tuple(stride) != (1, 1, 1):
            fo = rounded(synth.features(8, ref.n_out, c_out), dtype)
            wt = rounded(synth.weights(8, kv, c_out, c_in), dtype)
            gi = rounded(rng.standard_normal((len(coords), c_in)), dtype)
            fod, wtd, gid = (torch.as_tensor(a, device=DEV).to(dtype) for a in (fo, wt, gi))
            gf, gw = backend.conv_backward(fod, wtd, km, gid, transposed=True)
            want_f, want_w = orc.conv_backward(fo, wt, ref, ks, gi, transposed=True)
            assert orc.rel_l2(gf.double().cpu().numpy(), want_f) <= TOL[dtype]
            assert orc.rel_l2(gw.double().cpu().numpy(), want_w) <= TOL[dtype]


def test_autograd_through_the_front_end():
    """conv3d (3x3x3 with bias) -> ReLU -> k2s2 down -> transposed up -> 1x1 head: parameter and input
    gradients of a scalar loss against the oracle chain evaluated in float64."""
    coords = synth.random_cloud(seed=72, n=3000, extent=16, batches=2)
    n = len(coords)
    torch.manual_seed(0)
    a = pe.conv3d(8, 16, 3, bias=True).to(DEV)
    down = pe.conv3d(16, 24, 2, 2).to(DEV)
    up = pe.conv3d(24, 16, 2, 2, transposed=True).to(DEV)
    head = pe.conv3d(16, 5, 1, bias=True).to(DEV)
    f = synth.features(9, n, 8).astype(np.float32)
    feats = torch.as_tensor(f, device=DEV).requires_grad_(True)
    x = pe.spTensor(feats, torch.as_tensor(coords, device=DEV), None, [0, 0, 0], coords[:, 1:].max(0).tolist(), batchsize=2)
    y = head(up(down(pe.ReLU()(a(x)))))
    g = np.random.default_rng(9).standard_normal((n, 5))
    (y.feats * torch.as_tensor(g, device=DEV).float()).sum().backward()
    # oracle chain
    m3, m2 = orc.kernel_map(coords, (3, 3, 3)), orc.kernel_map(coords, (2, 2, 2), (2, 2, 2))
    P = lambda t: t.detach().double().cpu().numpy()
    wa, ba, wd_, wu, wh, bh = P(a.kernel), P(a.bias), P(down.kernel), P(up.kernel), P(head.kernel), P(head.bias)
    h1 = orc.conv_forward(f, wa, m3, (3, 3, 3), bias=ba)
    r1 = np.maximum(h1, 0)
    h2 = orc.conv_forward(r1, wd_, m2, (2, 2, 2))
    h3 = orc.conv_forward(h2, wu, m2, (2, 2, 2), transposed=True)
    assert orc.rel_l2(P(y.feats), h3 @ wh + bh) <= 1e-5
    g3 = g @ wh.T
    g2, gwu = orc.conv_backward(h2, wu, m2, (2, 2, 2), g3, transposed=True)
    gr1, gwd = orc.conv_backward(r1, wd_, m2, (2, 2, 2), g2)
    gh1 = gr1 * (h1 > 0)
    gx, gwa = orc.conv_backward(f, wa, m3, (3, 3, 3), gh1)
    for got, want in ((head.kernel.grad, h3.T @ g), (head.bias.grad, g.sum(0)), (up.kernel.grad, gwu), (down.kernel.grad, gwd),
                      (a.kernel.grad, gwa), (a.bias.grad, gh1.sum(0)), (feats.grad, gx)):
        assert orc.rel_l2(P(got), want) <= 2e-5


def test_unet_training_step_produces_finite_gradients():
    coords = synth.random_cloud(seed=73, n=4000, extent=32)
    f = synth.features(11, len(coords), 4).astype(np.float32)
    torch.manual_seed(3)
    model = nets.SparseResUNet(4, 6, stem=8, enc=(8, 16, 16, 32), dec=(32, 16, 16, 8)).to(DEV).train()
    x = pe.spTensor(torch.as_tensor(f, device=DEV), torch.as_tensor(coords, device=DEV), None, [0, 0, 0],
                    coords[:, 1:].max(0).tolist())
    out = model(x)
    target = torch.randint(0, 6, (len(coords),), device=DEV)
    loss = torch.nn.functional.cross_entropy(out.feats, target)
    loss.backward()
    params = [p for p in model.parameters() if p.requires_grad]
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in params)
    assert sum(float(p.grad.abs().sum()) for p in params) > 0
    before = float(loss.detach())
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    opt.step()
    with torch.no_grad():
        x2 = pe.spTensor(torch.as_tensor(f, device=DEV), torch.as_tensor(coords, device=DEV), None, [0, 0, 0],
                         coords[:, 1:].max(0).tolist())
        after = float(torch.nn.functional.cross_entropy(model(x2).feats, target))
    assert after < before


@pytest.mark.parametrize("dtype,c_in,c_out", [(torch.float32, 16, 24), (torch.float16, 72, 136)])
def test_kernel_gradient_long_runs(dtype, c_in, c_out):
    """Enough pairs that a workgroup of the kernel-gradient kernel takes a run of several 128-pair quanta
    and crosses from one offset to the next inside the run (its accumulators are flushed there), with
    channel counts that leave partial blocks."""
    coords = synth.random_cloud(seed=81, n=70000, extent=42)
    ref = orc.kernel_map(coords, (3, 3, 3))
    assert (ref.M // 128 + len(coords) // 128) * (1 if c_in <= 64 and c_out <= 64 else 4) >= 2 * 2048
    f = synth.features(12, len(coords), c_in)
    go = synth.features(13, len(coords), c_out)
    w = synth.weights(12, 27, c_in, c_out)
    _, gw_want = orc.conv_backward(rounded(f, dtype), rounded(w, dtype), ref, (3, 3, 3), rounded(go, dtype))
    km = gpu_map(coords, (3, 3, 3), want_csr=True)
    gw = backend.conv_wgrad(torch.as_tensor(f, device=DEV).to(dtype), torch.as_tensor(go, device=DEV).to(dtype), km)
    assert gw.dtype == torch.float32 and gw.shape == (27, c_in, c_out)
    assert orc.rel_l2(gw.double().cpu().numpy(), gw_want) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("n,c_in,c_out", [(0, 8, 8), (1, 3, 5), (127, 32, 20), (5000, 96, 20), (40000, 64, 128), (3001, 130, 70)])
def test_dense_layer_kernel_gradient(n, c_in, c_out, dtype):
    """The 1x1 layer's kernel gradient is feats^T @ grad_out: checked against that product in float64 on
    the rounded operands (the kernel sums in fp32; rows are summed in a different order per run)."""
    g = torch.Generator().manual_seed(n + c_in)
    a = torch.randn(n, c_in, generator=g).to(dtype).to(DEV)
    b = torch.randn(n, c_out, generator=g).to(dtype).to(DEV)
    gw = backend.dense_wgrad(a, b)
    assert gw.dtype == torch.float32 and tuple(gw.shape) == (c_in, c_out)
    ref = a.double().t() @ b.double()
    scale = float(ref.abs().max()) if n else 1.0
    assert float((gw.double() - ref).abs().max()) <= 1e-5 * max(scale, 1.0) + 1e-6 * max(n, 1) ** 0.5
    with pytest.raises(TypeError):
        backend.dense_wgrad(a, b.to(torch.float64))
    with pytest.raises(ValueError):
        backend.dense_wgrad(a, torch.zeros(n + 1, c_out, dtype=dtype, device=DEV))


def test_unet_fused_training_path_matches_the_composition_of_torch_modules():
    """The training path of the network (norm + residual + ReLU in the norm's own passes, the concatenation
    kernel, transposed layers that store once) against the same network with torch's BatchNorm1d, add, relu and
    cat around this package's convolutions: output and every parameter gradient, fp32.
    The two forwards agree to rounding (1e-6), but a single activation within that distance of zero takes the
    other branch of its ReLU in one of them, and one changed mask element moves a gradient tensor of 4*10^4
    elements by 1/sqrt(4*10^4) = 0.5 % of its norm: the gradient bar is 1e-2 (a wrong mask, sign or missing
    term moves it by order one), the output bar 1e-5."""
    import copy
    from pcengine_amd import batchnorm, utils
    coords = synth.random_cloud(seed=74, n=5000, extent=60)
    f = synth.features(12, len(coords), 4).astype(np.float32)
    torch.manual_seed(5)
    model = nets.SparseResUNet(4, 6, stem=8, enc=(8, 16, 16, 32), dec=(32, 16, 16, 8)).to(DEV).train()
    twin = copy.deepcopy(model)
    weight = torch.randn(len(coords), 6, device=DEV)

    def run(net):
        x = pe.spTensor(torch.as_tensor(f, device=DEV), torch.as_tensor(coords, device=DEV), None, [0, 0, 0],
                        coords[:, 1:].max(0).tolist())
        out = net(x).feats
        (out * weight).sum().backward()
        return out.detach()

    out_a = run(model)

    def torch_features(self, x, residual=None, act=None):
        y = torch.nn.BatchNorm1d.forward(self, x)
        if residual is not None:
            y = y + residual
        return torch.relu(y) if act == "relu" else y
    old_features, old_cat = batchnorm.BatchNorm._features, nets.cat
    batchnorm.BatchNorm._features = torch_features
    nets.cat = lambda inputs: inputs[0]._like(torch.cat([t.feats for t in inputs], dim=1))
    try:
        out_b = run(twin)
    finally:
        batchnorm.BatchNorm._features, nets.cat = old_features, old_cat
    P = lambda t: t.double().cpu().numpy()
    assert orc.rel_l2(P(out_a), P(out_b)) <= 1e-5
    worst = 0.0
    for (name, p), q in zip(model.named_parameters(), twin.parameters()):
        assert p.grad is not None and q.grad is not None, name
        worst = max(worst, orc.rel_l2(P(p.grad), P(q.grad)))
        assert orc.rel_l2(P(p.grad), P(q.grad)) <= 1e-2, (name, worst)
    for a, b in zip(model.buffers(), twin.buffers()):
        assert orc.rel_l2(P(a), P(b)) <= 1e-5
