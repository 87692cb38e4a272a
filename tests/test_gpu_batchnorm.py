"""BatchNorm on the GPU (column sums + column affine kernels of the library) against torch.nn.BatchNorm1d
evaluated in float64 on the CPU: outputs, running statistics and all three gradients."""
import numpy as np
import pytest
import torch

import pcengine_amd as pe
from oracle import oracle as orc
from pcengine_amd import _lib, backend, synth
from tests.util import DEV

pytestmark = pytest.mark.gpu


def _tensor(f, dtype):
    coords = torch.zeros((f.shape[0], 4), dtype=torch.int32, device=DEV)
    return pe.spTensor(torch.as_tensor(f, device=DEV).to(dtype).requires_grad_(True), coords, None, [0, 0, 0], [1, 1, 1])


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.float16, 1e-3)])
@pytest.mark.parametrize("n,c", [(70000, 64), (5000, 20), (333, 5), (4097, 256), (2, 8)])
@pytest.mark.parametrize("affine,momentum", [(True, 0.1), (False, None)])
def test_batchnorm_training_matches_torch(n, c, dtype, tol, affine, momentum):
    rng = np.random.default_rng(n + c)
    f = (rng.standard_normal((n, c)) * rng.uniform(0.5, 3.0, c) + rng.uniform(-2, 2, c)).astype(np.float32)
    go = rng.standard_normal((n, c)).astype(np.float32)
    fr = torch.as_tensor(f).to(dtype).double().requires_grad_(True)      # the values the GPU sees
    gr = torch.as_tensor(go).to(dtype).double()
    ref = torch.nn.BatchNorm1d(c, affine=affine, momentum=momentum).double()
    bn = pe.BatchNorm(c, affine=affine, momentum=momentum).to(DEV)
    if affine:
        w = rng.uniform(0.5, 1.5, c)
        b = rng.uniform(-1, 1, c)
        with torch.no_grad():
            ref.weight.copy_(torch.as_tensor(w)); ref.bias.copy_(torch.as_tensor(b))
            bn.weight.copy_(torch.as_tensor(w)); bn.bias.copy_(torch.as_tensor(b))
    for _ in range(2):        # two steps: the running statistics accumulate
        fr.grad = None
        yr = ref(fr)
        yr.backward(gr)
        x = _tensor(f, dtype)
        y = bn(x)
        y.feats.backward(torch.as_tensor(go, device=DEV).to(dtype))
    assert y.feats.dtype == dtype
    # two rows: the variance is the square of half their difference, and eps = 1e-5 decides the last digits
    assert orc.rel_l2(y.feats.detach().double().cpu().numpy(), yr.detach().numpy()) <= (tol if n > 2 else 50 * tol)
    assert orc.rel_l2(x.feats.grad.double().cpu().numpy(), fr.grad.numpy()) <= (tol if n > 2 else 1e-2)
    assert orc.rel_l2(bn.running_mean.double().cpu().numpy(), ref.running_mean.numpy()) <= 1e-6
    assert orc.rel_l2(bn.running_var.double().cpu().numpy(), ref.running_var.numpy()) <= 1e-5
    assert int(bn.num_batches_tracked) == 2
    if affine:
        assert orc.rel_l2(bn.weight.grad.double().cpu().numpy(), ref.weight.grad.numpy()) <= (max(tol, 1e-5) if n > 2 else 1e-2)
        assert orc.rel_l2(bn.bias.grad.double().cpu().numpy(), ref.bias.grad.numpy()) <= max(tol, 1e-5)


def test_batchnorm_eval_mode_and_input_gradient():
    rng = np.random.default_rng(9)
    n, c = 3000, 48
    f = rng.standard_normal((n, c)).astype(np.float32)
    ref = torch.nn.BatchNorm1d(c).double()
    bn = pe.BatchNorm(c).to(DEV)
    with torch.no_grad():
        for m in (ref, bn):
            m.running_mean.copy_(torch.as_tensor(rng.uniform(-1, 1, c)).to(m.running_mean.dtype)) if m is ref else None
        bn.running_mean.copy_(ref.running_mean.float()); bn.running_var.copy_(ref.running_var.float())
        ref.weight.uniform_(0.5, 1.5); bn.weight.copy_(ref.weight.float())
    ref.eval(); bn.eval()
    fr = torch.as_tensor(f).double().requires_grad_(True)
    yr = ref(fr)
    yr.sum().backward()
    x = _tensor(f, torch.float32)
    y = bn(x)
    y.feats.sum().backward()
    assert orc.rel_l2(y.feats.detach().double().cpu().numpy(), yr.detach().numpy()) <= 2e-6
    assert orc.rel_l2(x.feats.grad.double().cpu().numpy(), fr.grad.numpy()) <= 2e-6
    assert int(bn.num_batches_tracked) == 0


def test_column_kernels_directly_and_their_errors():
    lib = _lib.load()
    rng = np.random.default_rng(3)
    a = rng.standard_normal((1000, 7)).astype(np.float32)
    b = rng.standard_normal((1000, 7)).astype(np.float32)
    ad, bd = torch.as_tensor(a, device=DEV), torch.as_tensor(b, device=DEV)
    s = backend.col_sums(ad, bd).cpu().numpy()
    assert np.allclose(s[0], a.astype(np.float64).sum(0), rtol=1e-6) and np.allclose(s[1], (a.astype(np.float64) * b).sum(0), rtol=1e-5, atol=1e-4)
    assert torch.equal(backend.col_sums(ad, bd), backend.col_sums(ad, bd))           # no atomics: same bits every run
    k = [torch.as_tensor(rng.standard_normal(7).astype(np.float32), device=DEV) for _ in range(3)]
    y = backend.col_affine(ad, k[0], k[2], d=bd, kd=k[1], act=("leaky_relu", 0.2)).cpu().numpy()
    want = a * k[0].cpu().numpy() + b * k[1].cpu().numpy() + k[2].cpu().numpy()
    want = np.where(want > 0, want, 0.2 * want)
    assert np.allclose(y, want, rtol=1e-6, atol=1e-6)
    one = ad.data_ptr()
    assert lib.pce_col_sums(one, None, 7, 10, 4, one, 1 << 20, one, None) == _lib.PCE_EINVAL        # dtype
    assert lib.pce_col_sums(one, None, 1, 10, 4, one, 8, one, None) == _lib.PCE_EWORKSPACE
    assert lib.pce_col_sums(one, None, 1, 0, 4, one, 1 << 20, one, None) == _lib.PCE_EINVAL
    assert lib.pce_col_affine(one, None, one, 1, 10, 4, one, None, None, 0, 0.0, None) == _lib.PCE_EINVAL   # k0 missing
    assert lib.pce_col_affine(one, one, one, 1, 10, 4, one, None, one, 0, 0.0, None) == _lib.PCE_EINVAL    # d without kd
    assert lib.pce_col_affine(one, None, one, 1, 10, 4, one, None, one, 9, 0.0, None) == _lib.PCE_EINVAL   # activation


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.float16, 1.5e-3)])
@pytest.mark.parametrize("n,c", [(30000, 64), (777, 20), (4097, 7)])
@pytest.mark.parametrize("with_residual", [False, True])
@pytest.mark.parametrize("act", ["relu", ("leaky_relu", 0.1), None])
def test_batchnorm_with_residual_and_activation(n, c, dtype, tol, with_residual, act):
    """act(norm(x) + residual) in the norm's own passes against the same composition of torch modules in
    float64: output and the gradients of x, weight, bias and the residual."""
    rng = np.random.default_rng(n * 3 + c)
    f = (rng.standard_normal((n, c)) * 1.5 + 0.3).astype(np.float32)
    r = rng.standard_normal((n, c)).astype(np.float32)
    go = rng.standard_normal((n, c)).astype(np.float32)
    w, b = rng.uniform(0.5, 1.5, c), rng.uniform(-1, 1, c)
    ref = torch.nn.BatchNorm1d(c).double()
    bn = pe.BatchNorm(c).to(DEV)
    with torch.no_grad():
        ref.weight.copy_(torch.as_tensor(w)); ref.bias.copy_(torch.as_tensor(b))
        bn.weight.copy_(torch.as_tensor(w)); bn.bias.copy_(torch.as_tensor(b))
    fr = torch.as_tensor(f).to(dtype).double().requires_grad_(True)
    rr = torch.as_tensor(r).to(dtype).double().requires_grad_(True)
    yr = ref(fr) + (rr if with_residual else 0.0)
    if act == "relu":
        yr = torch.relu(yr)
    elif act is not None:
        yr = torch.nn.functional.leaky_relu(yr, act[1])
    yr.backward(torch.as_tensor(go).to(dtype).double())
    x, res = _tensor(f, dtype), _tensor(r, dtype)
    y = bn(x, residual=res if with_residual else None, act=act)
    y.feats.backward(torch.as_tensor(go, device=DEV).to(dtype))
    assert y.feats.dtype == dtype
    assert orc.rel_l2(y.feats.detach().double().cpu().numpy(), yr.detach().numpy()) <= tol
    # an output that rounds to zero in fp16 masks its gradient where float64 keeps a tiny positive value
    assert orc.rel_l2(x.feats.grad.double().cpu().numpy(), fr.grad.numpy()) <= 3 * tol
    assert orc.rel_l2(bn.weight.grad.double().cpu().numpy(), ref.weight.grad.numpy()) <= 3 * max(tol, 1e-5)
    assert orc.rel_l2(bn.bias.grad.double().cpu().numpy(), ref.bias.grad.numpy()) <= 3 * max(tol, 1e-5)
    if with_residual:
        assert orc.rel_l2(res.feats.grad.double().cpu().numpy(), rr.grad.numpy()) <= 3 * tol
    else:
        assert res.feats.grad is None


def test_batchnorm_activation_arguments():
    bn = pe.BatchNorm(8).to(DEV)
    with pytest.raises(ValueError):      # torch.nn.BatchNorm1d refuses batch statistics of one row
        bn(_tensor(np.ones((1, 8), np.float32), torch.float32))
    x = _tensor(np.ones((16, 8), np.float32), torch.float32)
    with pytest.raises(ValueError):
        bn(x, act="gelu")
    with pytest.raises(ValueError):
        bn(x, act=("leaky_relu", -0.1))
    y, mean, rstd = backend.bn_forward(x.feats.detach(), None, None, None, None, True, -1.0, 1e-5, act="relu")
    with pytest.raises(ValueError):
        backend.bn_backward(x.feats.detach(), y, None, mean, rstd, True, y_act=None, act="relu")
    with pytest.raises(ValueError):
        backend.bn_forward(x.feats.detach(), None, None, None, None, True, -1.0, 1e-5, residual=torch.zeros(3, 8, device=DEV))
