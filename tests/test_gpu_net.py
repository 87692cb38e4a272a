"""The MinkUNet-style network end to end against a float64 oracle forward with the same weights."""
import numpy as np
import pytest
import torch

import pcengine_amd as pe
from oracle import oracle as orc
from pcengine_amd import nets, synth
from tests.util import DEV

pytestmark = pytest.mark.gpu


def _oracle_forward(model, coords, feats):
    """Walks the module tree and restates every layer with the oracle's maps (float64)."""
    maps = {}

    def conv(m, c, f):
        w = m.kernel.detach().double().cpu().numpy()
        b = None if m.bias is None else m.bias.detach().double().cpu().numpy()
        ks, st = tuple(m.kernel_size), tuple(m.stride)
        if ks == (1, 1, 1) and st == (1, 1, 1):
            out = f @ w
            return c, out + b if b is not None else out
        if m.transposed:
            fine, km = maps[("up", len(c))]
            return fine, orc.conv_forward(f, w, km, ks, transposed=True, bias=b)
        key = (ks, st, len(c), c[:, 1:].max())
        if key not in maps:
            maps[key] = orc.kernel_map(c, ks, st)
            if st != (1, 1, 1):
                maps[("up", maps[key].n_out)] = (c, maps[key])
        km = maps[key]
        return km.out_coords, orc.conv_forward(f, w, km, ks, bias=b)

    def convbn(m, c, f):
        c, f = conv(m.conv, c, f)
        if m.bn is not None:
            bn = m.bn
            s = (bn.weight / torch.sqrt(bn.running_var + bn.eps)).detach().double().cpu().numpy()
            f = (f - bn.running_mean.double().cpu().numpy()) * s + bn.bias.detach().double().cpu().numpy()
        return c, np.maximum(f, 0) if m.relu is not None else f

    def res(m, c, f):
        c1, y = convbn(m.a, c, f)
        c1, y = convbn(m.b, c1, y)
        s = f if m.shortcut is None else convbn(m.shortcut, c, f)[1]
        return c1, np.maximum(y + s, 0)

    c, f = coords, feats
    for m in model.stem:
        c, f = convbn(m, c, f)
    skips = [(c, f)]
    for down, enc in zip(model.down, model.enc):
        c, f = convbn(down, c, f)
        for r in enc:
            c, f = res(r, c, f)
        skips.append((c, f))
    skips.pop()
    for up, dec in zip(model.up, model.dec):
        c, f = convbn(up, c, f)
        sc, sf = skips.pop()
        assert np.array_equal(sc, c)
        f = np.concatenate([f, sf], 1)
        for r in dec:
            c, f = res(r, c, f)
    return conv(model.head, c, f)


def _model(seed=0):
    torch.manual_seed(seed)
    m = nets.SparseResUNet(4, 20, stem=16, enc=(16, 32, 48, 64), dec=(64, 48, 24, 24)).to(DEV)
    for mod in m.modules():
        if isinstance(mod, pe.BatchNorm):
            with torch.no_grad():
                mod.running_mean.uniform_(-0.1, 0.1)
                mod.running_var.uniform_(0.5, 1.5)
                mod.weight.uniform_(0.8, 1.2)
                mod.bias.uniform_(-0.1, 0.1)
    return m.eval()


@pytest.mark.parametrize("flow", ["auto", "fds", "os", "fod", "gms"])
def test_unet_fp32_matches_oracle_and_bn_folding(flow, monkeypatch):
    if flow != "auto":
        monkeypatch.setenv("PCENGINE_DATAFLOW", flow)
    coords = synth.random_cloud(seed=61, n=12000, extent=40, batches=2)
    f = synth.features(8, len(coords), 4)
    model = _model()
    want_c, want = _oracle_forward(model, coords, f.astype(np.float64))

    def run():
        x = pe.spTensor(torch.as_tensor(f, device=DEV), torch.as_tensor(coords, device=DEV), None, [0, 0, 0],
                        coords[:, 1:].max(0).tolist())
        with torch.no_grad():
            return model(x)
    y = run()
    assert np.array_equal(y.coords.cpu().numpy(), want_c) and y.feats.shape == (len(coords), 20)
    assert orc.rel_l2(y.feats.double().cpu().numpy(), want) <= 2e-5
    model.fuse_bn()
    assert not any(isinstance(m, pe.BatchNorm) for m in model.modules())
    z = run()
    assert orc.rel_l2(z.feats.double().cpu().numpy(), want) <= 2e-5


def test_unet_fp16_runs_close_to_fp32():
    coords = synth.random_cloud(seed=62, n=9000, extent=36)
    f = synth.features(9, len(coords), 4)
    model = _model(1).fuse_bn()
    mk = lambda dt: pe.spTensor(torch.as_tensor(f, device=DEV).to(dt), torch.as_tensor(coords, device=DEV), None,
                                [0, 0, 0], coords[:, 1:].max(0).tolist())
    with torch.no_grad():
        ref = model(mk(torch.float32)).feats
        out = model.half()(mk(torch.float16)).feats
    assert out.dtype == torch.float16
    # forty fp16 layers deep: storage rounding accumulates, the per-layer bar (1e-3) does not apply end to end
    assert orc.rel_l2(out.double().cpu().numpy(), ref.double().cpu().numpy()) <= 2e-2


def test_prebuilt_maps_cover_the_whole_network(monkeypatch):
    """prebuild_maps builds the nine maps of the U-Net (five submanifold, four strided) before any
    convolution -- the output coordinates of the four strided levels in one chained build -- ; the layers then find
    all of them cached, and the result does not depend on it: built lazily, level by level, the maps and the
    output are the same bit for bit."""
    from pcengine_amd import backend, spconv
    coords = synth.random_cloud(seed=63, n=6000, extent=32)
    f = synth.features(10, len(coords), 4)
    model = _model(2).fuse_bn()
    mk = lambda: pe.spTensor(torch.as_tensor(f, device=DEV).float(), torch.as_tensor(coords, device=DEV), None,
                             [0, 0, 0], coords[:, 1:].max(0).tolist())
    x = mk()
    spconv.prebuild_maps(x, model.map_plan())
    assert len(x.kmaps) == 9 and len(x.cbook) == 5
    calls = []
    real = backend.build_kernel_map
    monkeypatch.setattr(backend, "build_kernel_map", lambda *a, **k: calls.append(1) or real(*a, **k))
    with torch.no_grad():
        y = model(x)
    assert calls == []
    # without the prebuild (maps built lazily, layer by layer) the output is bit-identical
    monkeypatch.setattr(spconv, "prebuild_maps", lambda *a, **k: None)
    monkeypatch.setattr(nets, "prebuild_maps", lambda *a, **k: None)
    with torch.no_grad():
        z = model(mk())
    assert len(calls) == 9 and torch.equal(y.feats, z.feats)
    for key, km in x.kmaps.items():
        other = z.kmaps[key]
        assert torch.equal(km.out_coords, other.out_coords) and torch.equal(km.imap, other.imap) and torch.equal(km.omap, other.omap)


def test_maps_prefetched_on_a_second_stream():
    """Forwards whose maps were built on a second stream while the previous forward ran (MapPrefetcher), the maps
    dropped as soon as the host returns: every output equals the plain forward's, bit for bit, and no layer
    builds a map."""
    from pcengine_amd import spconv
    clouds = [synth.random_cloud(seed=70 + i, n=15000 + 1000 * i, extent=36) for i in range(3)]
    model = _model(2).fuse_bn().half()
    feats = [torch.as_tensor(synth.features(12 + i, len(c), 4), device=DEV).half() for i, c in enumerate(clouds)]
    cds = [torch.as_tensor(c, device=DEV) for c in clouds]
    mk = lambda i: pe.spTensor(feats[i], cds[i], None, [0, 0, 0], clouds[i][:, 1:].max(0).tolist())
    with torch.no_grad():
        want = [model(mk(i)).feats.clone() for i in range(3)]
    torch.cuda.synchronize()
    pf = spconv.MapPrefetcher(model.map_plan(), DEV)
    order = [0, 1, 2, 0, 1, 2, 2, 1, 0]
    outs = []
    nxt = mk(order[0])
    pf.submit(nxt)
    with torch.no_grad():
        for k, i in enumerate(order):
            cur = nxt
            pf.take(cur)
            assert len(cur.kmaps) == 9
            outs.append(model(cur).feats)
            if k + 1 < len(order):
                nxt = mk(order[k + 1])
                pf.submit(nxt)
            del cur
    torch.cuda.synchronize()
    for i, o in zip(order, outs):
        assert torch.equal(o, want[i])

