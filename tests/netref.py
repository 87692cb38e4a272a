"""Float64 restatements of the MinkUNet-style network for the parity tests: the whole forward over the
oracle's maps, the oracle's maps of every resolution level, and a per-layer checker that verifies sampled
output rows of every convolution a real forward executes.  Test infrastructure only."""
import numpy as np
import torch

from oracle import oracle as orc

K3, K2, S1, S2, P0 = (3, 3, 3), (2, 2, 2), (1, 1, 1), (2, 2, 2), (0, 0, 0)


def oracle_pyramid(coords: np.ndarray, levels: int = 5):
    """[(coords_l, cmax_l, submanifold map, k2s2 map or None)] for the resolution levels of a network forward.
    The bound on the output coordinates of a strided layer is the one the front end carries from level to
    level (script/spconv.py:358-360, 455-457), not the largest coordinate present."""
    out = []
    cmax = [int(v) for v in coords[:, 1:].max(axis=0)]
    for lv in range(levels):
        sub = orc.kernel_map(coords, K3)
        down = orc.kernel_map(coords, K2, S2, P0, cmax=cmax) if lv + 1 < levels else None
        out.append((coords, cmax, sub, down))
        if down is not None:
            coords = down.out_coords
            cmax = orc.strided_coords_max(cmax, K2, S2, P0)
    return out


def _np64(t):
    return t.detach().double().cpu().numpy()


def oracle_forward(model, coords: np.ndarray, feats: np.ndarray, pyramid=None):
    """Walks the module tree of a SparseResUNet and restates every layer in float64 over the oracle's maps
    (BatchNorm in inference form where it has not been folded).  Returns (coords, features)."""
    pyramid = pyramid or oracle_pyramid(coords)
    level_of = {len(p[0]): i for i, p in enumerate(pyramid)}

    def conv(m, lv, f):
        w = _np64(m.kernel)
        b = None if m.bias is None else _np64(m.bias)
        ks, st = tuple(m.kernel_size), tuple(m.stride)
        if ks == (1, 1, 1) and st == S1:
            out = f @ w
            return lv, out + b if b is not None else out
        if m.transposed:
            return lv - 1, orc.conv_forward(f, w, pyramid[lv - 1][3], ks, transposed=True, bias=b)
        if st == S1:
            return lv, orc.conv_forward(f, w, pyramid[lv][2], ks, bias=b)
        return lv + 1, orc.conv_forward(f, w, pyramid[lv][3], ks, bias=b)

    def convbn(m, lv, f):
        lv, f = conv(m.conv, lv, f)
        if m.bn is not None:
            bn = m.bn
            s = _np64(bn.weight / torch.sqrt(bn.running_var + bn.eps))
            f = (f - _np64(bn.running_mean)) * s + _np64(bn.bias)
        return lv, np.maximum(f, 0) if m.relu is not None else f

    def res(m, lv, f):
        _, y = convbn(m.a, lv, f)
        _, y = convbn(m.b, lv, y)
        s = f if m.shortcut is None else convbn(m.shortcut, lv, f)[1]
        return lv, np.maximum(y + s, 0)

    lv, f = level_of[len(coords)], feats.astype(np.float64)
    for m in model.stem:
        lv, f = convbn(m, lv, f)
    skips = [f]
    for down, enc in zip(model.down, model.enc):
        lv, f = convbn(down, lv, f)
        for r in enc:
            lv, f = res(r, lv, f)
        skips.append(f)
    skips.pop()
    for up, dec in zip(model.up, model.dec):
        lv, f = convbn(up, lv, f)
        f = np.concatenate([f, skips.pop()], 1)
        for r in dec:
            lv, f = res(r, lv, f)
    lv, f = conv(model.head, lv, f)
    return pyramid[lv][0], f


def _act(x: np.ndarray, act):
    if act is None:
        return x
    if act == "relu":
        return np.maximum(x, 0.0)
    return np.where(x > 0, x, x * act[1])


class LayerChecker:
    """Wraps ``backend.conv_forward`` / ``backend.dense_forward`` during a real forward: after every call it
    recomputes `rows` sampled output rows in float64 from the call's own inputs (the fp16 / fp32 features and
    weights the kernel saw) over the ORACLE's map of that level, and records the rel-L2 error of those rows."""

    def __init__(self, backend, pyramid, rows: int = 128, seed: int = 0):
        self.backend, self.pyramid = backend, pyramid
        self.level_of = {len(p[0]): i for i, p in enumerate(pyramid)}
        self.rows, self.rng = rows, np.random.default_rng(seed)
        self.real_conv, self.real_dense = backend.conv_forward, backend.dense_forward
        self.records = []     # (kind, n_in, n_out, c_in, c_out, dataflow, rel_l2)

    def install(self, monkeypatch):
        monkeypatch.setattr(self.backend, "conv_forward", self.conv_forward)
        monkeypatch.setattr(self.backend, "dense_forward", self.dense_forward)

    def _sample(self, n):
        return np.sort(self.rng.choice(n, size=min(self.rows, n), replace=False))

    def _finish(self, kind, exp, rows, out, bias, residual, act, n_in, c_in, dataflow):
        idx = torch.as_tensor(rows, device=out.device)
        if bias is not None:
            exp = exp + _np64(bias)
        if residual is not None:
            exp = exp + _np64(residual[idx])
        exp = _act(exp, act)
        err = orc.rel_l2(_np64(out[idx]), exp)
        self.records.append((kind, n_in, out.shape[0], c_in, out.shape[1], dataflow, err))

    def dense_forward(self, feats, weight, packed=None, bias=None, residual=None, act=None):
        out = self.real_dense(feats, weight, packed, bias=bias, residual=residual, act=act)
        rows = self._sample(feats.shape[0])
        idx = torch.as_tensor(rows, device=feats.device)
        exp = _np64(feats[idx]) @ _np64(weight)
        self._finish("1x1", exp, rows, out, bias, residual, act, feats.shape[0], feats.shape[1], -1)
        return out

    def conv_forward(self, feats, weight, km, dataflow, transposed=False, buffer=None, packed=None, out=None, bias=None,
                     residual=None, act=None, **kw):
        out = self.real_conv(feats, weight, km, dataflow, transposed=transposed, buffer=buffer, packed=packed, out=out,
                             bias=bias, residual=residual, act=act, **kw)
        lv = self.level_of[km.n_in]
        ref = self.pyramid[lv][2] if km.subm else self.pyramid[lv][3]
        assert ref.M == km.M and ref.n_out == km.n_out, "the GPU map and the oracle's map differ in size"
        src, dst = (ref.omap, ref.imap) if transposed else (ref.imap, ref.omap)
        w = _np64(weight if weight.dim() == 3 else weight.unsqueeze(0))
        rows = self._sample(out.shape[0])
        pos = -np.ones(out.shape[0], np.int64)
        pos[rows] = np.arange(len(rows))
        sel = np.nonzero(pos[dst] >= 0)[0]
        kp_of = np.searchsorted(ref.kpos.astype(np.int64), sel, side="right") - 1
        need = np.unique(np.concatenate([src[sel].astype(np.int64), rows if km.subm else np.zeros(0, np.int64)]))
        got = _np64(feats[torch.as_tensor(need, device=feats.device)])
        where = -np.ones(feats.shape[0], np.int64)
        where[need] = np.arange(len(need))
        exp = np.zeros((len(rows), w.shape[2]))
        if km.subm:
            exp += got[where[rows]] @ w[orc.mid_offset(km.ks)]
        for kp in np.unique(kp_of):
            p = sel[kp_of == kp]
            np.add.at(exp, pos[dst[p]], got[where[src[p]]] @ w[kp])
        kind = ("T" if transposed else "") + ("subm3" if km.subm else "k2s2")
        self._finish(kind, exp, rows, out, bias, residual, act, feats.shape[0], feats.shape[1], dataflow)
        return out
