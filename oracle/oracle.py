"""CPU oracle for the sparse-convolution hot path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  Nothing in ``pcengine_amd`` does.

It restates, in closed form with numpy, what the reference computes on the GPU:

* packed codes / strides                    script/utils.py:116-138, 233-242
* kernel offsets d(kp)                      backend/hash.cuh:138-149 (submanifold),
                                            backend/hash.cuh:232-237 (strided)
* output coordinates of a strided conv      backend/hash.cuh:585-608, backend/hash.cu:141-173,
                                            script/spconv.py:354-360
* kernel map in canonical (kp, input) order backend/hash.cuh:265-419, script/spconv.py:370-372
* kpos / qkpos                              backend/hash.cuh:478-497
* CSR-coded map for gather-GEMM-scatter     backend/hash.cuh:7-9,97-260,422-437, backend/hash.cu:210-243
* forward values                            backend/spconv.cu:224-398 (centre GEMM + per-offset
                                            gather-matmul-scatter), script/spconv.py:236-253 (transposed)

Pinning (none of this is "parity unpinned"):  the reference ships no golden
vectors, so every function is pinned by tests/test_oracle.py against
(a) an O(N^2) brute force over coordinate tuples, (b) the literal sequential
restatement of the reference kernels in oracle/ref_literal.c (hash with step-97
probing and equality on the reference's linear hash value), and (c) dense
``torch.nn.functional.conv3d`` / ``conv_transpose3d`` on densified small clouds.
Where the reference leaves an order to atomic timing (rank of a pair inside an
offset, backend/hash.cuh:163) the oracle fixes it to the (kp, input row) order
that the reference's own fetch-on-demand compaction produces.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import numpy as np

try:                                   # only used to add rows quickly; the sums are the same
    import scipy.sparse as _sp
except ImportError:                    # pragma: no cover
    _sp = None


def _add_rows(out: np.ndarray, rows: np.ndarray, values: np.ndarray) -> None:
    """out[rows[j]] += values[j] for every j (rows may repeat): ``np.add.at``, or the product with the 0/1
    selection matrix when scipy is there (the same float64 sums, seconds instead of minutes on 10^6 pairs)."""
    if _sp is None or len(rows) < 64:
        np.add.at(out, rows, values)
        return
    sel = _sp.csr_matrix((np.ones(len(rows)), (rows.astype(np.int64), np.arange(len(rows)))), shape=(out.shape[0], len(rows)))
    out += sel @ values

CODE_A = 94273   # script/utils.py:233-234
CODE_B = 311
CSR_CODE = 1186111   # backend/hash.cuh:7-9
COORD_BOUND = 3259   # backend/hash.cuh:503
QUANTUM = 128        # backend/hash.cu:203-205


def encode3(v: Sequence[int]) -> int:
    return CODE_A * int(v[0]) + CODE_B * int(v[1]) + int(v[2])


def decode3(code: int) -> Tuple[int, int, int]:
    x = code // CODE_A
    y = (code - x * CODE_A) // CODE_B
    return (x, y, code - x * CODE_A - y * CODE_B)


def output_stride(l_stride_code: int, t_stride_code: int, transposed: bool = False) -> int:
    ls, ts = decode3(l_stride_code), decode3(t_stride_code)
    if transposed:
        return encode3([t // l for t, l in zip(ts, ls)])
    return encode3([t * l for t, l in zip(ts, ls)])


def kernel_volume(ks: Sequence[int]) -> int:
    return int(ks[0]) * int(ks[1]) * int(ks[2])


def mid_offset(ks: Sequence[int]) -> int:
    return (ks[0] - 1) // 2 * ks[1] * ks[2] + (ks[1] - 1) // 2 * ks[2] + (ks[2] - 1) // 2


def offsets(ks: Sequence[int], strided: bool) -> np.ndarray:
    """d(kp) as int64 [kv, 3]; kp = (ix*ksy + iy)*ksz + iz."""
    kv = kernel_volume(ks)
    kp = np.arange(kv)
    idx = np.stack([kp // (ks[2] * ks[1]), (kp // ks[2]) % ks[1], kp % ks[2]], axis=1)
    d = idx - (np.asarray(ks) - 1) // 2
    if strided:
        bump = np.array([0 if (k % 2 == 0 or k == 1) else 1 for k in ks])
        d = d + bump
    return d.astype(np.int64)


def pack(coords: np.ndarray) -> np.ndarray:
    """Exact, order-preserving int64 key of (b,x,y,z); valid for |coordinate| < 2**15."""
    c = coords.astype(np.int64)
    off = 1 << 15
    return ((c[:, 0] << 48) | ((c[:, 1] + off) << 32) | ((c[:, 2] + off) << 16) | (c[:, 3] + off))


def ravel_code(q: np.ndarray) -> np.ndarray:
    """Mixed-radix code of integer voxel coordinates after shifting by the per-axis minimum
    (ravel_hash, script/utils.py:18-30): ((x-min_x)*E_y + (y-min_y))*E_z + (z-min_z)."""
    x = (q - q.min(axis=0)).astype(np.uint64)
    ext = x.max(axis=0).astype(np.uint64) + np.uint64(1)
    h = np.zeros(len(x), np.uint64)
    for k in range(x.shape[1] - 1):
        h += x[:, k]
        h *= ext[k + 1]
    return h + x[:, -1]


def sparse_quantize(points: np.ndarray, voxel_size):
    """Voxelisation (sparse_quantize, script/utils.py:33-55): floor(points / voxel) in float64, the
    unique voxels in ascending ravelled-code order, the first point of each (numpy.unique's
    return_index) and the voxel of every point (return_inverse)."""
    q = np.floor(np.asarray(points) / np.asarray(voxel_size, np.float64)).astype(np.int32)
    _, index, inverse = np.unique(ravel_code(q), return_index=True, return_inverse=True)
    return q[index], index, inverse


def ref_linear_hash(coords: np.ndarray) -> np.ndarray:
    """The reference's hash value (backend/hash.cuh:11-15), wrapping uint64 arithmetic."""
    c = coords.astype(np.int64).astype(np.uint64)  # sign extension like (uint64_t)int
    with np.errstate(over="ignore"):
        return (c[:, 0] * np.uint64(23783141) + c[:, 1] * np.uint64(73856093)
                + c[:, 2] * np.uint64(19349669) + c[:, 3] * np.uint64(83492791) + np.uint64(1))


class CoordIndex:
    """Exact membership oracle: sorted packed keys + searchsorted."""

    def __init__(self, coords: np.ndarray):
        keys = pack(coords)
        self.order = np.argsort(keys, kind="stable")
        self.keys = keys[self.order]

    def find(self, q: np.ndarray) -> np.ndarray:
        qk = pack(q)
        pos = np.searchsorted(self.keys, qk)
        pos_c = np.minimum(pos, len(self.keys) - 1)
        hit = (self.keys[pos_c] == qk) if len(self.keys) else np.zeros(len(qk), bool)
        return np.where(hit, self.order[pos_c], -1).astype(np.int64)


def strided_coords_max(cmax: Sequence[int], ks, stride, pad) -> list:
    """script/spconv.py:358-360."""
    return [(int(cmax[i]) + 2 * pad[i] - (ks[i] - 1)) // stride[i] for i in range(3)]


def _trunc_div(a: np.ndarray, b: int) -> np.ndarray:
    return (np.sign(a) * (np.abs(a) // b)).astype(np.int64)


def _trunc_mod(a: np.ndarray, b: int) -> np.ndarray:
    return a - _trunc_div(a, b) * b


def out_coords_strided(coords: np.ndarray, ks, stride, pad, cmin, cmax_out) -> np.ndarray:
    """Generic output-coordinate rule (backend/hash.cuh:585-608) then sort+unique on the
    base-3259 code and decode (backend/hash.cu:153-173).  ``cmax_out`` is the already
    reduced bound of script/spconv.py:358-360."""
    d = offsets(ks, strided=True)
    c = coords.astype(np.int64)
    codes = []
    for kp in range(d.shape[0]):
        cand = c[:, 1:] - d[kp] + np.asarray(pad)
        ok = np.ones(len(c), bool)
        div = np.empty_like(cand)
        for a in range(3):
            div[:, a] = _trunc_div(cand[:, a], stride[a])
            ok &= (div[:, a] >= cmin[a]) & (div[:, a] <= cmax_out[a]) & (_trunc_mod(cand[:, a], stride[a]) == 0)
        code = ((c[:, 0] * COORD_BOUND + div[:, 0]) * COORD_BOUND + div[:, 1]) * COORD_BOUND + div[:, 2]
        codes.append(code[ok])
    u = np.unique(np.concatenate(codes)) if codes else np.zeros(0, np.int64)
    out = np.empty((len(u), 4), np.int64)
    out[:, 3] = u % COORD_BOUND
    u = u // COORD_BOUND
    out[:, 2] = u % COORD_BOUND
    u = u // COORD_BOUND
    out[:, 1] = u % COORD_BOUND
    out[:, 0] = u // COORD_BOUND
    return out.astype(np.int32)


def out_coords_fast_path_literal(coords: np.ndarray, total_stride) -> np.ndarray:
    """The reference's k==stride shortcut exactly as written (backend/hash.cuh:503-529,
    backend/hash.cu:110-139): coordinates floored to a multiple of the stride but NOT
    divided.  It disagrees with the query kernels (which assume divided coordinates), so
    the engine does not use it; kept to document the divergence."""
    c = coords.astype(np.int64)
    s = np.asarray(total_stride)
    f = c[:, 1:] // s * s
    code = ((c[:, 0] * COORD_BOUND + f[:, 0]) * COORD_BOUND + f[:, 1]) * COORD_BOUND + f[:, 2]
    u = np.unique(code)
    out = np.empty((len(u), 4), np.int64)
    out[:, 3] = u % COORD_BOUND
    u //= COORD_BOUND
    out[:, 2] = u % COORD_BOUND
    u //= COORD_BOUND
    out[:, 1] = u % COORD_BOUND
    out[:, 0] = u // COORD_BOUND
    return out.astype(np.int32)


@dataclass
class KernelMap:
    n_in: int
    n_out: int
    kv: int
    subm: bool
    imap: np.ndarray      # int32 [M]  input row of each pair, pairs sorted by (kp, input row)
    omap: np.ndarray      # int32 [M]  output row
    knnz: np.ndarray      # int32 [kv]
    kpos: np.ndarray      # int32 [kv+1]
    qkpos: np.ndarray     # int32 [kv+1]
    out_coords: np.ndarray

    @property
    def M(self) -> int:
        return int(self.kpos[-1])

    @property
    def qsum(self) -> int:
        return int(self.qkpos[-1])


def scans(knnz: np.ndarray, q: int = QUANTUM):
    """backend/hash.cuh:478-497."""
    kpos = np.zeros(len(knnz) + 1, np.int64)
    qkpos = np.zeros(len(knnz) + 1, np.int64)
    kpos[1:] = np.cumsum(knnz)
    qkpos[1:] = np.cumsum((knnz.astype(np.int64) + q - 1) // q * q)
    return kpos.astype(np.int32), qkpos.astype(np.int32)


def kernel_map(in_coords: np.ndarray, ks, stride=(1, 1, 1), pad=(0, 0, 0),
               cmin=(0, 0, 0), cmax=None, subm: Optional[bool] = None) -> KernelMap:
    """Canonical map: for every output row o and offset kp, the input at
    ``o*stride - pad + d(kp)`` (backend/hash.cuh:218-258), centre offset skipped for
    submanifold layers (backend/hash.cuh:146); pairs listed by (kp, input row)."""
    if subm is None:
        subm = tuple(stride) == (1, 1, 1)
    kv = kernel_volume(ks)
    if cmax is None:
        cmax = in_coords[:, 1:].max(axis=0).tolist()
    if subm:
        out_coords = in_coords
        d = offsets(ks, strided=False)
        base = in_coords.astype(np.int64).copy()
    else:
        cmax_out = strided_coords_max(cmax, ks, stride, pad)
        out_coords = out_coords_strided(in_coords, ks, stride, pad, cmin, cmax_out)
        d = offsets(ks, strided=True)
        base = out_coords.astype(np.int64).copy()
        base[:, 1:] = base[:, 1:] * np.asarray(stride) - np.asarray(pad)
    index = CoordIndex(in_coords)
    mid = mid_offset(ks)
    imaps, omaps, knnz = [], [], np.zeros(kv, np.int64)
    for kp in range(kv):
        if subm and kp == mid:
            imaps.append(np.zeros(0, np.int64)); omaps.append(np.zeros(0, np.int64))
            continue
        q = base.copy()
        q[:, 1:] += d[kp]
        i = index.find(q)
        o = np.nonzero(i >= 0)[0]
        i = i[o]
        order = np.argsort(i, kind="stable")
        imaps.append(i[order]); omaps.append(o[order]); knnz[kp] = len(o)
    kpos, qkpos = scans(knnz)
    return KernelMap(n_in=len(in_coords), n_out=len(out_coords), kv=kv, subm=bool(subm),
                     imap=np.concatenate(imaps).astype(np.int32),
                     omap=np.concatenate(omaps).astype(np.int32),
                     knnz=knnz.astype(np.int32), kpos=kpos, qkpos=qkpos,
                     out_coords=out_coords)


def csr_maps(km: KernelMap):
    """CSR-coded view for gather-GEMM-scatter: per row, codes ``kp*1186111 + rank`` in
    ascending kp (backend/hash.cuh:163-166 then backend/hash.cu:210-243), rank = position
    of the pair inside its offset in the canonical order."""
    M = km.M
    kp_of = np.repeat(np.arange(km.kv), km.knnz.astype(np.int64))
    rank = np.arange(M) - km.kpos[:-1].astype(np.int64)[kp_of]
    code = (kp_of * CSR_CODE + rank).astype(np.int64)
    assert km.knnz.max(initial=0) < CSR_CODE

    def one(rows, n):
        cnt = np.bincount(rows, minlength=n)
        ptr = np.zeros(n + 1, np.int64)
        ptr[1:] = np.cumsum(cnt)
        order = np.lexsort((kp_of, rows))
        return ptr.astype(np.int32), code[order].astype(np.int32)

    icsr, icodes = one(km.imap.astype(np.int64), km.n_in)
    ocsr, ocodes = one(km.omap.astype(np.int64), km.n_out)
    return icsr, icodes, ocsr, ocodes


def dense_neighbour_table(km: KernelMap) -> np.ndarray:
    """Output-major table nbr[kp, o] = input row or -1 (the layout of the reference's
    dense fetch-on-demand map, script/spconv.py:345, with the roles of input and output
    swapped); for submanifold layers the centre offset holds the row itself."""
    nbr = -np.ones((km.kv, km.n_out), np.int32)
    kp_of = np.repeat(np.arange(km.kv), km.knnz.astype(np.int64))
    nbr[kp_of, km.omap] = km.imap
    return nbr


def conv_forward(feats: np.ndarray, weight: np.ndarray, km: KernelMap, ks,
                 transposed: bool = False, bias: Optional[np.ndarray] = None) -> np.ndarray:
    """float64 forward: centre GEMM for submanifold layers (backend/spconv.cu:273-298) plus,
    per offset, gather rows by imap, multiply by W[kp], add into rows omap
    (backend/spconv.cuh:427-530).  Transposed: the same pairs with roles swapped
    (script/spconv.py:236-244)."""
    f = feats.astype(np.float64)
    w = weight.astype(np.float64)
    if w.ndim == 2:
        w = w[None]
    src, dst = (km.omap, km.imap) if transposed else (km.imap, km.omap)
    n_dst = km.n_in if transposed else km.n_out
    out = np.zeros((n_dst, w.shape[2]), np.float64)
    if km.subm:
        out += f @ w[mid_offset(ks)]
    for kp in range(km.kv):
        a, b = int(km.kpos[kp]), int(km.kpos[kp + 1])
        if a == b:
            continue
        _add_rows(out, dst[a:b], f[src[a:b]] @ w[kp])
    if bias is not None:
        out += bias.astype(np.float64)
    return out


def conv_backward(feats: np.ndarray, weight: np.ndarray, km: KernelMap, ks, grad_out: np.ndarray,
                  transposed: bool = False):
    """float64 gradients of ``conv_forward`` with respect to features and kernel
    (ConvolutionBackwardD1, backend/spconv.cu:400-629; script/spconv.py:172-201): for every pair
    (src row s, dst row d, offset kp): grad_feats[s] += grad_out[d] @ W[kp]^T and
    grad_W[kp] += feats[s]^T (x) grad_out[d]; the centre offset of a submanifold layer pairs every
    row with itself."""
    f = feats.astype(np.float64)
    w = weight.astype(np.float64)
    g = grad_out.astype(np.float64)
    src, dst = (km.omap, km.imap) if transposed else (km.imap, km.omap)
    gf = np.zeros_like(f)
    gw = np.zeros_like(w)
    if km.subm:
        m = mid_offset(ks)
        gf += g @ w[m].T
        gw[m] += f.T @ g
    for kp in range(km.kv):
        a, b = int(km.kpos[kp]), int(km.kpos[kp + 1])
        if a == b:
            continue
        _add_rows(gf, src[a:b], g[dst[a:b]] @ w[kp].T)
        gw[kp] += f[src[a:b]].T @ g[dst[a:b]]
    return gf, gw


def brute_force_pairs(in_coords: np.ndarray, out_coords: np.ndarray, ks, stride, pad, subm: bool):
    """O(N_in * N_out * kv) definition straight from the geometry; tiny inputs only."""
    d = offsets(ks, strided=not subm)
    mid = mid_offset(ks)
    table = {tuple(int(v) for v in c): i for i, c in enumerate(in_coords)}
    pairs = []
    for kp in range(d.shape[0]):
        if subm and kp == mid:
            continue
        for o, c in enumerate(out_coords):
            q = (int(c[0]),
                 int(c[1]) * stride[0] - pad[0] + int(d[kp, 0]),
                 int(c[2]) * stride[1] - pad[1] + int(d[kp, 1]),
                 int(c[3]) * stride[2] - pad[2] + int(d[kp, 2]))
            i = table.get(q)
            if i is not None:
                pairs.append((kp, i, o))
    pairs.sort()
    return pairs


def rel_l2(a: np.ndarray, b: np.ndarray) -> float:
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    den = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / den) if den > 0 else float(np.linalg.norm(a - b))
