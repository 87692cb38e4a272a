"""Torch-facing wrappers over the C ABI.

Two layers live here:

* ``build_kernel_map`` / ``conv_forward`` / ``dense_forward`` — what this package's own front
  end (spconv.py) calls: one native call per map, one per convolution.
* ``mapping_d1_cuda``, ``mapping_d2_cuda``, ``conv_fwd_d1_cuda``, ``conv_fwd_d2_cuda``,
  ``conv_bwd_d1_cuda`` — the five names of the reference's pybind module
  (backend/pybind_cuda.cpp:8-14) with the reference's argument order, so that code written
  against ``PCEngine.backend`` keeps working.

Torch is used for device memory and the current stream only.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import Geom, DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS, DATAFLOW_OSO, PCE_F16, PCE_F32, QUANTUM, CSR_CODE

CODE_A, CODE_B = 94273, 311  # packed 3-vectors, script/utils.py:233-242


def decode3(code: int) -> Tuple[int, int, int]:
    x = code // CODE_A
    y = (code - x * CODE_A) // CODE_B
    return (x, y, code - x * CODE_A - y * CODE_B)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device) -> int:
    if _arena is not None and _arena.stream_device == device:      # inside allocate_from: looked up once per forward
        return _arena.stream
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)       # the handle of torch's current stream without a Stream object (4 us per layer)
    return torch.cuda.current_stream(device).cuda_stream


def _require_cuda(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU: pcengine_amd has no CPU compute path")


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return PCE_F16
    if t.dtype == torch.float32:
        return PCE_F32
    raise TypeError(f"features must be float16 or float32, got {t.dtype}")


def _mid(ks: Sequence[int]) -> int:
    return (ks[0] - 1) // 2 * ks[1] * ks[2] + (ks[1] - 1) // 2 * ks[2] + (ks[2] - 1) // 2


class _Cut:
    """A per-pair array of a map: allocated for the largest possible pair count and cut to the real one on first
    use (a network reads a few of the six arrays of each of its maps; cutting all of them up front is Python time
    the host spends before the first convolution is queued)."""

    def __init__(self, optional: bool, pairs: bool = False):
        self.optional = optional
        self.pairs = pairs       # a pair list: a map built without them (has_pairs False) builds them on first read

    def __set_name__(self, owner, name):
        self.slot = "_cut_" + name

    def __get__(self, obj, owner=None):
        if obj is None:
            if self.optional:
                return None              # the dataclass default
            raise AttributeError         # a required field: no default
        if self.pairs and not obj.__dict__.get("has_pairs", True):
            ensure_pairs(obj)
        v = obj.__dict__.get(self.slot)
        if isinstance(v, tuple):
            if len(v) == 2:              # (array at capacity, count)
                v = v[0][:v[1]]
            else:                        # (int32 view of an arena, first element, count[, shape]): a map of a PyramidPlan
                t = v[0][v[1]:v[1] + v[2]]
                v = t.view(v[3]) if len(v) > 3 else t
            obj.__dict__[self.slot] = v
        return v

    def __set__(self, obj, value):
        obj.__dict__[self.slot] = value


@dataclass
class KernelMap:
    """Kernel map of one (kernel size, tensor stride, layer stride) key.

    Pair lists are in (offset, input row) order.  Indexing and ``len`` reproduce the list the
    reference stores in ``spTensor.kmaps`` (script/spconv.py:382, 431): six entries for the
    fetch-on-demand map, eight when the CSR view has been built.
    """
    ks: Tuple[int, int, int]
    stride: Tuple[int, int, int]
    pad: Tuple[int, int, int]
    subm: bool
    n_in: int
    n_out: int
    kv: int
    M: int
    qsum: int
    imap: torch.Tensor = _Cut(False, pairs=True)
    omap: torch.Tensor = _Cut(False, pairs=True)
    knnz: torch.Tensor = _Cut(False)
    kpos: torch.Tensor = _Cut(False)
    qkpos: torch.Tensor = _Cut(False)
    out_coords: torch.Tensor = _Cut(False)
    nbr_out: Optional[torch.Tensor] = _Cut(True)
    nbr_in: Optional[torch.Tensor] = _Cut(True)
    icsr: Optional[torch.Tensor] = _Cut(True)
    icode: Optional[torch.Tensor] = _Cut(True)
    ocsr: Optional[torch.Tensor] = _Cut(True)
    ocode: Optional[torch.Tensor] = _Cut(True)
    islot: Optional[torch.Tensor] = _Cut(True)   # pair -> position of its entry in icode / ocode
    oslot: Optional[torch.Tensor] = _Cut(True)
    route: Optional[torch.Tensor] = None   # routing array of a layer without centre offset (pair_route), built on first use
    route_t: Optional[torch.Tensor] = None # the same for the transposed layer over this map
    order: Optional[torch.Tensor] = _Cut(True)   # rows in neighbour-pattern order and their offset masks (row_order), built on first use
    order_heavy: int = 0                   # how many rows of that order have three neighbours or more (its last part)
    order_nonzero: int = -1                # how many have any neighbour (-1: not known)
    order_single: int = -1                 # how many have exactly one (-1: not known)
    tag: str = "auto"           # 'D1' / 'D2' when the reference's init_tag protocol fixed it
    in_coords: Optional[torch.Tensor] = None
    geom: Optional[Geom] = None
    knnz_host: list = field(default_factory=list)
    kpos_host: object = None     # ctypes int32 arrays (kv+1) mirrored on the host by the map build's one read-back
    qkpos_host: object = None
    has_pairs: bool = True       # False: built as neighbour table, row order and counts only (want_pairs=False)
    batchsize: int = 0           # the batch count the build was given (0: none)

    @property
    def has_csr(self) -> bool:
        return self.icsr is not None

    def device_tensors(self):
        """Tensors that cover the device allocations this map reads (views share them): what another stream has to
        be told about (``Tensor.record_stream``) before it uses a map whose memory was allocated on this one."""
        pair_arrays = self.__dict__.get("_cut_imap")
        first = pair_arrays[0] if isinstance(pair_arrays, tuple) else pair_arrays     # (for a planned map: the arena)
        arena = self.__dict__.get("_arena")
        if arena is not None:
            return [t for t in (arena, self.route, self.route_t) if t is not None]
        return [t for t in (first, self.knnz, self.out_coords, self.nbr_out, self.nbr_in, self.icsr, self.route, self.route_t)
                if t is not None]

    def _as_list(self):
        if self.tag == "D1" and self.has_csr:
            return [self.icode, self.ocode, self.icsr, self.ocsr, self.kpos, self.qkpos, self.qsum, (self.n_in, self.n_out)]
        return [self.imap, self.omap, self.kpos, self.qkpos, self.qsum, (self.n_in, self.n_out)]

    def __len__(self):
        return len(self._as_list())

    def __getitem__(self, i):
        return self._as_list()[i]


@dataclass
class PendingMap:
    """A map build whose kernels are queued but whose counts have not been read back yet."""
    out_coords: torch.Tensor
    finish: object      # () -> KernelMap, valid after the stream of the build has been synchronised


def strided_coords_max(cmax, ks, stride, pad):
    """script/spconv.py:358-360."""
    return [(int(cmax[a]) + 2 * pad[a] - (ks[a] - 1)) // stride[a] for a in range(3)]


def build_out_coords(in_coords: torch.Tensor, geom: Geom, batchsize: int = 0) -> torch.Tensor:
    """Sorted unique output coordinates of a strided layer (one host sync for the count).

    ``batchsize`` > 0 bounds the batch indices and lets the library use its occupancy-bitmap path;
    a cloud that holds a larger batch index than announced is redone without the bound."""
    lib = _lib.load()
    _require_cuda(in_coords, "coords")
    n_in = in_coords.shape[0]
    s = _stream(in_coords.device)
    for n_batch in ((int(batchsize), 0) if batchsize > 0 else (0,)):
        ws_bytes = lib.pce_outcoords_workspace_bytes(n_in, geom, n_batch)
        if ws_bytes < 0:
            _lib.check(_lib.PCE_EINVAL)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=in_coords.device)
        n_out = _lib.c_int64(0)
        rc = lib.pce_outcoords_build(in_coords.data_ptr(), n_in, geom, n_batch, ws.data_ptr(), ws_bytes, n_out, s)
        if rc == _lib.PCE_EINVAL and n_batch > 0 and b"n_batch" in lib.pce_last_error():
            continue
        _lib.check(rc)
        out = torch.empty((n_out.value, 4), dtype=torch.int32, device=in_coords.device)
        _lib.check(lib.pce_outcoords_emit(ws.data_ptr(), n_in, geom, n_batch, n_out.value, _ptr(out), s))
        return out


CHAIN_NOT_APPLICABLE = 100   # PCE_CHAIN_NOT_APPLICABLE
MAX_CHAIN = 8                # PCE_MAX_CHAIN


def build_out_coords_chain(in_coords: torch.Tensor, geoms: Sequence[Geom], batchsize: int) -> Optional[List[torch.Tensor]]:
    """Output coordinates of several strided layers in a row (each reads what the one before it wrote) with one
    wait of the host, or None where that does not apply (a level too large or too empty for the occupancy bitmap,
    no batch count, a batch index beyond it): the caller then builds level by level."""
    lib = _lib.load()
    _require_cuda(in_coords, "coords")
    levels = len(geoms)
    if levels < 1 or levels > MAX_CHAIN or batchsize <= 0:
        return None
    n_in = in_coords.shape[0]
    garr = (Geom * levels)(*geoms)
    ws_bytes, cap = (_lib.c_int64 * levels)(), (_lib.c_int64 * levels)()
    rc = lib.pce_outcoords_chain_plan(n_in, levels, garr, int(batchsize), ws_bytes, cap)
    if rc == CHAIN_NOT_APPLICABLE:
        return None
    _lib.check(rc)
    # workspaces and coordinate buffers of all levels in one allocation, each on a 256-byte boundary
    sizes = []
    for l in range(levels):
        for n in ((ws_bytes[l] + 3) // 4, 4 * cap[l]):
            sizes += [n, -n % 64]
    pieces = torch.empty(sum(sizes), dtype=torch.int32, device=in_coords.device).split_with_sizes(sizes)
    ws = (_lib.ctypes.c_void_p * levels)(*[pieces[4 * l].data_ptr() for l in range(levels)])
    outs = (_lib.ctypes.c_void_p * levels)(*[pieces[4 * l + 2].data_ptr() for l in range(levels)])
    n_out = (_lib.c_int64 * levels)()
    rc = lib.pce_outcoords_chain(in_coords.data_ptr(), n_in, levels, garr, int(batchsize), ws, ws_bytes, outs, n_out,
                                 _stream(in_coords.device))
    if rc == _lib.PCE_EINVAL and b"n_batch" in lib.pce_last_error():
        return None
    _lib.check(rc)
    return [pieces[4 * l + 2][:4 * n_out[l]].view(n_out[l], 4) for l in range(levels)]


def voxelize(points: torch.Tensor, voxel_size, batch_index: int = 0, return_index: bool = False,
             return_inverse: bool = False):
    """Voxelisation on the GPU (sparse_quantize of script/utils.py:33-55): ``points`` [P,3] float32 or
    float64 on the device -> coords int32 [V,4] = (batch_index, x, y, z) of the unique voxels in
    ascending (x,y,z) order, optionally the first point of every voxel (int32 [V]) and the voxel of
    every point (int32 [P]).  Also returns the integer coordinate bounds (min, max) as lists."""
    lib = _lib.load()
    _require_cuda(points, "points")
    if points.dim() != 2 or points.shape[1] != 3 or points.dtype not in (torch.float32, torch.float64):
        raise ValueError("points must be float32 or float64 [P, 3]")
    points = points.contiguous()
    n = points.shape[0]
    if n == 0:
        raise ValueError("no points to voxelise")
    if isinstance(voxel_size, (int, float)):
        voxel_size = (voxel_size,) * 3
    vs = (_lib.ctypes.c_double * 3)(*[float(v) for v in voxel_size])
    dev = points.device
    s = _stream(dev)
    ws_bytes = lib.pce_voxelize_workspace_bytes(n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    n_vox = _lib.c_int64(0)
    cmin, cmax = (_lib.c_int32 * 3)(), (_lib.c_int32 * 3)()
    dt = _lib.PCE_F32 if points.dtype == torch.float32 else _lib.PCE_F64
    _lib.check(lib.pce_voxelize(points.data_ptr(), dt, n, vs, ws.data_ptr(), ws_bytes, n_vox, cmin, cmax, s))
    v = n_vox.value
    coords = torch.empty((v, 4), dtype=torch.int32, device=dev)
    index = torch.empty(v, dtype=torch.int32, device=dev) if return_index else None
    inverse = torch.empty(n, dtype=torch.int32, device=dev) if return_inverse else None
    _lib.check(lib.pce_voxelize_emit(ws.data_ptr(), n, v, cmin, cmax, int(batch_index), coords.data_ptr(), _ptr(index),
                                     _ptr(inverse), s))
    outs = [coords]
    if return_index:
        outs.append(index)
    if return_inverse:
        outs.append(inverse)
    outs.append((list(cmin), list(cmax)))
    return tuple(outs)


class _MapJob:
    """One kernel-map build between its preparation (outputs allocated, arguments laid out) and the
    read-back of its counts."""

    def __init__(self, in_coords, ks, stride, pad, cmin, cmax_out, subm, want_csr, want_nbr_out, want_nbr_in,
                 out_coords, batchsize, want_order=None, want_pairs=True):
        lib = _lib.load()
        _require_cuda(in_coords, "coords")
        if in_coords.dtype != torch.int32 or in_coords.dim() != 2 or in_coords.shape[1] != 4:
            raise ValueError("coords must be int32 [N, 4] = (b, x, y, z)")
        in_coords = in_coords.contiguous()
        dev = in_coords.device
        n_in = in_coords.shape[0]
        kv = int(ks[0]) * int(ks[1]) * int(ks[2])
        geom = Geom.make(ks, stride, pad, cmin, cmax_out, subm)
        if subm:
            out_coords = in_coords
        elif out_coords is None:
            out_coords = build_out_coords(in_coords, geom, batchsize)
        n_out = out_coords.shape[0]
        if n_in == 0 or n_out == 0:
            raise ValueError(f"empty sparse tensor (n_in={n_in}, n_out={n_out})")
        self.args = (tuple(ks), tuple(stride), tuple(pad), list(cmin), list(cmax_out), bool(subm))
        self.in_coords, self.out_coords, self.geom = in_coords, out_coords, geom
        self.n_in, self.n_out, self.kv, self.want_csr, self.dev = n_in, n_out, kv, bool(want_csr), dev
        self.meta_len = kv + 2 * (kv + 1) + 8      # knnz | kpos | qkpos | status (4 words, then the heavy rows of the order)
        # the row order of the ordered output-stationary dataflow comes with every submanifold map, and every strided
        # map of at most 8 offsets (the layers the selector gives to that dataflow), that has the output-major table
        # it is derived from (three launches per batch of maps, 2 n + 8192 ints)
        if want_order is None:
            want_order = (subm or kv <= 8) and want_nbr_out
        self.want_order = bool(want_order) and want_nbr_out and kv <= 31
        # the batch count lets the library index sorted coordinates by column instead of hashing them; a build that
        # finds them unsorted, or outside the box the geometry states, is redone through the hash table (finish)
        self.n_batch, self.no_grid = max(int(batchsize), 0), False
        # a caller that reads only the neighbour table, the row order and the counts (the output-stationary
        # dataflows) waives the pair lists; the library then skips them where it can (3x3x3 submanifold map over the
        # column grid) and says so in its status word 5
        self.table_only = not want_pairs and not want_csr and want_nbr_out and not want_nbr_in
        self.ws_bytes = lib.pce_kmap_workspace_bytes_grid(n_in, n_out, geom, self.n_batch, int(want_csr))
        if self.ws_bytes < 0:
            _lib.check(_lib.PCE_EINVAL)
        # the arrays of the build, in int32 elements: one allocation holds those of every job of a batch (place)
        cap = kv * n_in
        self.want = [("ws", (self.ws_bytes + 3) // 4), ("imap", cap), ("omap", cap)]
        if want_nbr_out:
            self.want.append(("nbr_out", kv * n_out))
        if want_nbr_in:
            self.want.append(("nbr_in", kv * n_in))
        if self.want_order:
            self.want.append(("order", lib.pce_row_order_elems(n_out)))
        if want_csr:
            self.want += [("icsr", n_in + 1), ("ocsr", n_out + 1), ("icode", cap), ("ocode", cap), ("islot", cap), ("oslot", cap)]
        self.ws = self.imap = self.omap = self.nbr_out = self.nbr_in = self.order = None
        self.icsr = self.ocsr = self.icode = self.ocode = self.islot = self.oslot = None

    @staticmethod
    def place(jobs) -> None:
        """One device allocation for the arrays of all `jobs`, each array on a 256-byte boundary."""
        jobs = [j for j in jobs if j.ws is None]
        if not jobs:
            return
        sizes = []
        for j in jobs:
            for _, n in j.want:
                sizes += [n, -n % 64]
        arena = torch.empty(sum(sizes), dtype=torch.int32, device=jobs[0].dev)
        pieces = arena.split_with_sizes(sizes)
        k = 0
        for j in jobs:
            for name, _ in j.want:
                setattr(j, name, pieces[k])
                k += 2

    def problem(self, meta: torch.Tensor) -> "_lib.KmapProblem":
        """``meta`` is this job's zeroed slice of the batch's count tensor."""
        kv = self.kv
        self.knnz, self.kpos, self.qkpos = meta[:kv], meta[kv:2 * kv + 1], meta[2 * kv + 1:3 * kv + 2]
        status = meta[3 * kv + 2:]
        p = _lib.KmapProblem()
        p.in_coords, p.n_in = self.in_coords.data_ptr(), self.n_in
        p.out_coords, p.n_out = self.out_coords.data_ptr(), self.n_out
        p.geom = self.geom
        p.ws, p.ws_bytes = self.ws.data_ptr(), self.ws_bytes
        p.imap, p.omap = self.imap.data_ptr(), self.omap.data_ptr()
        p.knnz, p.kpos, p.qkpos = self.knnz.data_ptr(), self.kpos.data_ptr(), self.qkpos.data_ptr()
        p.icsr, p.icode, p.ocsr, p.ocode = _ptr(self.icsr), _ptr(self.icode), _ptr(self.ocsr), _ptr(self.ocode)
        p.islot, p.oslot = _ptr(self.islot), _ptr(self.oslot)
        p.nbr_out, p.nbr_in = _ptr(self.nbr_out), _ptr(self.nbr_in)
        p.status = status.data_ptr()
        p.n_batch = self.n_batch
        p.flags = (_lib.KMAP_NO_GRID if self.no_grid else 0) | (_lib.KMAP_TABLE_ONLY if self.table_only else 0)
        p.order = _ptr(self.order)
        return p

    def finish(self, host: list) -> KernelMap:
        kv, M = self.kv, None
        st = host[3 * kv + 2:]
        if st[0]:
            raise ValueError(f"a coordinate is outside the supported range (|c| < {32000}, batch < 32768)")
        if st[1]:
            raise _lib.PCEError("hash table exhausted while building the kernel map")
        if self.want_csr and st[2]:
            raise OverflowError(f"an offset holds >= {CSR_CODE} pairs: the CSR code of the gather-GEMM-scatter map overflows")
        if st[3] and not self.no_grid:
            # unsorted coordinates, or some outside the stated bounds / batch count: the same build through the hash table
            self.no_grid = True
            return build_kernel_maps([self])[0]
        M, qsum = host[2 * kv], host[3 * kv + 1]
        ks, stride, pad, cmin, cmax_out, subm = self.args
        cut = lambda t: None if t is None else (t, M)     # cut to the pair count when first read
        km = KernelMap(ks=ks, stride=stride, pad=pad, subm=subm, n_in=self.n_in, n_out=self.n_out, kv=kv,
                       M=M, qsum=qsum, imap=cut(self.imap), omap=cut(self.omap), knnz=self.knnz, kpos=self.kpos,
                       qkpos=self.qkpos, out_coords=self.out_coords, nbr_out=self.nbr_out, nbr_in=self.nbr_in,
                       icsr=self.icsr, ocsr=self.ocsr, icode=cut(self.icode), ocode=cut(self.ocode),
                       islot=cut(self.islot), oslot=cut(self.oslot), in_coords=self.in_coords, geom=self.geom,
                       knnz_host=host[:kv], order=self.order, order_heavy=st[4] if self.order is not None else 0,
                       has_pairs=not st[5], batchsize=self.n_batch, order_nonzero=st[6] if self.order is not None else -1,
                       order_single=st[7] if self.order is not None else -1)
        km._cmin, km._cmax = cmin, cmax_out
        km.kpos_host = (_lib.c_int32 * (kv + 1))(*host[kv:2 * kv + 1])
        km.qkpos_host = (_lib.c_int32 * (kv + 1))(*host[2 * kv + 1:3 * kv + 2])
        return km


KMAP_MAX_BATCH = 16


def prepare_map(in_coords: torch.Tensor, ks, stride, pad, cmin, cmax_out, subm: bool, want_csr: bool = False,
                want_nbr_out: bool = True, want_nbr_in: bool = False, out_coords: Optional[torch.Tensor] = None,
                batchsize: int = 0, want_order: Optional[bool] = None, want_pairs: bool = True) -> _MapJob:
    """First half of a map build: the output coordinates of a strided layer (``.out_coords``, final)
    and the output buffers.  ``build_kernel_maps`` takes the result in place of a request."""
    return _MapJob(in_coords, ks, stride, pad, cmin, cmax_out, subm, want_csr, want_nbr_out, want_nbr_in, out_coords,
                   batchsize, want_order, want_pairs)


def build_kernel_maps(requests: List[dict], defer: bool = False):
    """Build the kernel maps of several layers with the launches of one build.

    Every request holds the keyword arguments of ``build_kernel_map`` (without ``defer``), or is the
    result of ``prepare_map`` on them.  The
    output coordinates of strided layers are computed first, request by request; the builds then
    run as batches of up to ``KMAP_MAX_BATCH`` problems, each stage one launch over the whole
    batch, and the counts of all maps come back in one copy.  ``defer=True`` returns
    ``PendingMap`` objects whose ``finish()`` may be called once the stream has been synchronised."""
    lib = _lib.load()
    jobs = [r if isinstance(r, _MapJob) else prepare_map(**r) for r in requests]
    if not jobs:
        return []
    dev = jobs[0].dev
    if any(j.dev != dev for j in jobs):
        raise ValueError("the maps of one batch live on one device")
    s = _stream(dev)
    starts = [0]
    for j in jobs:
        starts.append(starts[-1] + j.meta_len)
    # the counts and status words of every map in one tensor: a single device->host copy reads them all
    meta = torch.zeros(starts[-1], dtype=torch.int32, device=dev)
    _MapJob.place(jobs)
    for b0 in range(0, len(jobs), KMAP_MAX_BATCH):
        chunk = jobs[b0:b0 + KMAP_MAX_BATCH]
        probs = (_lib.KmapProblem * len(chunk))(*[j.problem(meta[starts[b0 + k]:starts[b0 + k + 1]])
                                                  for k, j in enumerate(chunk)])
        _lib.check(lib.pce_kmap_build_batch(probs, len(chunk), s))
    if defer:
        # the counts travel to pinned host memory behind the kernels; the caller synchronises the stream
        # once and then calls finish() on each
        meta_host = torch.empty(meta.shape, dtype=torch.int32, pin_memory=True)
        meta_host.copy_(meta, non_blocking=True)
        cache = {}

        def finisher(k):
            def fin():
                if "host" not in cache:
                    cache["host"] = meta_host.tolist()
                return jobs[k].finish(cache["host"][starts[k]:starts[k + 1]])
            return fin
        return [PendingMap(out_coords=j.out_coords, finish=finisher(k)) for k, j in enumerate(jobs)]
    host = meta.cpu().tolist()   # the one synchronisation of the builds
    return [j.finish(host[starts[k]:starts[k + 1]]) for k, j in enumerate(jobs)]


def build_kernel_map(in_coords: torch.Tensor, ks, stride, pad, cmin, cmax_out, subm: bool,
                     want_csr: bool = False, want_nbr_out: bool = True, want_nbr_in: bool = False,
                     out_coords: Optional[torch.Tensor] = None, batchsize: int = 0, defer: bool = False,
                     want_order: Optional[bool] = None, want_pairs: bool = True):
    """Hash the output coordinates, probe every (input row, offset) and emit the canonical map.

    ``cmax_out`` is the bound on output coordinates (already reduced for strided layers).
    ``defer=True`` returns a ``PendingMap`` instead of waiting for the pair counts: its output
    coordinates are final, ``finish()`` yields the ``KernelMap`` once the stream has been
    synchronised.  ``want_pairs=False``: the caller reads the neighbour table, the row order and the counts only
    (``KernelMap.has_pairs`` tells whether the build skipped the pair lists; reading ``imap`` / ``omap`` of such a
    map builds them then)."""
    return build_kernel_maps([dict(in_coords=in_coords, ks=ks, stride=stride, pad=pad, cmin=cmin, cmax_out=cmax_out,
                                   subm=subm, want_csr=want_csr, want_nbr_out=want_nbr_out, want_nbr_in=want_nbr_in,
                                   out_coords=out_coords, batchsize=batchsize, want_order=want_order,
                                   want_pairs=want_pairs)], defer=defer)[0]


class ForwardArena:
    """One device allocation the layer outputs of a forward pass are cut from, in the order the layers ask
    (``allocate_from``), plus one staging buffer all layers share (the reference's ``spTensor.buffer``,
    script/sptensor.py:63-78).  The first forward over a cloud measures what the network asks for; the arena is then
    sized with headroom, and forwards that fit it allocate nothing.  A request that does not fit (a larger cloud) is
    served by ``torch.empty`` and the arena grows before the next forward.  Tensors cut from it, the network's output
    included, are valid until the next ``begin()``.  ``limit`` bounds the arena; a forward that needs more keeps
    ``torch.empty`` for what does not fit."""

    def __init__(self, device, limit: int = 8 << 30, headroom: float = 1.125):
        self.device, self.limit, self.headroom = torch.device(device), int(limit), headroom
        self.buf = None
        self.off = self.need = 0
        self.scratch = None
        self.stream, self.stream_device = 0, None

    def begin(self) -> None:
        want = min(int(self.need * self.headroom), self.limit)
        if self.need and (self.buf is None or self.buf.numel() < min(self.need, self.limit)):
            self.buf = None        # release before the larger one is taken
            self.buf = torch.empty(want, dtype=torch.uint8, device=self.device)
        self.off = self.need = 0

    def empty(self, shape, dtype, device) -> torch.Tensor:
        shape = (shape,) if isinstance(shape, int) else tuple(shape)
        numel = 1
        for d in shape:
            numel *= int(d)
        nbytes = numel * _ITEMSIZE[dtype]
        start = self.need
        self.need = start + (nbytes + 255) // 256 * 256
        if self.buf is None or self.need > self.buf.numel() or torch.device(device) != self.device:
            return torch.empty(shape, dtype=dtype, device=device)
        return self.buf[start:start + nbytes].view(dtype).view(shape)

    def staging(self, numel: int, dtype, device) -> torch.Tensor:
        """The shared staging buffer, at least ``numel`` elements of ``dtype`` (grown when a layer needs more)."""
        nbytes = int(numel) * _ITEMSIZE[dtype]
        if self.scratch is None or self.scratch.numel() < nbytes or self.scratch.device != torch.device(device):
            self.scratch = None
            self.scratch = torch.empty(int(nbytes * self.headroom) + 256, dtype=torch.uint8, device=device)
        return self.scratch[:nbytes].view(dtype)


_ITEMSIZE = {torch.float16: 2, torch.bfloat16: 2, torch.float32: 4, torch.float64: 8, torch.int32: 4, torch.int64: 8, torch.uint8: 1}
_arena: Optional[ForwardArena] = None


class allocate_from:
    """Context manager: inside it the outputs, routing arrays and staging buffers of the forward operators of this
    module come from ``arena`` (a ``ForwardArena``) and not from ``torch.empty``.  Not for concurrent use."""

    def __init__(self, arena: Optional[ForwardArena]):
        self.arena = arena

    def __enter__(self):
        global _arena
        self.prev, _arena = _arena, None
        if self.arena is not None:
            self.arena.begin()
            # the stream the forward runs on: the current one as the forward starts (a forward that switches streams
            # inside the context is not served)
            self.arena.stream_device = self.arena.device
            self.arena.stream = torch.cuda.current_stream(self.arena.device).cuda_stream
        _arena = self.arena
        return self.arena

    def __exit__(self, *exc):
        global _arena
        _arena = self.prev


def _new(shape, dtype, device) -> torch.Tensor:
    """Uninitialised device memory for an operator's output: from the active arena, else from torch."""
    if _arena is not None:
        return _arena.empty(shape, dtype, device)
    return torch.empty(shape, dtype=dtype, device=device)


def _staging(numel: int, dtype, device) -> torch.Tensor:
    if _arena is not None:
        return _arena.staging(numel, dtype, device)
    return torch.empty(max(int(numel), 1), dtype=dtype, device=device)


class PlanNotApplicable(Exception):
    """The native planner does not take this pyramid (a level that is not a bitmap chain, an unsorted cloud): the
    caller builds map by map."""


class PyramidPlan:
    """All kernel maps of a network on one cloud in ONE device allocation and two library calls
    (``pce_pyramid_plan`` / ``pce_pyramid_build``): the chained output coordinates of the strided levels and every
    requested map, laid out from upper bounds so that nothing is allocated, sized or described by the host between
    the two waits for counts.  ``requests``: (level_in, level_out, ks, stride, pad, cmin, cmax_out, subm, want_csr,
    want_nbr_in, table_only) per map; ``strided``: the geometry of every strided level, in order.  The plan serves
    any cloud of at most ``n_cap`` rows inside the same box; the maps of a build live in the plan's arena and are
    valid until its next build."""

    def __init__(self, n_cap: int, strided: Sequence[Geom], requests: Sequence[tuple], n_batch: int, device):
        lib = _lib.load()
        if lib.pce_pyramid_plan_sizeof() != _lib.ctypes.sizeof(_lib.PyrPlan):
            raise _lib.PCEError("pce_pyr_plan_t of the library and of this binding differ")
        if len(strided) > _lib.PYR_MAX_LEVELS or not 0 < len(requests) <= _lib.PYR_MAX_MAPS or n_batch <= 0:
            raise PlanNotApplicable()
        self.plan = _lib.PyrPlan()
        self.args = []
        reqs = (_lib.PyrRequest * len(requests))()
        for r, (lin, lout, ks, stride, pad, cmin, cmax_out, subm, want_csr, want_nbr_in, table_only) in zip(reqs, requests):
            kv = int(ks[0]) * int(ks[1]) * int(ks[2])
            if kv > 31:
                raise PlanNotApplicable()
            r.level_in, r.level_out = lin, lout
            r.geom = Geom.make(ks, stride, pad, cmin, cmax_out, subm)
            r.want_csr, r.want_nbr_in, r.table_only = int(want_csr), int(want_nbr_in), int(table_only)
            self.args.append((tuple(ks), tuple(stride), tuple(pad), list(cmin), list(cmax_out), bool(subm)))
        garr = (Geom * max(len(strided), 1))(*strided)
        rc = lib.pce_pyramid_plan(int(n_cap), len(strided), garr, int(n_batch), reqs, len(requests), self.plan)
        if rc == CHAIN_NOT_APPLICABLE:
            raise PlanNotApplicable()
        _lib.check(rc)
        self.n_cap, self.n_batch, self.device = int(n_cap), int(n_batch), device
        self.arena = torch.empty(self.plan.arena_bytes, dtype=torch.uint8, device=device)
        self.arena32 = self.arena.view(torch.int32)

    def build(self, in_coords: torch.Tensor):
        """(coordinates of every level, the maps in request order) for one cloud.  Raises ``PlanNotApplicable`` when
        the cloud has more rows than the plan or its rows are not sorted inside the stated box."""
        lib = _lib.load()
        _require_cuda(in_coords, "coords")
        n = in_coords.shape[0]
        if n > self.n_cap or n == 0 or in_coords.dtype != torch.int32 or not in_coords.is_contiguous():
            raise PlanNotApplicable()
        plan = self.plan
        rc = lib.pce_pyramid_build(plan, in_coords.data_ptr(), n, self.arena.data_ptr(), self.arena.numel(), _stream(in_coords.device))
        if rc in (_lib.PYR_UNSORTED, CHAIN_NOT_APPLICABLE) or (rc == _lib.PCE_EINVAL and b"n_batch" in lib.pce_last_error()):
            raise PlanNotApplicable()
        _lib.check(rc)
        a32 = self.arena32
        coords = [in_coords]
        for l in range(1, plan.n_levels + 1):
            nl = plan.level_n[l]
            coords.append(a32[plan.off_coords[l] // 4:plan.off_coords[l] // 4 + 4 * nl].view(nl, 4))
        maps = []
        for i in range(plan.n_maps):
            m, r = plan.map[i], plan.req[i]
            kv, n_in, n_out, M = m.kv, m.n_in, m.n_out, m.n_pairs
            meta = m.meta[:3 * kv + 2 + 8]
            st = meta[3 * kv + 2:]
            off = m.off
            at = lambda a, count: None if off[a] < 0 else (a32, off[a] // 4, count)
            mo = off[_lib.PYR_META] // 4
            has_pairs = not st[5]
            ks, stride, pad, cmin, cmax_out, subm = self.args[i]
            order = at(_lib.PYR_ORDER, lib.pce_row_order_elems(n_out)) if off[_lib.PYR_ORDER] >= 0 else None
            km = KernelMap(ks=ks, stride=stride, pad=pad, subm=subm, n_in=n_in, n_out=n_out, kv=kv, M=M, qsum=m.qsum,
                           imap=at(_lib.PYR_IMAP, M), omap=at(_lib.PYR_OMAP, M), knnz=(a32, mo, kv), kpos=(a32, mo + kv, kv + 1),
                           qkpos=(a32, mo + 2 * kv + 1, kv + 1), out_coords=coords[r.level_out],
                           nbr_out=at(_lib.PYR_NBR_OUT, kv * n_out), nbr_in=at(_lib.PYR_NBR_IN, kv * n_in),
                           icsr=at(_lib.PYR_ICSR, n_in + 1), ocsr=at(_lib.PYR_OCSR, n_out + 1), icode=at(_lib.PYR_ICODE, M),
                           ocode=at(_lib.PYR_OCODE, M), islot=at(_lib.PYR_ISLOT, M), oslot=at(_lib.PYR_OSLOT, M),
                           in_coords=coords[r.level_in], geom=r.geom, knnz_host=meta[:kv], order=order,
                           order_heavy=st[4] if order is not None else 0, has_pairs=has_pairs, batchsize=self.n_batch,
                           order_nonzero=st[6] if order is not None else -1, order_single=st[7] if order is not None else -1)
            km._cmin, km._cmax = cmin, cmax_out
            km.kpos_host = (_lib.c_int32 * (kv + 1))(*meta[kv:2 * kv + 1])
            km.qkpos_host = (_lib.c_int32 * (kv + 1))(*meta[2 * kv + 1:3 * kv + 2])
            km._arena = self.arena
            maps.append(km)
        return coords, maps


def ensure_pairs(km: KernelMap) -> None:
    """Pair lists of a map that was built without them (first use of a dataflow that reads them)."""
    if km.has_pairs:
        return
    km.has_pairs = True          # before the build below reads anything of `km`
    full = build_kernel_map(km.in_coords, km.ks, km.stride, km.pad, km._cmin, km._cmax, km.subm, want_csr=False,
                            want_nbr_out=False, out_coords=km.out_coords, batchsize=km.batchsize)
    km.imap, km.omap = full.imap, full.omap


def ensure_csr(km: KernelMap) -> None:
    """Build the CSR-coded view of an existing map (first use of gather-GEMM-scatter on it)."""
    if km.has_csr:
        return
    full = build_kernel_map(km.in_coords, km.ks, km.stride, km.pad, km._cmin, km._cmax, km.subm, want_csr=True,
                            want_nbr_out=False, out_coords=km.out_coords)
    km.icsr, km.icode, km.ocsr, km.ocode = full.icsr, full.icode, full.ocsr, full.ocode
    km.islot, km.oslot = full.islot, full.oslot
    if not km.has_pairs:
        km.has_pairs = True
        km.imap, km.omap = full.imap, full.omap


def pair_route(km: KernelMap, transposed: bool = False) -> torch.Tensor:
    """Routing array of a layer without centre offset, cached on the map (``pce_pair_route``): the number of output
    rows whose pair count is not one, the destination of every pair (the output row where the pair is the row's
    only one, else ``n_out`` + its partial-row slot) and the list of those rows.  ``transposed``: the array of
    the transposed layer, whose output rows are the map's input rows."""
    route = km.route_t if transposed else km.route
    if route is None:
        ensure_csr(km)
        lib = _lib.load()
        omap, oslot, ocsr, n_out = (km.imap, km.islot, km.icsr, km.n_in) if transposed else (km.omap, km.oslot, km.ocsr, km.n_out)
        elems = lib.pce_pair_route_elems(km.M, n_out)
        route = _new(elems, torch.int32, omap.device)
        _lib.check(lib.pce_pair_route(omap.data_ptr(), oslot.data_ptr(), ocsr.data_ptr(), km.M, n_out,
                                      route.data_ptr(), elems, _stream(omap.device)))
        if transposed:
            km.route_t = route
        else:
            km.route = route
    return route


def row_order(km: KernelMap) -> torch.Tensor:
    """Row order of the ordered output-stationary dataflow (``pce_row_order``), cached on the map: the output rows
    with rows without neighbours first (a submanifold layer has those; the centre offset does not count) and the
    others sorted by the offsets they have."""
    if km.order is None:
        ensure_nbr(km, False)
        lib = _lib.load()
        elems = lib.pce_row_order_elems(km.n_out)
        order = torch.empty(elems, dtype=torch.int32, device=km.nbr_out.device)
        counts = (_lib.c_int64 * 3)()
        _lib.check(lib.pce_row_order(km.nbr_out.data_ptr(), km.kv, km.n_out, _mid(km.ks) if km.subm else -1, order.data_ptr(),
                                     elems, counts, _stream(order.device)))
        km.order, km.order_heavy, km.order_nonzero, km.order_single = order, counts[0], counts[1], counts[2]
    return km.order


_oso_takes_cache = {}


def oso_takes(km: KernelMap, c_in: int, c_out: int, dtype: torch.dtype, transposed: bool = False) -> bool:
    """Layers the ordered output-stationary dataflow takes (``pce_conv_oso_takes``; never a transposed layer)."""
    if transposed or dtype not in (torch.float16, torch.float32):
        return False
    key = (dtype, c_in, c_out, km.kv, km.subm, km.ks)
    ans = _oso_takes_cache.get(key)
    if ans is None:
        code = PCE_F16 if dtype == torch.float16 else PCE_F32
        ans = _oso_takes_cache[key] = bool(_lib.load().pce_conv_oso_takes(code, c_in, c_out, km.kv, _mid(km.ks) if km.subm else -1))
    return ans


def ensure_nbr(km: KernelMap, transposed: bool) -> None:
    if (km.nbr_in if transposed else km.nbr_out) is not None:
        return
    full = build_kernel_map(km.in_coords, km.ks, km.stride, km.pad, km._cmin, km._cmax, km.subm, want_csr=False,
                            want_nbr_out=True, want_nbr_in=True, out_coords=km.out_coords)
    km.nbr_out, km.nbr_in = full.nbr_out, full.nbr_in
    if full.order is not None:
        km.order, km.order_heavy = full.order, full.order_heavy
        km.order_nonzero, km.order_single = full.order_nonzero, full.order_single


def select_dataflow(km: KernelMap, c_in: int, c_out: int, dtype: torch.dtype, transposed: bool = False) -> int:
    lib = _lib.load()
    n_out = km.n_in if transposed else km.n_out
    n_in = km.n_out if transposed else km.n_in
    df = lib.pce_select_dataflow(n_in, n_out, km.M, c_in, c_out, km.kv, _mid(km.ks) if km.subm else -1, int(bool(transposed)),
                                 PCE_F16 if dtype == torch.float16 else PCE_F32)
    if not km.has_pairs and df not in (DATAFLOW_OSO, DATAFLOW_OS):
        # a map built without pair lists (its layers were expected to read the neighbour table only): rather than
        # build them now, the layer takes the table-reading dataflow that is closest (a band of densities where the
        # ordered dataflow is within a tenth of deferred scatter)
        df = DATAFLOW_OSO if oso_takes(km, c_in, c_out, dtype, transposed) else DATAFLOW_OS
    return df


def pack_weights(weight: torch.Tensor) -> Optional[torch.Tensor]:
    """fp16 weights [kv, c_in, c_out] in the order the kernels stage them into LDS (None for fp32).
    At inference the weights are constants: callers pack once and pass the copy along."""
    lib = _lib.load()
    if weight.dtype != torch.float16:
        return None
    _require_cuda(weight, "weight")
    weight = weight.contiguous()
    if weight.dim() == 2:
        weight = weight.unsqueeze(0)
    kv, c_in, c_out = weight.shape
    nbytes = lib.pce_packed_weight_bytes(PCE_F16, kv, c_in, c_out)
    packed = torch.empty(nbytes, dtype=torch.uint8, device=weight.device)
    _lib.check(lib.pce_pack_weights(weight.data_ptr(), PCE_F16, kv, c_in, c_out, packed.data_ptr(), _stream(weight.device)))
    return packed


def _act_code(act) -> Tuple[int, float]:
    """``act``: None, 'relu', or ('leaky_relu', negative_slope) -> (PCE_ACT_*, slope)."""
    if act is None:
        return _lib.ACT_NONE, 0.0
    if act == "relu":
        return _lib.ACT_RELU, 0.0
    if isinstance(act, tuple) and len(act) == 2 and act[0] == "leaky_relu":
        return _lib.ACT_LEAKY_RELU, float(act[1])
    raise ValueError(f"unknown activation {act!r}")


def _row_stride(t: torch.Tensor) -> int:
    """Elements between consecutive rows of a feature matrix the kernels can read or write in place: 0 for a dense
    matrix, the stride for a column slice of a wider row-major matrix (16-byte aligned, stride a multiple of 8
    elements), -1 for any other layout (the caller makes a dense copy)."""
    if t.dim() != 2:
        return -1
    if t.is_contiguous():
        return 0
    if (t.stride(1) == 1 and t.stride(0) > t.shape[1] and t.stride(0) % 8 == 0 and t.shape[1] % 8 == 0
            and t.data_ptr() % 16 == 0):
        return t.stride(0)
    return -1


def _epilogue(feats: torch.Tensor, n_out: int, c_out: int, bias, residual, act, ld_in: int = 0, ld_out: int = 0):
    """(ctypes struct or None, tensors to keep alive) for ``out = act(conv + bias + residual)``.
    ``act``: None, 'relu', or ('leaky_relu', negative_slope).  ``ld_in`` / ``ld_out``: row strides of a
    feature matrix and an output that are column slices of wider matrices (0: dense)."""
    if bias is None and residual is None and act is None and not ld_in and not ld_out:
        return None, ()
    e = _lib.Epilogue()
    e.ld_in, e.ld_out = ld_in, ld_out
    keep = []
    if bias is not None:
        if bias.requires_grad or bias.dtype != feats.dtype or bias.device != feats.device or not bias.is_contiguous():
            bias = bias.detach().to(device=feats.device, dtype=feats.dtype).contiguous()
        if bias.numel() != c_out:
            raise ValueError(f"bias has {bias.numel()} elements, the layer has {c_out} output channels")
        e.bias = bias.data_ptr()
        keep.append(bias)
    if residual is not None:
        _require_cuda(residual, "residual")
        if residual.shape != (n_out, c_out) or residual.dtype != feats.dtype:
            raise ValueError(f"residual must be [{n_out}, {c_out}] {feats.dtype}")
        residual = residual.contiguous()
        e.residual = residual.data_ptr()
        keep.append(residual)
    e.act, e.slope = _act_code(act)
    return e, keep


def dense_forward(feats: torch.Tensor, weight: torch.Tensor, packed: Optional[torch.Tensor] = None,
                  bias: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None, act=None) -> torch.Tensor:
    """act(feats @ weight + bias + residual) for the 1x1 stride-1 layer (script/spconv.py:297-304)."""
    lib = _lib.load()
    _require_cuda(feats, "feats")
    feats = feats.contiguous()
    weight = weight.contiguous()
    if feats.shape[1] != weight.shape[0]:
        raise ValueError("Input feature size and kernel size mismatch")
    out = _new((feats.shape[0], weight.shape[1]), feats.dtype, feats.device)
    epi, _keep = _epilogue(feats, feats.shape[0], weight.shape[1], bias, residual, act)
    _lib.check(lib.pce_conv_fwd_dense(feats.data_ptr(), weight.data_ptr(), _ptr(packed), out.data_ptr(), _dtype_code(feats),
                                      feats.shape[0], feats.shape[1], weight.shape[1], epi, _stream(feats.device)))
    return out


def conv_forward(feats: torch.Tensor, weight: torch.Tensor, km: KernelMap, dataflow: int, transposed: bool = False,
                 buffer: Optional[torch.Tensor] = None, packed: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                 residual: Optional[torch.Tensor] = None, act=None, route_single_pairs: bool = True) -> torch.Tensor:
    """One forward convolution over an existing map with the chosen dataflow:
    ``act(conv(feats) + bias + residual)``, the last three optional and applied inside the kernels
    (``act``: None, 'relu' or ('leaky_relu', slope)).

    ``out`` (optional) is a preallocated [n_out, c_out] tensor of the feature dtype: with it, a
    large enough ``buffer`` and a dataflow other than plain fetch-on-demand the call allocates
    nothing, so a loop of layers can be captured into a HIP graph."""
    lib = _lib.load()
    _require_cuda(feats, "feats")
    # the deferred-scatter and output-stationary kernels take column slices of wider matrices in place (the halves
    # of a concatenated skip connection); everything else gets dense rows
    strided_ok = dataflow in (DATAFLOW_FDS, DATAFLOW_OS, DATAFLOW_OSO)
    ld_in = _row_stride(feats) if strided_ok else -1
    if ld_in < 0:
        feats, ld_in = feats.contiguous(), 0
    weight = weight.contiguous()
    if weight.dim() == 2:
        weight = weight.unsqueeze(0)
    if feats.dtype != weight.dtype:
        raise TypeError(f"features are {feats.dtype} but the kernel is {weight.dtype}")
    kv, c_in, c_out = weight.shape
    if feats.shape[1] != c_in:
        raise ValueError("Input feature size and kernel size mismatch")   # backend/spconv.cu:38-40
    if kv != km.kv:
        raise ValueError(f"kernel volume {kv} does not match the map ({km.kv})")
    if transposed and km.subm and all(k % 2 == 1 for k in km.ks):
        # a submanifold map with odd kernel sizes is its own mirror image: pair (i, o, kp) exists iff
        # (o, i, kv-1-kp) does, so the transposed layer is the plain layer with the offsets of the kernel reversed
        weight, packed, transposed = weight.flip(0).contiguous(), None, False
        packed = pack_weights(weight)
    n_in, n_out = (km.n_out, km.n_in) if transposed else (km.n_in, km.n_out)
    if feats.shape[0] != n_in:
        raise ValueError(f"features have {feats.shape[0]} rows, the map expects {n_in}")
    dt = _dtype_code(feats)
    dev = feats.device
    s = _stream(dev)
    mid = _mid(km.ks) if km.subm else -1
    ld_out, slice_out = 0, None
    if out is None:
        out = _new((n_out, c_out), feats.dtype, dev)
    elif out.shape != (n_out, c_out) or out.dtype != feats.dtype or out.device != dev:
        raise ValueError(f"out must be a [{n_out}, {c_out}] {feats.dtype} tensor on {dev}")
    elif not out.is_contiguous():
        ld_out = _row_stride(out)
        if ld_out < 0:
            raise ValueError("out must be contiguous or a column slice of a row-major matrix (16-byte aligned, "
                             "row stride and width multiples of 8 elements)")
        if not strided_ok:       # this dataflow stores dense rows: they are copied into the slice afterwards
            slice_out, ld_out = out, 0
            out = _new((n_out, c_out), feats.dtype, dev)
    epi, _keep = _epilogue(feats, n_out, c_out, bias, residual, act, ld_in, ld_out)
    if dataflow == DATAFLOW_FOD:
        imap, omap = (km.omap, km.imap) if transposed else (km.imap, km.omap)
        ws_bytes = lib.pce_conv_fod_workspace_bytes(n_out, c_out, dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
        _lib.check(lib.pce_conv_fwd_fod(feats.data_ptr(), weight.data_ptr(), _ptr(packed), out.data_ptr(), dt, n_in, n_out,
                                        c_in, c_out, kv, mid, imap.data_ptr(), omap.data_ptr(), km.kpos.data_ptr(),
                                        km.qkpos.data_ptr(), km.qsum, _ptr(ws), ws_bytes, epi, s))
    elif dataflow == DATAFLOW_FDS:
        ensure_csr(km)
        # A transposed layer whose kernel equals its stride gives every fine voxel at most one parent; when no
        # parent was clipped away (M == n_out) every output row has exactly one pair and needs no partial rows.
        single = transposed and tuple(km.ks) == tuple(km.stride) and km.M == n_out and km.M > 0
        need = 0 if single else km.M * c_out
        if not single and (buffer is None or buffer.numel() < need or buffer.dtype != feats.dtype or buffer.device != dev):
            buffer = _staging(max(need, 1), feats.dtype, dev)
        imap, omap = (km.omap, km.imap) if transposed else (km.imap, km.omap)
        ocsr, oslot = (km.icsr, km.islot) if transposed else (km.ocsr, km.oslot)
        # A strided layer whose kernel equals its stride gives every input one pair; on surface-like clouds nearly
        # every output row then has a single pair, which stores the finished row itself (see pair_route).  The
        # transposed layer over such a map has at most one pair per output row: exactly one unless the voxel's
        # parent was clipped away, and those rows (no pair) are the only ones left to the row sum.
        route = None
        if (route_single_pairs and not single and not km.subm and tuple(km.ks) == tuple(km.stride)
                and km.M > 0 and feats.dtype == torch.float16 and c_in >= 64 and c_in % 32 == 0 and c_out >= 96 and c_out % 8 == 0):
            route = pair_route(km, transposed)
        _lib.check(lib.pce_conv_fwd_fds(feats.data_ptr(), weight.data_ptr(), _ptr(packed), out.data_ptr(), dt, n_in, n_out,
                                        c_in, c_out, kv, mid, imap.data_ptr(), omap.data_ptr(), oslot.data_ptr(), km.kpos.data_ptr(),
                                        km.qkpos.data_ptr(), km.kpos_host, km.qkpos_host, ocsr.data_ptr(), _ptr(route), km.M, km.qsum,
                                        None if single else buffer.data_ptr(), 0 if single else buffer.numel(), epi, s))
    elif dataflow == DATAFLOW_GMS:
        ensure_csr(km)
        need = km.qsum * (c_in + c_out)
        if buffer is None or buffer.numel() < need or buffer.dtype != feats.dtype or buffer.device != dev:
            buffer = _staging(max(need, 1), feats.dtype, dev)
        icsr, icode, ocsr, ocode = (km.ocsr, km.ocode, km.icsr, km.icode) if transposed else (km.icsr, km.icode, km.ocsr, km.ocode)
        _lib.check(lib.pce_conv_fwd_gms(feats.data_ptr(), weight.data_ptr(), _ptr(packed), out.data_ptr(), dt, n_in, n_out,
                                        c_in, c_out, kv, mid, icsr.data_ptr(), icode.data_ptr(), ocsr.data_ptr(), ocode.data_ptr(),
                                        km.kpos.data_ptr(), km.qkpos.data_ptr(), km.qsum, buffer.data_ptr(), buffer.numel(), epi, s))
    elif dataflow == DATAFLOW_OSO:
        if not oso_takes(km, c_in, c_out, feats.dtype, transposed):
            raise ValueError("the ordered output-stationary dataflow takes layers (not transposed, at most 31 offsets) in fp16 "
                             "of at most 64 channels (c_in a multiple of 16, c_out of 8), of 64 or 96 -> 65..128 and 128 -> "
                             "65..96 channels, or submanifold layers in fp32 of at most 32 (multiples of 8)")
        if packed is None:
            packed = pack_weights(weight)      # None for fp32: that form reads the weights as they are
        order = row_order(km)
        _lib.check(lib.pce_conv_fwd_oso(feats.data_ptr(), weight.data_ptr(), _ptr(packed), out.data_ptr(), dt, n_in, n_out,
                                        c_in, c_out, kv, mid, km.nbr_out.data_ptr(), order.data_ptr(),
                                        (_lib.c_int64 * 3)(km.order_heavy, km.order_nonzero, km.order_single), epi, s))
    elif dataflow == DATAFLOW_OS:
        ensure_nbr(km, transposed)
        nbr = km.nbr_in if transposed else km.nbr_out
        if transposed and km.subm:
            # submanifold layer with an even kernel size (no mirror symmetry): the input-major table is the probe
            # result, whose centre row is empty; the transposed layer needs the identity there
            if getattr(km, "_nbr_in_t", None) is None:
                t = km.nbr_in.clone().view(km.kv, km.n_in)
                t[_mid(km.ks)] = torch.arange(km.n_in, dtype=torch.int32, device=t.device)
                km._nbr_in_t = t.view(-1)
            nbr = km._nbr_in_t
        _lib.check(lib.pce_conv_fwd_os(feats.data_ptr(), weight.data_ptr(), _ptr(packed), out.data_ptr(), dt, n_in, n_out,
                                       c_in, c_out, kv, nbr.data_ptr(), epi, s))
    else:
        raise NotImplementedError(f"unknown dataflow {dataflow}")
    if slice_out is not None:
        slice_out.copy_(out)
        return slice_out
    return out


def col_sums(a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float64 [2, c]: column sums of ``a`` [n, c] and of ``a * b`` (``a * a`` without ``b``)."""
    lib = _lib.load()
    _require_cuda(a, "a")
    if a.dim() != 2 or a.dtype not in (torch.float16, torch.float32) or (b is not None and (b.shape != a.shape or b.dtype != a.dtype)):
        raise ValueError("col_sums takes fp16 or fp32 matrices of one shape and dtype")
    a = a.contiguous()
    b = None if b is None else b.contiguous()
    n, c = a.shape
    out = torch.empty((2, c), dtype=torch.float64, device=a.device)
    ws_bytes = lib.pce_col_sums_workspace_bytes(n, c)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=a.device)
    _lib.check(lib.pce_col_sums(a.data_ptr(), _ptr(b), _dtype_code(a), n, c, ws.data_ptr(), ws_bytes, out.data_ptr(),
                                _stream(a.device)))
    return out


def col_affine(x: torch.Tensor, kx: torch.Tensor, k0: torch.Tensor, d: Optional[torch.Tensor] = None,
               kd: Optional[torch.Tensor] = None, act=None) -> torch.Tensor:
    """``act(x * kx + d * kd + k0)`` with fp32 per-column coefficients; the result has x's dtype."""
    lib = _lib.load()
    _require_cuda(x, "x")
    x = x.contiguous()
    d = None if d is None else d.contiguous()
    n, c = x.shape
    coef = [None if k is None else k.to(device=x.device, dtype=torch.float32).contiguous() for k in (kx, kd, k0)]
    y = torch.empty_like(x)
    code, slope = _act_code(act)
    _lib.check(lib.pce_col_affine(x.data_ptr(), _ptr(d), y.data_ptr(), _dtype_code(x), n, c, _ptr(coef[0]), _ptr(coef[1]),
                                  _ptr(coef[2]), code, slope, _stream(x.device)))
    return y


def concat_cols(a: torch.Tensor, b: torch.Tensor) -> Optional[torch.Tensor]:
    """``torch.cat([a, b], dim=1)`` for two feature matrices on the same rows in one streaming kernel, or None
    when the layout does not fit it (rows that are not whole 16-byte vectors, other dtypes, CPU tensors)."""
    if not (a.is_cuda and b.is_cuda and a.device == b.device and a.dim() == 2 and b.dim() == 2 and a.dtype == b.dtype
            and a.dtype in (torch.float16, torch.float32) and a.shape[0] == b.shape[0] and a.shape[0] > 0):
        return None
    per = 8 if a.dtype == torch.float16 else 4
    c_a, c_b = a.shape[1], b.shape[1]
    if c_a == 0 or c_b == 0 or c_a % per or c_b % per or (c_a + c_b) // per > 256:
        return None
    a, b = a.contiguous(), b.contiguous()
    if a.data_ptr() % 16 or b.data_ptr() % 16:
        return None
    out = torch.empty((a.shape[0], c_a + c_b), dtype=a.dtype, device=a.device)
    _lib.check(_lib.load().pce_concat_cols(a.data_ptr(), c_a, b.data_ptr(), c_b, out.data_ptr(), _dtype_code(a), a.shape[0],
                                           _stream(a.device)))
    return out


def _f32(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None else t.detach().to(dtype=torch.float32).contiguous()


def bn_forward(x: torch.Tensor, weight, bias, running_mean, running_var, use_batch_stats: bool, momentum: float, eps: float,
               act=None, residual: Optional[torch.Tensor] = None):
    """``act(batch_norm(x) + residual)`` over the rows of ``x`` [n, c] (fp16 / fp32) in three launches.
    ``momentum`` < 0 leaves the running statistics alone; they must be fp32 and are updated in place
    otherwise.  Returns (y, save_mean, save_rstd)."""
    lib = _lib.load()
    _require_cuda(x, "x")
    x = x.contiguous()
    n, c = x.shape
    for name, t in (("running_mean", running_mean), ("running_var", running_var)):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != c):
            raise ValueError(f"{name} must be a contiguous fp32 tensor of {c} elements")
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != x.dtype or residual.device != x.device:
            raise ValueError("the residual must match the normalised tensor in shape, dtype and device")
        residual = residual.contiguous()
    w, b = _f32(weight), _f32(bias)
    y = torch.empty_like(x)
    save = torch.empty((2, c), dtype=torch.float32, device=x.device)
    ws_bytes = lib.pce_bn_workspace_bytes(n, c)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    code, slope = _act_code(act)
    _lib.check(lib.pce_bn_forward(x.data_ptr(), _ptr(residual), y.data_ptr(), _dtype_code(x), n, c, _ptr(w), _ptr(b),
                                  _ptr(running_mean), _ptr(running_var), int(use_batch_stats), float(momentum), float(eps),
                                  save[0].data_ptr(), save[1].data_ptr(), ws.data_ptr(), ws_bytes, code, slope, _stream(x.device)))
    return y, save[0], save[1]


def bn_backward(x: torch.Tensor, dy: torch.Tensor, weight, save_mean: torch.Tensor, save_rstd: torch.Tensor,
                use_batch_stats: bool, y_act: Optional[torch.Tensor] = None, act=None):
    """(dx, grad_weight fp32, grad_bias fp32) of ``bn_forward``.  With ``act`` and its output ``y_act`` the
    incoming gradient is taken with respect to the activation's output and masked while it is read."""
    lib = _lib.load()
    x = x.contiguous()
    dy = dy.to(x.dtype).contiguous()
    n, c = x.shape
    w = _f32(weight)
    code, slope = _act_code(act)
    if code != _lib.ACT_NONE:
        if y_act is None or y_act.shape != x.shape or y_act.dtype != x.dtype:
            raise ValueError("the gradient of an activation needs its output, shaped and typed like x")
        if code == _lib.ACT_LEAKY_RELU and not slope > 0:
            raise ValueError("the output of a LeakyReLU tells the sign of its input only for a positive slope")
        y_act = y_act.contiguous()
    else:
        y_act = None
    dx = torch.empty_like(x)
    grads = torch.empty((2, c), dtype=torch.float32, device=x.device)
    ws_bytes = lib.pce_bn_workspace_bytes(n, c)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    _lib.check(lib.pce_bn_backward(x.data_ptr(), dy.data_ptr(), _ptr(y_act), code, slope, dx.data_ptr(), _dtype_code(x), n, c,
                                   _ptr(w), save_mean.data_ptr(), save_rstd.data_ptr(), int(use_batch_stats),
                                   grads[0].data_ptr(), grads[1].data_ptr(), ws.data_ptr(), ws_bytes, _stream(x.device)))
    return dx, grads[0], grads[1]


def conv_wgrad(feats: torch.Tensor, grad_out: torch.Tensor, km: KernelMap, transposed: bool = False) -> torch.Tensor:
    """Gradient of ``conv_forward`` with respect to the kernel: fp32 [kv, c_in, c_out]."""
    lib = _lib.load()
    _require_cuda(feats, "feats")
    feats, grad_out = feats.contiguous(), grad_out.contiguous()
    if feats.dtype != grad_out.dtype:
        raise TypeError(f"features are {feats.dtype} but the output gradient is {grad_out.dtype}")
    n_in, n_out = (km.n_out, km.n_in) if transposed else (km.n_in, km.n_out)
    if feats.shape[0] != n_in or grad_out.shape[0] != n_out:
        raise ValueError(f"the map expects {n_in} feature rows and {n_out} gradient rows")
    imap, omap = (km.omap, km.imap) if transposed else (km.imap, km.omap)
    c_in, c_out = feats.shape[1], grad_out.shape[1]
    gw = torch.empty((km.kv, c_in, c_out), dtype=torch.float32, device=feats.device)
    _lib.check(lib.pce_conv_wgrad(feats.data_ptr(), grad_out.data_ptr(), _dtype_code(feats), n_in, n_out, c_in, c_out, km.kv,
                                  _mid(km.ks) if km.subm else -1, imap.data_ptr(), omap.data_ptr(), km.kpos.data_ptr(),
                                  km.qkpos.data_ptr(), km.qsum, gw.data_ptr(), _stream(feats.device)))
    return gw


_ZERO_POS = {}


def dense_wgrad(feats: torch.Tensor, grad_out: torch.Tensor) -> torch.Tensor:
    """Gradient of ``dense_forward`` with respect to its [c_in, c_out] matrix, in fp32: the kernel-gradient
    kernel run over row tiles only (one offset, every row paired with itself, no pair list)."""
    lib = _lib.load()
    _require_cuda(feats, "feats")
    feats, grad_out = feats.contiguous(), grad_out.contiguous()
    if feats.dtype != grad_out.dtype:
        raise TypeError(f"features are {feats.dtype} but the output gradient is {grad_out.dtype}")
    if feats.dim() != 2 or grad_out.dim() != 2 or feats.shape[0] != grad_out.shape[0]:
        raise ValueError("features and output gradient must be matrices with the same number of rows")
    n, c_in, c_out = feats.shape[0], feats.shape[1], grad_out.shape[1]
    pos = _ZERO_POS.get(feats.device)
    if pos is None:
        pos = _ZERO_POS[feats.device] = torch.zeros(2, dtype=torch.int32, device=feats.device)
    if n == 0:  # empty tensors have no data pointer to hand over
        return torch.zeros((c_in, c_out), dtype=torch.float32, device=feats.device)
    gw = torch.empty((c_in, c_out), dtype=torch.float32, device=feats.device)
    _lib.check(lib.pce_conv_wgrad(feats.data_ptr(), grad_out.data_ptr(), _dtype_code(feats), n, n, c_in, c_out, 1, 0, None, None,
                                  pos.data_ptr(), pos.data_ptr(), 0, gw.data_ptr(), _stream(feats.device)))
    return gw


def conv_backward(feats: torch.Tensor, weight: torch.Tensor, km: KernelMap, grad_out: torch.Tensor, transposed: bool = False,
                  need_feats: bool = True, need_weight: bool = True, dataflow: Optional[int] = None):
    """(grad_feats, grad_weight) of ``conv_forward``.  The feature gradient is the convolution of
    ``grad_out`` with the per-offset transposed kernel over the same pairs with the roles swapped,
    run by the forward kernels; the kernel gradient comes from ``pce_conv_wgrad`` (fp32 sums,
    returned in the kernel's dtype)."""
    gf = gw = None
    w3 = weight if weight.dim() == 3 else weight.unsqueeze(0)
    if need_feats:
        wt = w3.transpose(1, 2).contiguous()
        df = dataflow if dataflow is not None else select_dataflow(km, wt.shape[1], wt.shape[2], wt.dtype, not transposed)
        gf = conv_forward(grad_out.contiguous(), wt, km, df, transposed=not transposed, packed=pack_weights(wt))
    if need_weight:
        gw = conv_wgrad(feats, grad_out, km, transposed).to(weight.dtype).reshape(weight.shape)
    return gf, gw


# ---------------------------------------------------------------------------------------------
# The reference's pybind names (backend/pybind_cuda.cpp:8-14), same argument order.
# ---------------------------------------------------------------------------------------------
def _geom_from_codes(k_size_code, l_stride_code, padding_code, mins, maxs, separate_mid):
    return decode3(k_size_code), decode3(l_stride_code), decode3(padding_code), list(mins), list(maxs), bool(separate_mid)


def mapping_d2_cuda(in_coords, batch_size, k_size_code, k_vol, c_in, c_out, l_stride_code, t_stride_code, padding_code,
                    min_x, min_y, min_z, max_x, max_y, max_z, map, kernel_nnz, kernel_kpos, kernel_qkpos, separate_mid):
    """HashMapD2 (backend/hash.h:37-58): fills the dense map ``map[kp*N_in + i] = o`` (caller
    pre-fills -1), the per-offset counts and both scans; returns the output coordinates (the
    input tensor itself for a submanifold layer)."""
    ks, stride, pad, cmin, cmax, subm = _geom_from_codes(k_size_code, l_stride_code, padding_code,
                                                         (min_x, min_y, min_z), (max_x, max_y, max_z), separate_mid)
    km = build_kernel_map(in_coords, ks, stride, pad, cmin, cmax, subm, want_nbr_out=False, want_nbr_in=True,
                          batchsize=int(batch_size))
    map.view(-1)[:km.kv * km.n_in].copy_(km.nbr_in)
    kernel_nnz[:km.kv].copy_(km.knnz)
    kernel_kpos[:km.kv + 1].copy_(km.kpos)
    kernel_qkpos[:km.kv + 1].copy_(km.qkpos)
    return in_coords if subm else km.out_coords


def mapping_d1_cuda(in_coords, k_size_code, k_vol, c_in, c_out, l_stride_code, t_stride_code, padding_code,
                    min_x, min_y, min_z, max_x, max_y, max_z, imap, omap, icsr, ocsr, kernel_nnz, kernel_kpos,
                    kernel_qkpos, separate_mid):
    """HashMapD1 (backend/hash.h:11-34): compacted CSR codes at the front of ``imap`` / ``omap``,
    row pointers in ``icsr`` / ``ocsr``, counts and scans.  ``kernel_kpos`` may have the
    reference's kv entries (script/spconv.py:396) or kv+1; only what fits is written."""
    ks, stride, pad, cmin, cmax, subm = _geom_from_codes(k_size_code, l_stride_code, padding_code,
                                                         (min_x, min_y, min_z), (max_x, max_y, max_z), separate_mid)
    km = build_kernel_map(in_coords, ks, stride, pad, cmin, cmax, subm, want_csr=True, want_nbr_out=False)
    if omap.numel() < km.M or ocsr.numel() < km.n_out + 1:
        raise OverflowError("omap / ocsr are too small for this map")
    imap.view(-1)[:km.M].copy_(km.icode)
    omap.view(-1)[:km.M].copy_(km.ocode)
    icsr[:km.n_in + 1].copy_(km.icsr)
    ocsr[:km.n_out + 1].copy_(km.ocsr)
    kernel_nnz[:km.kv].copy_(km.knnz)
    n = min(kernel_kpos.numel(), km.kv + 1)
    kernel_kpos[:n].copy_(km.kpos[:n])
    kernel_qkpos[:km.kv + 1].copy_(km.qkpos)
    return in_coords if subm else km.out_coords


def _ksize_mid(ksize_code: int, separate_mid: bool) -> int:
    return _mid(decode3(ksize_code)) if separate_mid else -1


def conv_fwd_d2_cuda(in_feats, kernel, ksize_code, sum_nnz, out_feats, kpos, qkpos, in_map, out_map, separate_mid, tf32):
    """ConvolutionForwardD2 (backend/spconv.h:28-40); ``sum_nnz`` is qkpos[-1] as in the reference."""
    lib = _lib.load()
    _require_cuda(in_feats, "in_feats")
    if in_feats.shape[1] != kernel.shape[1]:
        raise ValueError("Input feature size and kernel size mismatch")
    kv, c_in, c_out = kernel.shape
    dt = _dtype_code(in_feats)
    n_in, n_out = in_feats.shape[0], out_feats.shape[0]
    ws_bytes = lib.pce_conv_fod_workspace_bytes(n_out, c_out, dt)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=in_feats.device) if ws_bytes else None
    _lib.check(lib.pce_conv_fwd_fod(in_feats.data_ptr(), kernel.data_ptr(), None, out_feats.data_ptr(), dt, n_in, n_out, c_in,
                                    c_out, kv, _ksize_mid(ksize_code, separate_mid), in_map.data_ptr(), out_map.data_ptr(),
                                    kpos.data_ptr(), qkpos.data_ptr(), int(sum_nnz), _ptr(ws), ws_bytes, None,
                                    _stream(in_feats.device)))


def conv_fwd_d1_cuda(in_feats, kernel, ksize_code, qsum_nnz, out_feats, kpos, qkpos, in_map, out_map, in_csr, out_csr,
                     buffer, separate_mid, tensorcore):
    """ConvolutionForwardD1 (backend/spconv.h:11-25)."""
    lib = _lib.load()
    _require_cuda(in_feats, "in_feats")
    if in_feats.shape[1] != kernel.shape[1]:
        raise ValueError("Input feature size and kernel size mismatch")
    kv, c_in, c_out = kernel.shape
    dt = _dtype_code(in_feats)
    if buffer.dtype != in_feats.dtype:
        raise TypeError("the staging buffer must have the dtype of the features")
    if kpos.numel() < kv + 1:
        # the reference front end allocates kv entries (script/spconv.py:396); the total is the last row pointer
        kpos = torch.cat([kpos[:kv], in_csr[in_feats.shape[0]:in_feats.shape[0] + 1]])
    _lib.check(lib.pce_conv_fwd_gms(in_feats.data_ptr(), kernel.data_ptr(), None, out_feats.data_ptr(), dt, in_feats.shape[0],
                                    out_feats.shape[0], c_in, c_out, kv, _ksize_mid(ksize_code, separate_mid),
                                    in_csr.data_ptr(), in_map.data_ptr(), out_csr.data_ptr(), out_map.data_ptr(),
                                    kpos.data_ptr(), qkpos.data_ptr(), int(qsum_nnz), buffer.data_ptr(), buffer.numel(), None,
                                    _stream(in_feats.device)))


def conv_bwd_d1_cuda(out_feats_grad, in_feats, kernel, ksize_code, sum_nnz, in_feats_grad, kernel_grad, kernel_nnz,
                     kernel_pos, in_map, out_map, in_csr, out_csr, buffer, tensorcore):
    """ConvolutionBackwardD1 (backend/spconv.h:43-58): fills ``in_feats_grad`` and ``kernel_grad``
    from the CSR-coded map of ``mapping_d1_cuda``.  The coded lists are decoded into the plain pair
    lists first (entry = kp * 1186111 + rank, pair index = kpos[kp] + rank)."""
    lib = _lib.load()
    _require_cuda(in_feats, "in_feats")
    if in_feats.shape[1] != kernel.shape[1]:
        raise ValueError("Input feature size and kernel size mismatch")
    kv, c_in, c_out = kernel.shape
    n_in, n_out = in_feats.shape[0], out_feats_grad.shape[0]
    dev = in_feats.device
    M = int(in_csr[n_in].item())
    kpos = kernel_pos[:kv].to(torch.int64)
    kpos_full = torch.cat([kpos, torch.tensor([M], device=dev, dtype=torch.int64)])

    def pairs(csr, code, n):
        rows = torch.repeat_interleave(torch.arange(n, device=dev, dtype=torch.int32), (csr[1:n + 1] - csr[:n]).long())
        c = code[:M].long()
        idx = kpos[c // CSR_CODE] + c % CSR_CODE
        out = torch.empty(M, dtype=torch.int32, device=dev)
        out[idx] = rows
        return out
    imap, omap = pairs(in_csr, in_map, n_in), pairs(out_csr, out_map, n_out)
    knnz = (kpos_full[1:] - kpos_full[:-1])
    q = (knnz + QUANTUM - 1) // QUANTUM * QUANTUM
    qkpos = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), torch.cumsum(q, 0)]).to(torch.int32)
    kp32 = kpos_full.to(torch.int32)
    qsum = int(qkpos[-1].item())
    separate_mid = n_in == n_out
    mid = _ksize_mid(ksize_code, separate_mid)
    dt = _dtype_code(in_feats)
    s = _stream(dev)
    gw = torch.empty((kv, c_in, c_out), dtype=torch.float32, device=dev)
    _lib.check(lib.pce_conv_wgrad(in_feats.data_ptr(), out_feats_grad.contiguous().data_ptr(), dt, n_in, n_out, c_in, c_out, kv,
                                  mid, imap.data_ptr(), omap.data_ptr(), kp32.data_ptr(), qkpos.data_ptr(), qsum,
                                  gw.data_ptr(), s))
    kernel_grad.copy_(gw.to(kernel_grad.dtype))
    wt = kernel.transpose(1, 2).contiguous()
    ws_bytes = lib.pce_conv_fod_workspace_bytes(n_in, c_in, dt)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    g = out_feats_grad.contiguous()
    tmp = in_feats_grad if in_feats_grad.dtype == in_feats.dtype else torch.empty_like(in_feats)
    _lib.check(lib.pce_conv_fwd_fod(g.data_ptr(), wt.data_ptr(), None, tmp.data_ptr(), dt, n_out, n_in, c_out, c_in, kv, mid,
                                    omap.data_ptr(), imap.data_ptr(), kp32.data_ptr(), qkpos.data_ptr(), qsum, _ptr(ws),
                                    ws_bytes, None, s))
    if tmp is not in_feats_grad:
        in_feats_grad.copy_(tmp.to(in_feats_grad.dtype))
