"""ctypes binding of libpcengine_amd.so (the C ABI declared in include/pcengine_amd.h).

The library is the only compute path: if it is missing, loading raises and every operator of
the package fails with that error.  There is no CPU fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_int32, c_int64, c_void_p, c_char_p, POINTER, Structure

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpcengine_amd.so")
MEASURE_LIB_PATH = os.path.join(_HERE, "lib", "libpcengine_amd_measure.so")

PCE_OK, PCE_EINVAL, PCE_ECAPACITY, PCE_EHIP, PCE_EWORKSPACE, PCE_ECOORD = range(6)
PCE_F16, PCE_F32, PCE_F64 = 0, 1, 2
DATAFLOW_FOD, DATAFLOW_GMS, DATAFLOW_OS, DATAFLOW_FDS, DATAFLOW_OSO = 0, 1, 2, 3, 4
QUANTUM = 128
KMAP_NO_GRID = 1
KMAP_TABLE_ONLY = 2
ABI_VERSION = 200        # PCE_ABI_VERSION of include/pcengine_amd.h
CSR_CODE = 1186111


class Geom(Structure):
    _fields_ = [("ks", c_int32 * 3), ("stride", c_int32 * 3), ("pad", c_int32 * 3),
                ("cmin", c_int32 * 3), ("cmax", c_int32 * 3), ("subm", c_int32)]

    @classmethod
    def make(cls, ks, stride, pad, cmin, cmax, subm):
        g = cls()
        for name, v in (("ks", ks), ("stride", stride), ("pad", pad), ("cmin", cmin), ("cmax", cmax)):
            arr = getattr(g, name)
            for a in range(3):
                arr[a] = int(v[a])
        g.subm = int(bool(subm))
        return g


class KmapProblem(Structure):
    """pce_kmap_problem_t: the arguments of one kernel-map build inside a batch."""
    _fields_ = ([("in_coords", c_void_p), ("n_in", c_int64), ("out_coords", c_void_p), ("n_out", c_int64),
                 ("geom", Geom), ("ws", c_void_p), ("ws_bytes", c_int64)] +
                [(name, c_void_p) for name in ("imap", "omap", "knnz", "kpos", "qkpos", "icsr", "icode", "ocsr", "ocode",
                                               "islot", "oslot", "nbr_out", "nbr_in", "status")] +
                [("n_batch", c_int32), ("flags", c_int32), ("order", c_void_p)])


PYR_MAX_LEVELS, PYR_MAX_MAPS, PYR_UNSORTED = 8, 16, 101
(PYR_IMAP, PYR_OMAP, PYR_NBR_OUT, PYR_NBR_IN, PYR_ORDER, PYR_ICSR, PYR_OCSR, PYR_ICODE, PYR_OCODE, PYR_ISLOT, PYR_OSLOT, PYR_META,
 PYR_WS, PYR_ARRAYS) = range(14)


class PyrRequest(Structure):
    """pce_pyr_request_t: one map of a network's pyramid."""
    _fields_ = [("level_in", c_int32), ("level_out", c_int32), ("geom", Geom), ("want_csr", c_int32), ("want_nbr_in", c_int32),
                ("table_only", c_int32), ("pad", c_int32)]


class PyrMap(Structure):
    """pce_pyr_map_t: where the arrays of one map live in the arena, and what its build counted."""
    _fields_ = [("off", c_int64 * PYR_ARRAYS), ("cap_in", c_int64), ("cap_out", c_int64), ("ws_bytes", c_int64),
                ("n_in", c_int64), ("n_out", c_int64), ("n_pairs", c_int64), ("qsum", c_int64),
                ("meta", c_int32 * (3 * 31 + 2 + 8)), ("kv", c_int32)]


class PyrPlan(Structure):
    """pce_pyr_plan_t."""
    _fields_ = [("n_levels", c_int32), ("n_maps", c_int32), ("n_batch", c_int32), ("pad", c_int32),
                ("strided", Geom * PYR_MAX_LEVELS),
                ("level_cap", c_int64 * (PYR_MAX_LEVELS + 1)), ("level_n", c_int64 * (PYR_MAX_LEVELS + 1)),
                ("off_coords", c_int64 * (PYR_MAX_LEVELS + 1)), ("off_chain_ws", c_int64 * PYR_MAX_LEVELS),
                ("chain_ws_bytes", c_int64 * PYR_MAX_LEVELS),
                ("off_meta", c_int64), ("meta_bytes", c_int64), ("arena_bytes", c_int64),
                ("req", PyrRequest * PYR_MAX_MAPS), ("map", PyrMap * PYR_MAX_MAPS)]


class Epilogue(Structure):
    """pce_epilogue_t: out = act(conv + bias + residual)."""
    _fields_ = [("bias", c_void_p), ("residual", c_void_p), ("act", c_int32), ("slope", ctypes.c_float),
                ("ld_in", c_int64), ("ld_out", c_int64)]


ACT_NONE, ACT_RELU, ACT_LEAKY_RELU = 0, 1, 2


class PCEError(RuntimeError):
    pass


_SIGNATURES = {
    "pce_version": (c_int32, []),
    "pce_last_error": (c_char_p, []),
    "pce_hash_slots": (c_int64, [c_int64]),
    "pce_hash_table_bytes": (c_int64, [c_int64]),
    "pce_hash_build": (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "pce_hash_query": (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "pce_outcoords_workspace_bytes": (c_int64, [c_int64, POINTER(Geom), c_int32]),
    "pce_outcoords_build": (c_int32, [c_void_p, c_int64, POINTER(Geom), c_int32, c_void_p, c_int64, POINTER(c_int64), c_void_p]),
    "pce_outcoords_emit": (c_int32, [c_void_p, c_int64, POINTER(Geom), c_int32, c_int64, c_void_p, c_void_p]),
    "pce_outcoords_chain_plan": (c_int32, [c_int64, c_int32, POINTER(Geom), c_int32, POINTER(c_int64), POINTER(c_int64)]),
    "pce_outcoords_chain": (c_int32, [c_void_p, c_int64, c_int32, POINTER(Geom), c_int32, POINTER(c_void_p), POINTER(c_int64),
                                      POINTER(c_void_p), POINTER(c_int64), c_void_p]),
    "pce_outcoords_chain_planned": (c_int32, [c_void_p, c_int64, c_int64, c_int32, POINTER(Geom), c_int32, POINTER(c_void_p),
                                              POINTER(c_int64), POINTER(c_void_p), POINTER(c_int64), c_void_p]),
    "pce_voxelize_workspace_bytes": (c_int64, [c_int64]),
    "pce_voxelize": (c_int32, [c_void_p, c_int32, c_int64, POINTER(ctypes.c_double), c_void_p, c_int64, POINTER(c_int64),
                               POINTER(c_int32), POINTER(c_int32), c_void_p]),
    "pce_voxelize_emit": (c_int32, [c_void_p, c_int64, c_int64, POINTER(c_int32), POINTER(c_int32), c_int32, c_void_p, c_void_p,
                                    c_void_p, c_void_p]),
    "pce_col_sums_workspace_bytes": (c_int64, [c_int64, c_int32]),
    "pce_col_sums": (c_int32, [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_int64, c_void_p, c_void_p]),
    "pce_col_affine": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_int32,
                                 ctypes.c_float, c_void_p]),
    "pce_bn_workspace_bytes": (c_int64, [c_int64, c_int32]),
    "pce_bn_forward": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int32, ctypes.c_float, ctypes.c_float, c_void_p, c_void_p, c_void_p, c_int64, c_int32,
                                 ctypes.c_float, c_void_p]),
    "pce_bn_backward": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, ctypes.c_float, c_void_p, c_int32, c_int64, c_int32,
                                  c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "pce_concat_cols": (c_int32, [c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_int32, c_int64, c_void_p]),
    "pce_kmap_workspace_bytes": (c_int64, [c_int64, c_int64, c_int32, c_int32]),
    "pce_kmap_workspace_bytes_grid": (c_int64, [c_int64, c_int64, POINTER(Geom), c_int32, c_int32]),
    "pce_kmap_build_batch": (c_int32, [POINTER(KmapProblem), c_int32, c_void_p]),
    "pce_kmap_build": (c_int32, [c_void_p, c_int64, c_void_p, c_int64, POINTER(Geom), c_void_p, c_int64] + [c_void_p] * 14 + [c_void_p]),
    "pce_conv_fod_workspace_bytes": (c_int64, [c_int64, c_int32, c_int32]),
    "pce_packed_weight_bytes": (c_int64, [c_int32, c_int32, c_int32, c_int32]),
    "pce_pack_weights": (c_int32, [c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "pce_conv_fwd_fds": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_int32), POINTER(c_int32), c_void_p, c_void_p,
                                   c_int64, c_int64, c_void_p, c_int64, POINTER(Epilogue), c_void_p]),
    "pce_pair_route": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "pce_pair_route_elems": (c_int64, [c_int64, c_int64]),
    "pce_conv_fwd_fod": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, POINTER(Epilogue), c_void_p]),
    "pce_conv_fod_static_capacity_bytes": (c_int64, []),
    "pce_conv_fod_static_init": (c_int32, []),
    "pce_conv_fwd_fod_static": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32,
                                          c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, POINTER(Epilogue), c_void_p]),
    "pce_conv_fwd_gms": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
                                   POINTER(Epilogue), c_void_p]),
    "pce_conv_fwd_os": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_void_p, POINTER(Epilogue), c_void_p]),
    "pce_conv_fwd_oso": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32,
                                   c_void_p, c_void_p, POINTER(c_int64), POINTER(Epilogue), c_void_p]),
    "pce_row_order": (c_int32, [c_void_p, c_int32, c_int64, c_int32, c_void_p, c_int64, POINTER(c_int64), c_void_p]),
    "pce_row_order_elems": (c_int64, [c_int64]),
    "pce_conv_fwd_dense": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, POINTER(Epilogue), c_void_p]),
    "pce_conv_wgrad": (c_int32, [c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p,
                                 c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "pce_pyramid_plan_sizeof": (c_int64, []),
    "pce_pyramid_plan": (c_int32, [c_int64, c_int32, POINTER(Geom), c_int32, POINTER(PyrRequest), c_int32, POINTER(PyrPlan)]),
    "pce_pyramid_build": (c_int32, [POINTER(PyrPlan), c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "pce_select_dataflow": (c_int32, [c_int64, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32]),
    "pce_conv_oso_takes": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int32]),
}

# only in the measurement build (include/pcengine_amd_measure.h)
_MEASURE_SIGNATURES = {"pce_set_stage_mask": (None, [ctypes.c_uint32])}

_lib = None
_measure_lib = None


def exported_names():
    return sorted(_SIGNATURES)


def _attach(lib: ctypes.CDLL, signatures: dict) -> None:
    for name, (res, args) in signatures.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args


def load() -> ctypes.CDLL:
    """Load the shared library (once) and attach the argument types."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise PCEError(
            f"{LIB_PATH} is missing: build it with `python -m pcengine_amd.build` "
            "(hipcc, --offload-arch=gfx950).  pcengine_amd has no other compute path.")
    lib = ctypes.CDLL(LIB_PATH)
    lib.pce_version.restype = c_int32
    if lib.pce_version() != ABI_VERSION:
        raise PCEError(f"{LIB_PATH} has ABI version {lib.pce_version()}, this package binds version {ABI_VERSION}: "
                       "rebuild it with `python -m pcengine_amd.build`")
    _attach(lib, _SIGNATURES)
    _lib = lib
    return lib


class measurement_build:
    """Context manager for benchmarks and A/B tests: inside it every operator of the package runs on
    libpcengine_amd_measure.so (the same kernels, plus ``pce_set_stage_mask``); on exit the mask is reset
    and the product library is back.  Not for concurrent use."""

    def __enter__(self) -> ctypes.CDLL:
        global _lib, _measure_lib
        load()
        if _measure_lib is None:
            if not os.path.exists(MEASURE_LIB_PATH):
                raise PCEError(f"{MEASURE_LIB_PATH} is missing: build it with `python -m pcengine_amd.build`")
            m = ctypes.CDLL(MEASURE_LIB_PATH)
            _attach(m, _SIGNATURES)
            _attach(m, _MEASURE_SIGNATURES)
            _measure_lib = m
        self._product, _lib = _lib, _measure_lib
        return _measure_lib

    def __exit__(self, *exc) -> None:
        global _lib
        _measure_lib.pce_set_stage_mask(0xFFFFFFFF)
        _lib = self._product


def check(rc: int) -> None:
    """Turn a status code into the exception class the reference's pybind layer would raise
    (std::invalid_argument -> ValueError, std::runtime_error -> RuntimeError)."""
    if rc == PCE_OK:
        return
    msg = load().pce_last_error().decode("utf-8", "replace")
    if rc == PCE_EINVAL:
        raise ValueError(msg)
    if rc == PCE_ECAPACITY:
        raise OverflowError(msg)
    raise PCEError(f"[pce status {rc}] {msg}")
