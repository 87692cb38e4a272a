"""CPU oracle (test infrastructure).  See oracle/oracle.py for the rules of use."""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "_build", "libref_literal.so")


def build_literal() -> str:
    """Compile oracle/ref_literal.c (gcc) and return the path of the shared object."""
    subprocess.run(["make", "-C", _HERE, "--no-print-directory"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB


def load_literal() -> ctypes.CDLL:
    if not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(os.path.join(_HERE, "ref_literal.c")):
        build_literal()
    lib = ctypes.CDLL(_LIB)
    lib.lit_coord_hash.restype = ctypes.c_uint64
    return lib
