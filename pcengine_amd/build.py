"""Builds libpcengine_amd.so (hand-written HIP for gfx950) in-tree with hipcc, and beside it
libpcengine_amd_measure.so: the same sources with -DPCE_MEASURE, which adds the stage mask that
bench.py uses to time one kernel of a dataflow alone (include/pcengine_amd_measure.h).

    python -m pcengine_amd.build            # compile
    python -m pcengine_amd.build --force    # recompile even if up to date
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libpcengine_amd.so")
MEASURE_LIB_PATH = os.path.join(LIB_DIR, "libpcengine_amd_measure.so")
SOURCES = ["pce_map.hip", "pce_conv.hip", "pce_plan.hip"]
MEASURE_SOURCES = ["pce_conv.hip"]      # the sources that read PCE_MEASURE; the others are shared as objects
HEADERS = [os.path.join(CSRC, "pce_common.h"), os.path.join(ROOT, "include", "pcengine_amd.h"),
           os.path.join(ROOT, "include", "pcengine_amd_measure.h")]

# packed fp32 instructions are switched off for every device compile of this project
HIPCC_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libpcengine_amd.so cannot be built")
    return exe


def up_to_date() -> bool:
    if not os.path.exists(LIB_PATH) or not os.path.exists(MEASURE_LIB_PATH):
        return False
    t = min(os.path.getmtime(LIB_PATH), os.path.getmtime(MEASURE_LIB_PATH))
    deps = [os.path.join(CSRC, s) for s in SOURCES] + HEADERS
    return all(os.path.getmtime(d) <= t for d in deps)


def build(force: bool = True, verbose: bool = False) -> str:
    if not force and up_to_date():
        return LIB_PATH
    os.makedirs(LIB_DIR, exist_ok=True)
    objs, measure_objs = [], []
    procs = []
    for src, measure in [(s, False) for s in SOURCES] + [(s, True) for s in MEASURE_SOURCES]:
        obj = os.path.join(LIB_DIR, src.replace(".hip", "_measure.o" if measure else ".o"))
        cmd = [_hipcc(), *HIPCC_FLAGS, *(["-DPCE_MEASURE"] if measure else []), "-I", os.path.join(ROOT, "include"),
               "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if measure:
            measure_objs.append(obj)
        else:
            objs.append(obj)
            if src not in MEASURE_SOURCES:
                measure_objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        # the host pass does not know the device feature flag and says so; nothing else is filtered
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out)
    for path, members in ((LIB_PATH, objs), (MEASURE_LIB_PATH, measure_objs)):
        subprocess.run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", path, *members], check=True)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force=True if "--force" in sys.argv or True else False, verbose=True))
