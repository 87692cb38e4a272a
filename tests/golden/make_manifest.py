"""Writes tests/golden/manifest.json: the frozen sizes and digests of the five benchmark inputs and of their
kernel maps, as the CPU oracle computes them.  The reference holds no stored vectors for this path, so the
manifest pins the seeded generators and the oracle against drift (a change in either shows up as a digest
mismatch in tests/test_oracle.py), and lets the GPU tests check full-size maps without running the oracle.

    python tests/golden/make_manifest.py            # rewrites the manifest (about a minute on 8 cores)

For the two network configurations (4 and 5) the manifest also holds the whole pyramid a MinkUNet-style forward
builds (script/spconv.py:330-372 once per distinct layer geometry): five resolution levels, at each the
submanifold 3x3x3 map and, between consecutive levels, the k2s2 map, nine maps in all.  The bound on the output
coordinates of level l+1 is the one the front end carries along, (max_l - (k-1)) // s (script/spconv.py:358-360).

Digests are SHA-256 over the little-endian int32 bytes of the arrays named."""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as orc            # noqa: E402
from pcengine_amd import synth              # noqa: E402

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "manifest.json")

# name -> (generator, layers whose maps are recorded as (kernel, stride, padding))
CONFIGS = {
    "cfg1": (lambda: synth.sphere_plane_cloud(), [((3, 3, 3), (1, 1, 1), (0, 0, 0))]),
    "cfg2": (lambda: synth.lidar_cloud(), [((3, 3, 3), (1, 1, 1), (0, 0, 0)), ((2, 2, 2), (2, 2, 2), (0, 0, 0))]),
    "cfg4": (lambda: synth.lidar_cloud_100k(), [((3, 3, 3), (1, 1, 1), (0, 0, 0)), ((2, 2, 2), (2, 2, 2), (0, 0, 0))]),
    "cfg5": (lambda: synth.indoor_batch(), [((3, 3, 3), (1, 1, 1), (0, 0, 0)), ((2, 2, 2), (2, 2, 2), (0, 0, 0))]),
}


def digest(*arrays) -> str:
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a, dtype="<i4").tobytes())
    return h.hexdigest()


def layer_entry(km) -> dict:
    return {"n_out": int(km.n_out), "pairs": int(len(km.imap)), "knnz": [int(v) for v in km.knnz],
            "qsum": int(km.qkpos[-1]), "out_coords_sha256": digest(km.out_coords),
            "pairs_sha256": digest(km.imap, km.omap)}


PYRAMIDS = ("cfg4", "cfg5")   # configurations whose network needs the maps of every resolution level
LEVELS = 5


def pyramid_entry(coords: np.ndarray, level0: dict) -> list:
    """Levels 0..4: voxel count, coordinate bound, the submanifold map and (but for the last level) the k2s2 map
    that leads to the next level.  `level0` holds the two maps of level 0, already computed."""
    levels = []
    cmax = [int(v) for v in coords[:, 1:].max(axis=0)]
    for lv in range(LEVELS):
        e = {"level": lv, "voxels": int(len(coords)), "coords_max": cmax, "coords_sha256": digest(coords), "layers": {}}
        if lv == 0:
            e["layers"]["k333_s111_p000"] = level0["k333_s111_p000"]
        else:
            e["layers"]["k333_s111_p000"] = layer_entry(orc.kernel_map(coords, (3, 3, 3)))
        if lv + 1 < LEVELS:
            down = orc.kernel_map(coords, (2, 2, 2), (2, 2, 2), (0, 0, 0), cmax=cmax)
            e["layers"]["k222_s222_p000"] = layer_entry(down)
            if lv == 0:
                assert e["layers"]["k222_s222_p000"] == level0["k222_s222_p000"]
            coords = down.out_coords
            cmax = orc.strided_coords_max(cmax, (2, 2, 2), (2, 2, 2), (0, 0, 0))
        levels.append(e)
    return levels


def config_entry(name: str) -> dict:
    gen, layers = CONFIGS[name]
    coords = gen()
    entry = {"voxels": int(len(coords)), "coords_max": [int(v) for v in coords[:, 1:].max(axis=0)],
             "batches": int(coords[:, 0].max()) + 1, "coords_sha256": digest(coords), "layers": {}}
    for ks, stride, pad in layers:
        key = "k%d%d%d_s%d%d%d_p%d%d%d" % (*ks, *stride, *pad)
        entry["layers"][key] = layer_entry(orc.kernel_map(coords, ks, stride, pad))
    if name in PYRAMIDS:
        entry["pyramid"] = pyramid_entry(coords, entry["layers"])
    return entry


def main() -> None:
    manifest = {name: config_entry(name) for name in CONFIGS}
    with open(PATH, "w") as f:
        json.dump(manifest, f, indent=1, sort_keys=True)
        f.write("\n")
    for name, e in manifest.items():
        print(name, e["voxels"], {k: (v["n_out"], v["pairs"]) for k, v in e["layers"].items()})
        for lv in e.get("pyramid", []):
            print("   level", lv["level"], lv["voxels"], {k: (v["n_out"], v["pairs"]) for k, v in lv["layers"].items()})


if __name__ == "__main__":
    main()
