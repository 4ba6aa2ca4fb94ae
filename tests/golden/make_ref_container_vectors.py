"""Writes tests/golden/ref_containers.json from the reference's own header-only
containers (oracle/_ref/libkraken_ref_containers.so, built by `make -C oracle ref`
from common/utils.h, common/skip_list.h and common/parallel_skip_list.h in the
reference tree). Run in the build container only; the JSON is what travels.

    python tests/golden/make_ref_container_vectors.py
"""
import ctypes as C
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding  # noqa: E402


def main():
    L = binding.ref_lib()
    if L is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle ref`")
    rng = np.random.default_rng(20240607)
    fixed = [0, 1, 2, 7, 8, 9, 255, 256, 2**31 - 1, 2**31, 2**32 - 1, 2**32, 2**63 - 1, 2**63,
             2**64 - 1, 0x9E3779B97F4A7C15, 0xDEADBEEFCAFEBABE, 1000003, 99999, 100000]
    keys = fixed + [int(x) for x in rng.integers(0, 2**64, size=108, dtype=np.uint64)]
    out = {
        "hash64": [[str(k), str(L.ref_hash64(k))] for k in keys],
        "hash64_pair": [[str(a), str(b), str(L.ref_hash64_pair(a, b))]
                        for a, b in zip(keys[:64], keys[64:128])],
    }
    # container walk: insert shuffled keys (some twice), report slot of each key, the export
    # order, and hit/miss for a probe set.
    m = L.ref_map_create()
    ins = [int(x) for x in rng.integers(0, 5000, size=600, dtype=np.uint64)]
    ins += [2**64 - 1, 2**63, 2**32 + 5]
    arr = np.array(ins, dtype=np.uint64)
    vals = np.arange(arr.size * 2, dtype=np.float32).reshape(arr.size, 2)
    fresh = L.ref_map_insert(m, arr.ctypes.data_as(C.POINTER(C.c_uint64)), arr.size,
                             vals.ctypes.data_as(C.POINTER(C.c_float)), 2)
    order = np.empty(arr.size, np.uint64)
    n = L.ref_map_keys(m, order.ctypes.data_as(C.POINTER(C.c_uint64)))
    probe = np.array([int(x) for x in rng.integers(0, 6000, size=300, dtype=np.uint64)] + ins[-3:],
                     dtype=np.uint64)
    hit = np.empty(probe.size, np.uint8)
    got = np.zeros((probe.size, 2), np.float32)
    L.ref_map_find(m, probe.ctypes.data_as(C.POINTER(C.c_uint64)), probe.size,
                   hit.ctypes.data_as(C.POINTER(C.c_uint8)),
                   got.ctypes.data_as(C.POINTER(C.c_float)), 2)
    out["container"] = {
        "inserted": [str(x) for x in ins],
        "fresh": int(fresh),
        "slots": [int(L.ref_map_hit_slot(m, int(k))) for k in ins[:40]],
        "export_order": [str(int(x)) for x in order[:n]],
        "probe": [str(int(x)) for x in probe],
        "hit": [int(x) for x in hit],
        "first_col": [float(x) for x in got[:, 0]],
    }
    L.ref_map_destroy(m)
    path = os.path.join(ROOT, "tests", "golden", "ref_containers.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=0)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
