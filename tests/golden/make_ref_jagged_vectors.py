"""Writes tests/golden/ref_jagged.json from the reference's own jagged pooling loops
(oracle/_ref/libkraken_ref_jagged.so, built by `make -C oracle ref` from
pytorch/py/jagged_ops.cc in the reference tree). Run in the build container only; the JSON
is what travels.

    python tests/golden/make_ref_jagged_vectors.py

Each case holds the inputs and what the reference returned. For the backward of the sum the
output buffer is pre-filled with a sentinel: the reference writes only the first row of each
bag (its destination pointer never advances, jagged_ops.cc:148-160) and the fixture records
exactly that.
"""
import ctypes as C
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding  # noqa: E402

SENTINEL = -12345.0


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def main():
    L = binding.ref_jagged_lib()
    if L is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle ref`")
    rng = np.random.default_rng(20240611)
    cases = []
    for col, lengths in ((5, [3, 0, 1, 7, 2, 0, 0, 20, 1]), (16, [1, 2, 3, 4, 13, 0, 9]), (1, [4, 4, 0, 1])):
        offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
        rows, k = int(offsets[-1]), len(lengths)
        v = rng.standard_normal((rows, col)).astype(np.float32)
        g = rng.standard_normal((k, col)).astype(np.float32)
        case = {"col": col, "offsets": offsets.tolist(), "values": v.ravel().tolist(),
                "grads": g.ravel().tolist(), "patch_value": 0.25, "sentinel": SENTINEL}
        for mode in ("sum", "mean"):
            out = np.empty((k, col), np.float32)
            getattr(L, "ref_jagged_%s_forward" % mode)(_p(v, C.c_float), col, _p(offsets, C.c_int64), k,
                                                       0.25, _p(out, C.c_float))
            case[mode + "_forward"] = out.ravel().tolist()
            vg = np.full((rows, col), SENTINEL, np.float32)
            getattr(L, "ref_jagged_%s_backward" % mode)(_p(offsets, C.c_int64), k, _p(g, C.c_float), col,
                                                        _p(vg, C.c_float))
            case[mode + "_backward"] = vg.ravel().tolist()
        cases.append(case)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_jagged.json")
    with open(path, "w") as f:
        json.dump({"cases": cases}, f)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
