"""Writes tests/golden/ref_router.json with the reference's own consistent-hash ring
(oracle/_ref/ref_router = common/router.cc compiled where it lies, built by `make -C oracle ref`).
Runs only where the reference tree is present; the file is committed as a fixture.

Per case: the node names (ids 0, 1, 2, ... in that order), the table id, the ring as
[hash_v, node_id] pairs in ascending hash order, the owner of sparse_id = splitmix64(r) for
r < n and of a few hand-picked ids ("ids"), and raw ring look-ups on and next to every virtual
node and at both ends of the hash space ("hits")."""
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
TOOL = os.path.join(HERE, "..", "..", "oracle", "_ref", "ref_router")

CASES = [(7, 200, ["ps0", "ps1", "ps2"]),
         (0, 100, ["127.0.0.1:50000"]),
         (12345678901234567, 200, ["a", "b", "c", "d", "e", "f", "g"])]


def main():
    if not os.path.exists(TOOL):
        sys.exit("build oracle/_ref/ref_router first: make -C oracle ref")
    out = []
    for table_id, n, names in CASES:
        text = subprocess.check_output([TOOL, str(table_id), str(n)] + names, text=True)
        case = {"table_id": table_id, "nodes": names, "ring": [], "ids": [], "hits": []}
        for line in text.splitlines():
            kind, a, b = line.split()
            case[{"vnode": "ring", "id": "ids", "hit": "hits"}[kind]].append([int(a), int(b)])
        out.append(case)
    with open(os.path.join(HERE, "ref_router.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
        f.write("\n")


if __name__ == "__main__":
    main()
