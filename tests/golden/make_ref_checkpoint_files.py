"""Writes tests/golden/ref_*.sparse / ref_*.dense / ref_rows_*.wire with the reference's own serializer
(oracle/_ref/ref_checkpoint, built by `make -C oracle ref` from the reference's sources where they
lie). Runs only where the reference tree is present; the files are committed as fixtures.

Row r of a sparse fixture: id = splitmix64(r); val[j] = pattern(id, 0, j); state s:
pattern(id, s + 1, j); steps = 1 + id % 7 (see oracle/ref_checkpoint.cc, mirrored in
tests/test_oracle_pins.py)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
TOOL = os.path.join(HERE, "..", "..", "oracle", "_ref", "ref_checkpoint")

# name, dim, rows, states, with Adam's step counter
SPARSE = [("ref_plain_d5", 5, 30, "-", 0),
          ("ref_adagrad_d4", 4, 40, "2", 0),
          ("ref_adam_d8", 8, 25, "3,4", 1),
          ("ref_rmsprop_all_d4", 4, 20, "6,7,1", 0)]


def main():
    if not os.path.exists(TOOL):
        sys.exit("build oracle/_ref/ref_checkpoint first: make -C oracle ref")
    for name, dim, rows, states, steps in SPARSE:
        subprocess.check_call([TOOL, "write-sparse", os.path.join(HERE, name + ".sparse"), str(dim), str(rows),
                               states, str(steps)])
    subprocess.check_call([TOOL, "write-dense", os.path.join(HERE, "ref_adam.dense"), "24"])
    # std::vector<Tensor> as a pull reply / a push request carries it: 33 rows of 5 and of 16 floats
    subprocess.check_call([TOOL, "write-rows", os.path.join(HERE, "ref_rows_d5.wire"), "33", "5"])
    subprocess.check_call([TOOL, "write-rows", os.path.join(HERE, "ref_rows_d16.wire"), "33", "16"])


if __name__ == "__main__":
    main()
