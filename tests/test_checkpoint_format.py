"""The table-file layout, pinned by files the reference's own serializer wrote
(tests/golden/ref_*.sparse, ref_*.dense; generator: tests/golden/make_ref_checkpoint_files.py over
oracle/ref_checkpoint.cc, which compiles common/serialize.h and the tensor sources where they
lie). The `struct` reader and writer of checkpoint_format.py are checked against those bytes
here, on the CPU; the library's C++ reader and writer are checked against the same files and
against this reader in test_gpu_checkpoint.py."""
import os
import struct

import numpy as np
import pytest

from checkpoint_format import pack_rows, pack_string, pack_value, parse_dense, parse_rows, parse_sparse

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
M64 = (1 << 64) - 1

# name, dim, rows, states, with Adam's step counter: as in make_ref_checkpoint_files.py
SPARSE = [("ref_plain_d5", 5, 30, [], False),
          ("ref_adagrad_d4", 4, 40, [2], False),
          ("ref_adam_d8", 8, 25, [3, 4], True),
          ("ref_rmsprop_all_d4", 4, 20, [6, 7, 1], False)]


def mix(x):
    z = (x + 0x9E3779B97F4A7C15) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def pattern(row_id, which, n):
    """oracle/ref_checkpoint.cc pattern(): multiples of 1/64 in [-16, 16]."""
    return np.array([((mix((row_id * 31 + which * 1000003 + j) & M64) % 2049) - 1024) / 64.0 for j in range(n)],
                    np.float32)


def expected_rows(dim, rows, states, steps):
    out = {}
    for r in range(rows):
        k = mix(r)
        out[k] = (pattern(k, 0, dim), {s: pattern(k, s + 1, dim) for s in states}, {0: 1 + k % 7} if steps else {})
    return out


@pytest.mark.parametrize("name,dim,rows,states,steps", SPARSE)
def test_reader_on_files_the_reference_wrote(name, dim, rows, states, steps):
    head, slots = parse_sparse(os.path.join(GOLDEN, name + ".sparse"))
    assert head == dict(type=1, id=7, name="emb", dim=dim, dtype=11, init=2,
                        conf={"mean": "0.000000", "stddev": "0.010000"})      # std::to_string
    assert len(slots) == 8
    want = expected_rows(dim, rows, states, steps)
    seen = 0
    for s, slot_rows in enumerate(slots):
        keys = [r[0] for r in slot_rows]
        assert keys == sorted(keys) and all(k % 8 == s for k in keys)
        for k, dims, val, st, cnt in slot_rows:
            w_val, w_st, w_cnt = want[k]
            assert dims == [dim] and np.array_equal(val, w_val)
            assert set(st) == set(w_st) and all(np.array_equal(st[x], w_st[x]) for x in st)
            assert cnt == w_cnt
            seen += 1
    assert seen == rows


@pytest.mark.parametrize("name,dim,rows,states,steps", SPARSE)
def test_writer_reproduces_the_reference_bytes(name, dim, rows, states, steps):
    """Files with at most one entry per map have one possible byte sequence; with several states
    the reference writes them in its hash map's order, so there the order is taken from the file."""
    path = os.path.join(GOLDEN, name + ".sparse")
    golden = open(path, "rb").read()
    _, slots = parse_sparse(path)
    body = struct.pack("<BQ", 1, 7) + pack_string("emb") + struct.pack("<qBB", dim, 11, 2)
    conf_order = ["mean", "stddev"] if golden.index(b"mean") < golden.index(b"stddev") else ["stddev", "mean"]
    conf = {"mean": "0.000000", "stddev": "0.010000"}
    body += struct.pack("<Q", 2) + b"".join(pack_string(k) + pack_string(conf[k]) for k in conf_order)
    body += struct.pack("<Q", 8)
    want = expected_rows(dim, rows, states, steps)
    for slot_rows in slots:
        body += struct.pack("<Q", len(slot_rows))
        for k, _, _, st_in_file, _ in slot_rows:
            val, st, cnt = want[k]
            body += struct.pack("<Q", k) + pack_value(val, {s: st[s] for s in st_in_file}, cnt)
    assert body == golden


def test_dense_file_the_reference_wrote():
    head, dims, val, states, counters = parse_dense(os.path.join(GOLDEN, "ref_adam.dense"))
    assert head == dict(type=0, id=3, name="dense0") and dims == [6, 4]
    assert np.array_equal(val, pattern(99, 0, 24))
    assert set(states) == {3, 4}
    assert np.array_equal(states[3], pattern(99, 4, 24)) and np.array_equal(states[4], pattern(99, 5, 24))
    assert counters == {0: 12}


@pytest.mark.parametrize("dim", [5, 16])
def test_row_blocks_the_reference_wrote(dim):
    """The body of a pull reply / the gradients of a push request: std::vector<Tensor>."""
    golden = open(os.path.join(GOLDEN, "ref_rows_d%d.wire" % dim), "rb").read()
    want = np.array([pattern(mix(r), 0, dim) for r in range(33)])
    assert len(golden) == 8 + 33 * (18 + 4 * dim)
    assert np.array_equal(parse_rows(golden), want)
    assert pack_rows(want) == golden



def test_malformed_dense_files_are_errors_before_any_gpu_work(tmp_path):
    """krk_dense_load_file reads the Value before it creates the table, so a file whose lengths
    no file could back is refused here, without a GPU: error code, no exception, no huge
    allocation."""
    import ctypes as C
    from kraken_amd import api
    L = api.lib()
    cases = {
        "huge tensor": struct.pack("<BQ", 0, 5) + pack_string("d") + struct.pack("<BQqB", 0, 1, 1 << 40, 11),
        "overflowing dims": struct.pack("<BQ", 0, 5) + pack_string("d") + struct.pack("<BQ", 0, 3) +
                            struct.pack("<qqq", 1 << 31, 1 << 31, 1 << 31) + b"\x0b",
        "huge name": struct.pack("<BQ", 0, 5) + struct.pack("<Q", 1 << 40) + b"d",
        "negative dim": struct.pack("<BQ", 0, 5) + pack_string("d") + struct.pack("<BQqB", 0, 1, -4, 11),
        "rank 17": struct.pack("<BQ", 0, 5) + pack_string("d") + struct.pack("<BQ", 0, 17),
        "cut": struct.pack("<BQ", 0, 5),
    }
    for what, body in cases.items():
        path = str(tmp_path / "bad.dense")
        open(path, "wb").write(body)
        out = C.c_void_p()
        rc = L.krk_dense_load_file(os.fsencode(path), C.byref(out), None, None, 0, None, None)
        assert rc == api.E_IO, what
        assert not out.value
