"""Table files in the reference's checkpoint layout (checkpoint/checkpoint.cc:444-509, 535-649,
common/serialize.h).

PARITY UNPINNED for the byte layout: the reference's writer cannot be built here (its Tensor
needs Eigen) and its tests hold no table file, so the layout is checked against a second,
independent reading of common/serialize.h written with `struct` below. What IS pinned is the
behaviour around the file: a table that goes through a file carries on exactly like the
oracle table that never left memory.
"""
import os
import struct

import numpy as np
import pytest

from util import OPTIM_CASES, STATE_OF, assert_close, make_optims, splitmix64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


# --- an independent reader / writer of the layout (common/serialize.h) ---------------------

class Cursor:
    def __init__(self, data):
        self.d, self.at = data, 0

    def take(self, fmt):
        v = struct.unpack_from("<" + fmt, self.d, self.at)
        self.at += struct.calcsize("<" + fmt)
        return v[0] if len(v) == 1 else v

    def string(self):                      # serialize.h:86-94
        n = self.take("Q")
        s = self.d[self.at:self.at + n].decode()
        self.at += n
        return s

    def tensor(self):                      # serialize.h:156-176
        assert self.take("B") == 0         # Layout::kStride
        rank = self.take("Q")
        dims = [self.take("q") for _ in range(rank)]
        assert self.take("B") == 11        # DType::kFloat32
        n = int(np.prod(dims)) if dims else 1
        v = np.frombuffer(self.d, np.float32, n, self.at).copy()
        self.at += 4 * n
        return dims, v

    def value(self):                       # serialize.h:296-298, 242-272
        dims, val = self.tensor()
        states = {}
        for _ in range(self.take("Q")):
            st = self.take("I")
            states[st] = self.tensor()[1]
        counters = {}
        for _ in range(self.take("Q")):
            st = self.take("I")
            counters[st] = self.take("q")
        return dims, val, states, counters


def parse_sparse(path):
    c = Cursor(open(path, "rb").read())
    head = dict(type=c.take("B"), id=c.take("Q"), name=c.string(), dim=c.take("q"), dtype=c.take("B"),
                init=c.take("B"))
    head["conf"] = {c.string(): c.string() for _ in range(c.take("Q"))}
    slots = []
    for _ in range(c.take("Q")):
        rows = []
        for _ in range(c.take("Q")):
            key = c.take("Q")
            rows.append((key,) + c.value())
        slots.append(rows)
    assert c.at == len(c.d)
    return head, slots


def pack_tensor(v, dims=None):
    v = np.ascontiguousarray(v, np.float32)
    dims = list(dims) if dims is not None else [v.size]
    return struct.pack("<BQ", 0, len(dims)) + b"".join(struct.pack("<q", d) for d in dims) + b"\x0b" + v.tobytes()


def pack_string(s):
    return struct.pack("<Q", len(s)) + s.encode()


def pack_value(val, states, counters, dims=None):
    out = pack_tensor(val, dims) + struct.pack("<Q", len(states))
    for st, v in states.items():
        out += struct.pack("<I", st) + pack_tensor(v, dims)
    out += struct.pack("<Q", len(counters))
    for st, c in counters.items():
        out += struct.pack("<Iq", st, c)
    return out


def _tables(api, oracle, dim, seed):
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": str(seed)})
    return api.SparseTable(dim, gi), oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=seed))


@pytest.mark.parametrize("name,type_,conf", [c for c in OPTIM_CASES if c[0] in (
    "sgd", "sgd_mom", "adagrad", "adam", "adam_amsgrad", "rmsprop_all")])
def test_sparse_file_layout_and_round_trip(api, oracle, tmp_path, name, type_, conf):
    dim = 8
    rng = np.random.default_rng(11)
    t, ref = _tables(api, oracle, dim, seed=4)
    ids = np.concatenate([splitmix64(np.arange(4000, dtype=np.uint64)), np.array([2**64 - 1, 0, 8, 16], np.uint64)])
    assert t.Pull(ids)[0] == 0 and ref.pull(ids)[0] == 0
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    touched = ids[::3]

    def grads(step, n):
        return (np.random.default_rng(step).integers(-64, 65, size=(n, dim)) / 4096.0).astype(np.float32)

    for step in range(2):
        g = grads(step, touched.size)
        assert t.Push(o_gpu, touched, g, 0.01) == 0 and ref.push(o_ref, touched, g, 0.01) == 0
    path = str(tmp_path / "emb.sparse")
    assert t.save(path, 7, "emb") == 0

    head, slots = parse_sparse(path)
    assert head["type"] == 1 and head["id"] == 7 and head["name"] == "emb" and head["dim"] == dim
    assert head["dtype"] == 11 and head["init"] == api.InitializerType.kNormal
    assert head["conf"] == {"mean": "0.000000", "stddev": "0.010000"}     # std::to_string, as conf() does
    assert len(slots) == 8                                                # parallel_skip_list.h:12-21
    seen = []
    for s, rows in enumerate(slots):
        keys = [r[0] for r in rows]
        assert all(k % 8 == s for k in keys) and keys == sorted(keys)     # HitSlot, ascending walk
        seen += keys
    assert sorted(seen) == sorted(ids.tolist())
    by_id = {r[0]: r for rows in slots for r in rows}
    rid, rval, _, rsteps = ref.export()
    states = {st: ref.export(state_type=st)[2] for st in STATE_OF[type_]}
    was_touched = set(touched.tolist())
    for i, k in enumerate(rid.tolist()):
        _, dims, val, st_map, counters = by_id[k]
        assert dims == [dim]
        assert_close(val, rval[i], "weights in file")
        for st, v in st_map.items():
            assert_close(v, states[st][i] if st in states else 0 * v, "state %d in file" % st)
        if type_ == 1:          # Adam: a counter exactly for the rows it touched (adam.cc:60)
            assert counters == ({0: 2} if k in was_touched else {})
            assert (k in was_touched) == bool(st_map)
        else:
            assert counters == {}
        if k in was_touched:
            for st in STATE_OF[type_]:
                if np.abs(states[st][i]).sum() > 0:
                    assert st in st_map

    # through the file into a fresh table (every second id routed elsewhere), then both keep training
    t2, _ = _tables(api, oracle, dim, seed=4)
    rc, taken = t2.load_file(path, 7, "emb", keep=lambda k: k % 2 == 0)
    even = ids[ids % np.uint64(2) == 0]
    assert rc == 0 and taken == even.size == len(t2)
    assert t2.load_file(path, 8, "emb")[0] == api.E_ARGUMENT          # another table id
    assert t2.load_file(path, 7, "other")[0] == api.E_ARGUMENT
    assert t2.load_file(str(tmp_path / "missing.sparse"), 7, "emb")[0] == api.E_IO
    for step in range(2, 4):
        g = grads(step, ids.size)
        assert ref.push(o_ref, ids, g, 0.01) == 0
        assert t2.Push(o_gpu, even, g[ids % np.uint64(2) == 0], 0.01) == 0
    rc, want = ref.pull(even)
    assert_close(t2.Pull(even)[1], want, name + " after the file")


def test_sparse_file_written_by_hand_is_read(api, oracle, tmp_path):
    """The other direction: a file assembled here from the layout (a reference-side writer would
    produce these bytes) loads with states, counters, a 2-slot layout and rows in any order."""
    dim = 4
    rows = {5: ([1, 2, 3, 4], {2: [.5, .5, .5, .5]}, {}),
            13: ([5, 6, 7, 8], {3: [.1, .2, .3, .4], 4: [1, 1, 1, 1]}, {0: 9}),
            2: ([0, 0, 0, 1], {}, {}),
            2**64 - 1: ([9, 9, 9, 9], {1: [2, 2, 2, 2]}, {})}
    body = struct.pack("<BQ", 1, 21) + pack_string("t") + struct.pack("<qBB", dim, 11, 0)
    body += struct.pack("<Q", 1) + pack_string("value") + pack_string("0.250000")
    body += struct.pack("<Q", 2)
    for group in ([13, 5], [2**64 - 1, 2]):
        body += struct.pack("<Q", len(group))
        for k in group:
            val, st, cnt = rows[k]
            body += struct.pack("<Q", k) + pack_value(val, st, cnt)
    path = str(tmp_path / "hand.sparse")
    open(path, "wb").write(body)
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "0.25"})
    t = api.SparseTable(dim, gi)
    rc, taken = t.load_file(path, 21, "t")
    assert rc == 0 and taken == 4 and len(t) == 4
    keys = np.array(list(rows), np.uint64)
    for st in range(1, 8):
        found, vals, state, steps = t.fetch(keys, state_type=st)
        assert found.all()
        for i, k in enumerate(rows):
            val, sts, cnt = rows[k]
            assert vals[i].tolist() == val
            assert np.allclose(state[i], sts.get(st, [0] * dim))
            assert steps[i] == (cnt.get(0, 1 if sts else 0))
    # cut anywhere: an error, never a crash
    for cut in (3, 20, len(body) // 2, len(body) - 1):
        open(path, "wb").write(body[:cut])
        assert api.SparseTable(dim, gi).load_file(path, 21, "t")[0] == api.E_IO


def test_dense_file_round_trip(api, oracle, tmp_path):
    rng = np.random.default_rng(2)
    w0 = rng.standard_normal(24).astype(np.float32)
    for name, type_, conf in [c for c in OPTIM_CASES if c[0] in ("sgd_mom", "adam", "rmsprop_all", "adagrad")]:
        t, ref = api.DenseTable(w0), oracle.DenseTable(w0)
        o_ref, o_gpu = make_optims(oracle, api, type_, conf)
        for step in range(3):
            g = (rng.integers(-64, 65, size=24) / 4096.0).astype(np.float32)
            assert t.Push(o_gpu, g, 0.01) == 0 and ref.push(o_ref, g, 0.01) == 0
        path = str(tmp_path / (name + ".dense"))
        assert t.save(path, 3, "dense0", shape=[4, 6]) == 0
        c = Cursor(open(path, "rb").read())
        assert c.take("B") == 0 and c.take("Q") == 3 and c.string() == "dense0"
        dims, val, st_map, counters = c.value()
        assert c.at == len(c.d) and dims == [4, 6]
        assert_close(val, ref.pull(), "weights in file")
        assert set(st_map) == set(st for st in STATE_OF[type_] if (st != 5 or conf.get("amsgrad")))
        assert counters == ({0: 3} if type_ == 1 else {})
        rc, t2, tid, tname, shape = api.DenseTable.from_file(path)
        assert rc == 0 and tid == 3 and tname == "dense0" and shape == [4, 6]
        for step in range(2):
            g = (rng.integers(-64, 65, size=24) / 4096.0).astype(np.float32)
            assert t2.Push(o_gpu, g, 0.01) == 0 and ref.push(o_ref, g, 0.01) == 0
        assert_close(t2.Pull()[1], ref.pull(), name + " after the file")
    assert api.DenseTable.from_file(str(tmp_path / "none.dense"))[0] == api.E_IO
