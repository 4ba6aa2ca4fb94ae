"""Table files in the reference's checkpoint layout (checkpoint/checkpoint.cc:444-509, 535-649,
common/serialize.h).

The byte layout is pinned by files that the reference's own serializer wrote (tests/golden/
ref_*.sparse, ref_*.dense, made by oracle/ref_checkpoint.cc from the reference's serialize.h and
tensor sources compiled in place): the library loads them, and what the library writes is read
back by the reference's own deserializer where that binary is present. The `struct` reader in
checkpoint_format.py is a second reading of common/serialize.h, pinned against the same files.
"""
import os
import struct
import subprocess

import numpy as np
import pytest

from util import OPTIM_CASES, STATE_OF, assert_close, make_optims, splitmix64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


from checkpoint_format import Cursor, pack_string, pack_value, parse_sparse  # noqa: E402


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
            assert steps[i] == cnt.get(0, 0)
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


# --- files written / read by the reference's own serializer -------------------------------------

from test_checkpoint_format import GOLDEN, SPARSE, expected_rows, pattern  # noqa: E402

REF_TOOL = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle", "_ref", "ref_checkpoint")


@pytest.mark.parametrize("name,dim,rows,states,steps", SPARSE)
def test_loads_sparse_files_the_reference_wrote(api, name, dim, rows, states, steps):
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01"})
    t = api.SparseTable(dim, gi)
    rc, taken = t.load_file(os.path.join(GOLDEN, name + ".sparse"), 7, "emb")
    assert rc == 0 and taken == rows == len(t)
    want = expected_rows(dim, rows, states, steps)
    keys = np.array(list(want), np.uint64)
    for st in range(1, 8):
        found, vals, state, got_steps = t.fetch(keys, state_type=st)
        assert found.all()
        for i, k in enumerate(want):
            w_val, w_st, w_cnt = want[k]
            assert np.array_equal(vals[i], w_val)
            assert np.array_equal(state[i], w_st.get(st, np.zeros(dim, np.float32)))
            assert got_steps[i] == (w_cnt[0] if w_cnt else 0)


@pytest.mark.parametrize("name,dim,rows,states,steps", SPARSE)
def test_writes_what_the_reference_wrote(api, tmp_path, name, dim, rows, states, steps):
    """The same table content saved by the library: identical bytes where the layout leaves no
    freedom (at most one state), the same parsed content otherwise (the reference emits several
    states in its hash map's order)."""
    golden_path = os.path.join(GOLDEN, name + ".sparse")
    gi = api.Initializer.create(api.InitializerType.kNormal, {"mean": "0.0", "stddev": "0.01"})
    t = api.SparseTable(dim, gi)
    assert t.load_file(golden_path, 7, "emb")[0] == 0
    path = str(tmp_path / "again.sparse")
    assert t.save(path, 7, "emb") == 0
    got, want = open(path, "rb").read(), open(golden_path, "rb").read()
    if len(states) <= 1:
        # the two conf entries may come in either order (an unordered_map on the reference's side)
        assert len(got) == len(want)
        a, b = parse_sparse(path), parse_sparse(golden_path)
        assert a[0] == b[0]

        def after_conf(data):
            c = Cursor(data)
            c.take("B"), c.take("Q"), c.string(), c.take("q"), c.take("B"), c.take("B")
            for _ in range(c.take("Q")):
                c.string(), c.string()
            return data[c.at:]

        assert got[:len(got) - len(after_conf(got))][:21] == want[:21]     # up to the conf map
        assert after_conf(got) == after_conf(want)
    a, b = parse_sparse(path), parse_sparse(golden_path)
    assert a[0] == b[0]
    for rows_a, rows_b in zip(a[1], b[1]):
        assert len(rows_a) == len(rows_b)
        for ra, rb in zip(rows_a, rows_b):
            assert ra[0] == rb[0] and ra[1] == rb[1] and np.array_equal(ra[2], rb[2])
            assert set(ra[3]) == set(rb[3]) and all(np.array_equal(ra[3][s], rb[3][s]) for s in ra[3])
            assert ra[4] == rb[4]


def test_dense_file_the_reference_wrote(api, tmp_path):
    rc, t, tid, tname, shape = api.DenseTable.from_file(os.path.join(GOLDEN, "ref_adam.dense"))
    assert rc == 0 and tid == 3 and tname == "dense0" and shape == [6, 4]
    assert np.array_equal(t.Pull()[1], pattern(99, 0, 24))
    assert np.array_equal(t.state(3), pattern(99, 4, 24)) and np.array_equal(t.state(4), pattern(99, 5, 24))
    assert t.steps == 12
    path = str(tmp_path / "again.dense")
    assert t.save(path, 3, "dense0", shape=[6, 4]) == 0
    from checkpoint_format import parse_dense
    a, b = parse_dense(path), parse_dense(os.path.join(GOLDEN, "ref_adam.dense"))
    assert a[0] == b[0] and a[1] == b[1] and np.array_equal(a[2], b[2]) and a[4] == b[4]
    assert set(a[3]) == set(b[3]) and all(np.array_equal(a[3][s], b[3][s]) for s in a[3])


@pytest.mark.skipif(not os.path.exists(REF_TOOL), reason="oracle/_ref/ref_checkpoint is built only where the "
                    "reference tree is present")
def test_reference_reader_reads_what_the_library_writes(api, oracle, tmp_path):
    """A table trained on the GPU, saved by the library, parsed by the reference's own
    Deserialize (oracle/ref_checkpoint.cc dump-sparse / dump-dense): every number it prints is
    the oracle table's."""
    dim = 8
    t, ref = _tables(api, oracle, dim, seed=6)
    ids = splitmix64(np.arange(300, dtype=np.uint64))
    t.Pull(ids)
    ref.pull(ids)
    o_ref, o_gpu = make_optims(oracle, api, 1, {})
    g = (np.random.default_rng(0).integers(-64, 65, size=(150, dim)) / 4096.0).astype(np.float32)
    for _ in range(3):
        assert t.Push(o_gpu, ids[:150], g, 0.01) == 0 and ref.push(o_ref, ids[:150], g, 0.01) == 0
    path = str(tmp_path / "gpu.sparse")
    assert t.save(path, 7, "emb") == 0
    text = subprocess.run([REF_TOOL, "dump-sparse", path], check=True, capture_output=True, text=True).stdout
    lines = text.splitlines()
    assert lines[0] == "type 1 id 7 name emb dim 8 dtype 11 init 2 conf mean=0.000000 stddev=0.010000"
    assert lines[1] == "slots 8"
    rid, rval, _, rsteps = ref.export()
    m = ref.export(state_type=3)[2]
    v = ref.export(state_type=4)[2]
    by_id = {int(k): i for i, k in enumerate(rid)}
    seen = 0
    for ln in lines[2:]:
        if ln.startswith("slot "):
            continue
        parts = ln.split(" | ")
        head = parts[0].split()
        assert head[0] == "id" and head[2] == "val" and head[3] == "[8]"
        i = by_id[int(head[1])]
        assert_close(np.array(head[4:], np.float32), rval[i], "weights the reference read")
        fields = {p.split()[0] + " " + p.split()[1]: p.split()[2:] for p in parts[1:]}
        if rsteps[i] > 0:
            assert_close(np.array(fields["state 3"][1:], np.float32), m[i], "first moment")
            assert_close(np.array(fields["state 4"][1:], np.float32), v[i], "second moment")
            assert int(fields["int 0"][0]) == rsteps[i] == 3
        else:
            assert not fields
        seen += 1
    assert seen == 300

    d = api.DenseTable(np.arange(12, dtype=np.float32))
    assert d.Push(o_gpu, np.ones(12, np.float32), 0.5) == 0
    dpath = str(tmp_path / "gpu.dense")
    assert d.save(dpath, 3, "dense0", shape=[3, 4]) == 0
    dl = subprocess.run([REF_TOOL, "dump-dense", dpath], check=True, capture_output=True, text=True).stdout.splitlines()
    assert dl[0] == "type 0 id 3 name dense0"
    assert dl[1].startswith("val [3x4] ") and " | state 3 [3x4] " in dl[1] and dl[1].endswith(" | int 0 1")


# --- requests and replies in the reference's wire layout -----------------------------------------

from checkpoint_format import pack_rows, parse_rows  # noqa: E402


@pytest.mark.parametrize("dim", [5, 16])
def test_pull_and_push_in_wire_layout(api, oracle, tmp_path, dim):
    """krk_sparse_pull_wire writes what the reference's Serialize writes for the pulled rows
    (checked byte for byte against a block the reference wrote, and read back by its Deserialize
    where that binary is present); krk_sparse_push_wire applies a block the reference wrote."""
    from test_checkpoint_format import mix
    golden = np.frombuffer(open(os.path.join(GOLDEN, "ref_rows_d%d.wire" % dim), "rb").read(), np.uint8)
    rows = parse_rows(golden)
    n = rows.shape[0]
    ids = np.array([mix(r) for r in range(n)], np.uint64)
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "0"})
    t = api.SparseTable(dim, gi)
    r = oracle.SparseTable(dim, oracle.init(oracle.INIT_CONSTANT, 0.0))
    t.Pull(ids)
    r.pull(ids)
    # SGD with lr -1 on zero rows: the rows become the gradients the reference serialized
    o_ref, o_gpu = make_optims(oracle, api, 3, {})
    wire = np.empty(golden.size // 8 + 1, np.uint64).view(np.uint8)[:golden.size]
    wire[:] = golden
    assert t.PushWire(o_gpu, ids, wire, -1.0) == 0
    assert r.push(o_ref, ids, rows, -1.0) == 0
    assert np.array_equal(t.Pull(ids)[1], rows) and np.array_equal(r.pull(ids)[1], rows)
    rc, reply = t.PullWire(ids)
    assert rc == 0 and reply.tobytes() == golden.tobytes()
    # page-locked buffers take the in-place path
    p_reply = api.pinned_empty(golden.size, np.uint8)
    assert t.PullWire(ids, reply=p_reply)[0] == 0 and np.array_equal(np.array(p_reply), golden)
    p_wire = api.pinned_copy(golden)
    assert t.PushWire(o_gpu, ids, p_wire, -1.0) == 0
    assert np.array_equal(t.Pull(ids)[1], 2 * rows)
    # a reply for ids in another order, with a new id, equals the struct writer's bytes
    mixed = np.concatenate([ids[::-1][:7], np.array([12345], np.uint64)])
    rc, reply = t.PullWire(mixed)
    assert rc == 0 and reply.tobytes() == pack_rows(t.Pull(mixed)[1])
    if os.path.exists(REF_TOOL):
        path = str(tmp_path / "reply.wire")
        open(path, "wb").write(reply.tobytes())
        text = subprocess.run([REF_TOOL, "dump-rows", path], check=True, capture_output=True, text=True).stdout
        lines = text.splitlines()
        assert lines[0] == "rows 8"
        got = np.array([ln.split()[1:] for ln in lines[1:]], np.float32)
        assert np.array_equal(got, t.Pull(mixed)[1])
    # malformed requests are refused whole: wrong count, wrong width, short buffer, a COO row
    before = t.Pull(ids)[1]
    bad = wire.copy()
    bad[0] = n - 1
    assert t.PushWire(o_gpu, ids, bad, 1.0) == 11
    bad = wire.copy()
    bad[8 + 9] = dim + 1
    assert t.PushWire(o_gpu, ids, bad, 1.0) == 11
    assert t.PushWire(o_gpu, ids, wire[:-4], 1.0) == 11
    bad = wire.copy()
    bad[8 + 3 * (18 + 4 * dim)] = 1
    assert t.PushWire(o_gpu, ids, bad, 1.0) == 11
    assert np.array_equal(t.Pull(ids)[1], before)
    assert t.PushWire(o_gpu, ids[:0], np.zeros(8, np.uint8), 1.0) == 0
    rc, empty = t.PullWire(ids[:0])
    assert rc == 0 and empty.tobytes() == struct.pack("<Q", 0)


def test_file_of_a_table_larger_than_the_writers_chunks(api, tmp_path):
    """2.5 million rows: the writer and the loader both walk the table in chunks of 2^20 rows;
    rows, states and counters on the far side of a chunk border must come through."""
    dim, n = 4, 2_500_000
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.05", "seed": "8"})
    t = api.SparseTable(dim, gi, capacity_hint=n)
    ids = splitmix64(np.arange(n, dtype=np.uint64))
    assert t.Pull(api.DeviceArray.from_host(ids), async_=True)[0] == 0
    o = api.Optim.create(api.OptimType.kAdam)
    touched = ids[::3]
    g = (np.random.default_rng(0).integers(-64, 65, size=(touched.size, dim)) / 1024.0).astype(np.float32)
    assert t.Push(o, touched, g, 0.01) == 0
    path = str(tmp_path / "big.sparse")
    assert t.save(path, 9, "big") == 0
    t2 = api.SparseTable(dim, gi)
    rc, taken = t2.load_file(path, 9, "big")
    assert rc == 0 and taken == n == len(t2)
    probe = np.concatenate([ids[:1000], ids[(1 << 20) - 500:(1 << 20) + 500], ids[-1000:], touched[-1000:]])
    for st in (3, 4):
        fa, va, sa, ca = t.fetch(probe, state_type=st)
        fb, vb, sb, cb = t2.fetch(probe, state_type=st)
        assert fa.all() and fb.all()
        assert np.array_equal(va, vb) and np.array_equal(sa, sb) and np.array_equal(ca, cb)
    a_id, a_val, _, a_steps = t.export()
    b_id, b_val, _, b_steps = t2.export()
    oa, ob = np.argsort(a_id), np.argsort(b_id)
    assert np.array_equal(a_id[oa], b_id[ob]) and np.array_equal(a_val[oa], b_val[ob])
    assert np.array_equal(a_steps[oa], b_steps[ob]) and int(a_steps.sum()) == touched.size


def test_load_leaves_rows_that_exist_untouched(api, oracle, tmp_path):
    """checkpoint/checkpoint.cc:640 inserts each Value with SkipList::Insert, which does nothing
    for an id that is present (common/skip_list.h:240-242): a row the table already holds keeps
    its weights, its optimizer state and its counter, all three; only absent ids come in."""
    dim = 8
    t, ref = _tables(api, oracle, dim, seed=5)
    ids = splitmix64(np.arange(3000, dtype=np.uint64))
    o_ref, o_gpu = make_optims(oracle, api, 1, {})                      # Adam: two states and a counter
    assert t.Pull(ids)[0] == 0 and ref.pull(ids)[0] == 0
    g = (np.random.default_rng(1).integers(-64, 65, size=(ids.size, dim)) / 4096.0).astype(np.float32)
    assert t.Push(o_gpu, ids, g, 0.01) == 0 and ref.push(o_ref, ids, g, 0.01) == 0
    path = str(tmp_path / "a.sparse")
    assert t.save(path, 3, "a") == 0

    # the receiving table holds every third id already, trained differently (three updates)
    t2, ref2 = _tables(api, oracle, dim, seed=9)
    mine = ids[::3]
    assert t2.Pull(mine)[0] == 0 and ref2.pull(mine)[0] == 0
    for step in range(3):
        g2 = (np.random.default_rng(10 + step).integers(-64, 65, size=(mine.size, dim)) / 4096.0).astype(np.float32)
        assert t2.Push(o_gpu, mine, g2, 0.02) == 0 and ref2.push(o_ref, mine, g2, 0.02) == 0
    rc, taken = t2.load_file(path, 3, "a")
    assert rc == 0 and taken == ids.size and len(t2) == ids.size
    other = np.setdiff1d(ids, mine)
    for st in (3, 4):
        found, vals, state, steps = t2.fetch(mine, state_type=st)
        assert found.all() and (steps == 3).all()                        # its own counter, not the file's 1
        assert_close(vals, ref2.pull(mine)[1], "weights of rows that were present")
        assert_close(state, _oracle_state(ref2, mine, st), "state %d of rows that were present" % st)
        found, vals, state, steps = t2.fetch(other, state_type=st)
        assert found.all() and (steps == 1).all()
        assert_close(vals, ref.pull(other)[1], "weights of rows from the file")
        assert_close(state, _oracle_state(ref, other, st), "state %d of rows from the file" % st)
    # and both kinds keep training like the oracle's rows
    g3 = (np.random.default_rng(77).integers(-64, 65, size=(ids.size, dim)) / 4096.0).astype(np.float32)
    assert t2.Push(o_gpu, ids, g3, 0.01) == 0
    pos = {int(k): i for i, k in enumerate(ids.tolist())}
    sel_m = np.array([pos[int(k)] for k in mine]); sel_o = np.array([pos[int(k)] for k in other])
    assert ref2.push(o_ref, mine, g3[sel_m], 0.01) == 0 and ref.push(o_ref, other, g3[sel_o], 0.01) == 0
    assert_close(t2.Pull(mine)[1], ref2.pull(mine)[1], "present rows after one more step")
    assert_close(t2.Pull(other)[1], ref.pull(other)[1], "loaded rows after one more step")


def _oracle_state(ref, ids, st):
    rid, _, state, _ = ref.export(state_type=st)
    where = {int(k): i for i, k in enumerate(rid.tolist())}
    return state[[where[int(k)] for k in ids.tolist()]]


def test_zero_momentum_buffer_survives_the_file(api, oracle, tmp_path):
    """A row whose first SGD-with-momentum update had an all-zero gradient holds a momentum buffer
    of zeros. It is a buffer all the same: the row's next update continues it,
    buf = momentum * buf + (1 - dampening) * g (ps/optim/sgd.cc:46-52), where a row without a buffer
    would take buf = g. With dampening != 0 the two differ, so the file must carry the buffer."""
    dim = 8
    t, ref = _tables(api, oracle, dim, seed=6)
    ids = splitmix64(np.arange(500, dtype=np.uint64))
    o_ref, o_gpu = make_optims(oracle, api, 3, {"momentum": 0.8, "dampening": 0.3})
    assert t.Pull(ids)[0] == 0 and ref.pull(ids)[0] == 0
    g0 = np.zeros((ids.size, dim), np.float32)
    g0[::2] = 0.125                                                    # every second row: a zero first gradient
    assert t.Push(o_gpu, ids, g0, 0.1) == 0 and ref.push(o_ref, ids, g0, 0.1) == 0
    path = str(tmp_path / "m.sparse")
    assert t.save(path, 4, "m") == 0
    _, slots = parse_sparse(path)
    assert all(1 in r[3] for rows in slots for r in rows)              # every row carries its buffer
    t2, _ = _tables(api, oracle, dim, seed=6)
    assert t2.load_file(path, 4, "m") == (0, ids.size)
    g1 = np.full((ids.size, dim), 0.25, np.float32)
    assert t2.Push(o_gpu, ids, g1, 0.1) == 0 and ref.push(o_ref, ids, g1, 0.1) == 0
    assert_close(t2.Pull(ids)[1], ref.pull(ids)[1], "update after the file continues the zero buffer")


def test_malformed_sparse_files_are_errors(api, tmp_path):
    """Lengths that no file could back (a tensor of 2^40 elements, a string of 2^31 bytes, dims whose
    product overflows) are refused before anything is allocated for them."""
    dim = 4
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "0.25"})
    head = struct.pack("<BQ", 1, 21) + pack_string("t") + struct.pack("<qBB", dim, 11, 0)
    head += struct.pack("<Q", 1) + pack_string("value") + pack_string("0.250000") + struct.pack("<Q", 1)
    cases = {
        "huge tensor": head + struct.pack("<Q", 1) + struct.pack("<Q", 5) + struct.pack("<BQqB", 0, 1, 1 << 40, 11),
        "overflowing dims": head + struct.pack("<Q", 1) + struct.pack("<Q", 5) +
                            struct.pack("<BQ", 0, 3) + struct.pack("<qqq", 1 << 31, 1 << 31, 1 << 31) + b"\x0b",
        "huge name": struct.pack("<BQ", 1, 21) + struct.pack("<Q", 1 << 31) + b"t",
        "huge conf value": struct.pack("<BQ", 1, 21) + pack_string("t") + struct.pack("<qBB", dim, 11, 0) +
                           struct.pack("<Q", 1) + pack_string("value") + struct.pack("<Q", 1 << 33),
    }
    for what, body in cases.items():
        path = str(tmp_path / "bad.sparse")
        open(path, "wb").write(body)
        t = api.SparseTable(dim, gi)
        assert t.load_file(path, 21, "t")[0] == api.E_IO, what
        assert len(t) == 0
