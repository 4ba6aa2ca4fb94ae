"""KRK_NOTE_ROWS / KRK_IDS_AS_PULLED: a pull that keeps the row of every position and a push_raw of
the same ids that uses them instead of looking the ids up again (the worker's own sequence,
worker/emitter.cc:131-182 then 510-531, 552-612 for combined requests).

Bar: bit-exact against the same calls without the flags (the flags change where the row numbers
come from, not what is added up or in which order), for new and resident ids, narrow and wide rows,
single tables and groups; every condition under which the notes must not be used falls back to the
look-up; and one check that the notes, not a look-up, are what the flagged call reads."""
import numpy as np
import pytest

from util import zipf_ids

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def _init(api):
    return api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.05", "seed": "21"})


def _h2d(api, dst, a):
    a = np.ascontiguousarray(a)
    assert a.nbytes == dst.nbytes
    api._check(api.lib().krk_memcpy_h2d(api.C.c_void_p(dst.ptr), a.ctypes.data_as(api.C.c_void_p), a.nbytes), "h2d")


def _same_tables(api, a, b, states):
    """weights, step counters and the given optimizer columns of two tables, id by id"""
    ea, eb = a.export(), b.export()
    oa, ob = np.argsort(ea[0]), np.argsort(eb[0])
    assert np.array_equal(ea[0][oa], eb[0][ob])
    assert np.array_equal(ea[1][oa], eb[1][ob])
    assert np.array_equal(ea[3][oa], eb[3][ob])
    for st in states:
        assert np.array_equal(a.export(st)[2][oa], b.export(st)[2][ob])


@pytest.mark.parametrize("dim", [16, 32, 5])
@pytest.mark.parametrize("optim", ["adagrad", "adam"])
def test_single_table_with_notes_equals_without(api, dim, optim):
    """Three steps of pull + push_raw over 8192 Zipf positions (fresh ids every step: the pull
    inserts them, the notes name rows that did not exist before), with and without the flags."""
    rng = np.random.default_rng(dim)
    o = api.Optim.create(api.OptimType.kAdagrad if optim == "adagrad" else api.OptimType.kAdam)
    a, b = api.SparseTable(dim, _init(api)), api.SparseTable(dim, _init(api))
    n = 8192
    seen = []
    d_ids = api.DeviceArray(n, np.uint64)
    d_g = api.DeviceArray((n, dim), np.float32)
    for step in range(3):
        ids = zipf_ids(rng, 1.1, 20000, n) + np.uint64(step * 5000)
        g = (rng.standard_normal((n, dim)) * 0.1).astype(np.float32)
        _h2d(api, d_ids, ids)
        _h2d(api, d_g, g)
        seen.append(ids)
        rc, va = a.Pull(d_ids, note_rows=True)
        assert rc == 0
        rc, vb = b.Pull(d_ids)
        assert rc == 0
        assert np.array_equal(va.to_host(), vb.to_host())
        assert a.PushRaw(o, d_ids, d_g, 0.05, as_pulled=True) == 0
        assert b.PushRaw(o, d_ids, d_g, 0.05) == 0
    u = np.unique(np.concatenate(seen))
    assert np.array_equal(a.Pull(u)[1], b.Pull(u)[1])
    S = api.StateType
    _same_tables(api, a, b, [S.kStateSum] if optim == "adagrad" else [S.kFirstMoment, S.kSecondMoment])
    for t in (a, b):
        t.close()


def test_notes_are_what_the_flagged_push_reads(api):
    """Pull X with the flag, overwrite the buffer with other ids Y, push with the flag: the rows of
    X are updated and those of Y are not (the header says so). Without the flag Y's rows move."""
    dim, n = 16, 4096
    o = api.Optim.create(api.OptimType.kSGD)
    t = api.SparseTable(dim, _init(api))
    x = np.arange(1, n + 1, dtype=np.uint64)
    y = x + np.uint64(100000)
    t.Pull(y)
    before_y = t.Pull(y)[1]
    d_ids = api.DeviceArray.from_host(x)
    d_g = api.DeviceArray.from_host(np.ones((n, dim), np.float32))
    rc, vx = t.Pull(d_ids, note_rows=True)
    before_x = vx.to_host()
    _h2d(api, d_ids, y)
    assert t.PushRaw(o, d_ids, d_g, 0.5, as_pulled=True) == 0
    assert np.array_equal(t.Pull(y)[1], before_y)
    assert np.array_equal(t.Pull(x)[1], before_x - np.float32(0.5))
    assert t.PushRaw(o, d_ids, d_g, 0.5) == 0                       # no flag: looked up, Y it is
    assert np.array_equal(t.Pull(y)[1], before_y - np.float32(0.5))
    assert np.array_equal(t.Pull(x)[1], before_x - np.float32(0.5))
    t.close()


def test_notes_are_dropped_when_they_do_not_apply(api):
    """Another buffer, another count, an erase in between, a pull above 8192 ids, a later flagged
    pull of other ids: each time the flagged push_raw must act on the ids it is given."""
    dim = 16
    o = api.Optim.create(api.OptimType.kSGD)
    t = api.SparseTable(dim, _init(api))
    rng = np.random.default_rng(3)
    x = rng.permutation(np.arange(1, 6001, dtype=np.uint64))
    y = x[::-1].copy() + np.uint64(50000)
    t.Pull(y)
    d_x = api.DeviceArray.from_host(x)
    d_y = api.DeviceArray.from_host(y)
    g = np.ones((x.size, dim), np.float32)
    d_g = api.DeviceArray.from_host(g)
    lr = np.float32(0.25)

    def check(ids_dev, ids_host, n=None):
        n = ids_host.size if n is None else n
        want_moved = t.Pull(ids_host[:n])[1] - lr
        others = np.concatenate([x, y])
        others = others[~np.isin(others, ids_host[:n])]
        want_still = t.Pull(others)[1]
        sub = ids_dev if n == ids_host.size else _prefix(ids_dev, n)
        subg = d_g if n == ids_host.size else _prefix(d_g, n)
        assert t.Push(o, sub, subg, float(lr), raw=True, as_pulled=True) == 0
        assert np.array_equal(t.Pull(ids_host[:n])[1], want_moved)
        assert np.array_equal(t.Pull(others)[1], want_still)

    class _View(api.DeviceArray):
        def __init__(self, base, n):                     # first n rows of base, same pointer
            self.shape = (n,) + base.shape[1:]
            self.dtype = base.dtype
            self.size = int(np.prod(self.shape))
            self.nbytes = self.size * self.dtype.itemsize
            self.ptr = base.ptr
            self.base = base

        def free(self):
            self.ptr = None

    def _prefix(d, n):
        return _View(d, n)

    assert t.Pull(d_x, note_rows=True)[0] == 0
    check(d_y, y)                                        # another buffer
    assert t.Pull(d_x, note_rows=True)[0] == 0
    check(d_x, x, n=3000)                                # same pointer, another count
    assert t.Pull(d_x, note_rows=True)[0] == 0
    gone = np.arange(200000, 200100, dtype=np.uint64)
    t.Pull(gone)
    t.erase(np.concatenate([gone, x[:500]]))             # rows move: x[:500] vanish, others renumbered
    # the erased ids are unknown to the table now: the flagged push must say so, not update stale rows
    rc = t.Push(o, d_x, d_g, float(lr), raw=True, as_pulled=True)
    assert rc == 12
    t.Pull(x[:500])
    big = np.arange(300000, 300000 + 9000, dtype=np.uint64)
    d_big = api.DeviceArray.from_host(big)
    d_gbig = api.DeviceArray.from_host(np.ones((big.size, dim), np.float32))
    assert t.Pull(d_big, note_rows=True)[0] == 0         # noted, but a push_raw this long sorts by itself
    before = t.Pull(big)[1]
    assert t.Push(o, d_big, d_gbig, float(lr), raw=True, as_pulled=True) == 0
    assert np.array_equal(t.Pull(big)[1], before - lr)
    assert t.Pull(d_x, note_rows=True)[0] == 0
    assert t.Pull(d_y, note_rows=True)[0] == 0           # the later pull's notes replace the earlier
    check(d_x, x)
    t.close()


@pytest.mark.parametrize("dim", [16, 64])
def test_group_with_notes_equals_without(api, dim):
    """Five tables, ragged requests (one empty, one of a single id, one of 8192), Adagrad, three
    steps with fresh ids: combined pull + push_raw with and without the flags, bit for bit."""
    rng = np.random.default_rng(dim + 1)
    o = api.Optim.create(api.OptimType.kAdagrad)
    counts = [3000, 0, 1, 8192, 777]
    ta = [api.SparseTable(dim, _init(api)) for _ in counts]
    tb = [api.SparseTable(dim, _init(api)) for _ in counts]
    ga, gb = api.TableGroup(ta), api.TableGroup(tb)
    off = ga._offsets(counts)
    total = int(off[-1])
    d_ids = api.DeviceArray(total, np.uint64)
    d_g = api.DeviceArray((total, dim), np.float32)
    seen = [[] for _ in counts]
    for step in range(3):
        per = [zipf_ids(rng, 1.05, 30000, c) + np.uint64(step * 7000) for c in counts]
        for s, p in zip(seen, per):
            s.append(p)
        _h2d(api, d_ids, np.concatenate(per))
        _h2d(api, d_g, (rng.standard_normal((total, dim)) * 0.1).astype(np.float32))
        rc, va = ga.CombinePull(d_ids, off, note_rows=True)
        assert rc == 0
        rc, vb = gb.CombinePull(d_ids, off)
        assert rc == 0
        assert np.array_equal(va.to_host(), vb.to_host())
        assert ga.CombinePushRaw(o, d_ids, off, d_g, 0.05, as_pulled=True) == 0
        assert gb.CombinePushRaw(o, d_ids, off, d_g, 0.05) == 0
    for a, b, s in zip(ta, tb, seen):
        u = np.unique(np.concatenate(s))
        if u.size:
            assert np.array_equal(a.Pull(u)[1], b.Pull(u)[1])
            _same_tables(api, a, b, [api.StateType.kStateSum])
    # other offsets with the same buffer: looked up again
    counts2 = [3000, 0, 1, 8192 - 5, 777 + 5]
    off2 = ga._offsets(counts2)
    assert ga.CombinePushRaw(o, d_ids, off2, d_g, 0.05, as_pulled=True) in (0, 12)
    ga.close()
    gb.close()


@pytest.mark.parametrize("dim", [16, 64, 5])
@pytest.mark.parametrize("optim", ["adagrad", "adam"])
def test_push_of_unique_ids_with_notes_equals_without(api, dim, optim):
    """krk_sparse_push after a noting pull of the same unique ids (narrow rows, the wide kernels,
    rows that are no multiple of four floats), three steps with fresh ids, against the plain calls."""
    rng = np.random.default_rng(100 + dim)
    o = api.Optim.create(api.OptimType.kAdagrad if optim == "adagrad" else api.OptimType.kAdam)
    a, b = api.SparseTable(dim, _init(api)), api.SparseTable(dim, _init(api))
    for step in range(3):
        ids = np.unique(zipf_ids(rng, 1.05, 40000, 12000) + np.uint64(step * 9000))
        rng.shuffle(ids)
        d_ids = api.DeviceArray.from_host(ids)
        d_g = api.DeviceArray.from_host((rng.standard_normal((ids.size, dim)) * 0.1).astype(np.float32))
        assert a.Pull(d_ids, note_rows=True)[0] == 0
        assert b.Pull(d_ids)[0] == 0
        assert a.Push(o, d_ids, d_g, 0.05, as_pulled=True) == 0
        assert b.Push(o, d_ids, d_g, 0.05) == 0
    S = api.StateType
    _same_tables(api, a, b, [S.kStateSum] if optim == "adagrad" else [S.kFirstMoment, S.kSecondMoment])
    a.close()
    b.close()


def test_flagged_push_reads_the_notes_and_drops_stale_ones(api):
    """As for push_raw: with the buffer overwritten after the pull the flagged push updates the
    rows that were pulled; after an erase it looks the ids up (and reports the missing ones)."""
    dim, n = 32, 5000
    o = api.Optim.create(api.OptimType.kSGD)
    t = api.SparseTable(dim, _init(api))
    x = np.arange(1, n + 1, dtype=np.uint64)
    y = x + np.uint64(100000)
    t.Pull(y)
    before_y = t.Pull(y)[1]
    d_ids = api.DeviceArray.from_host(x)
    d_g = api.DeviceArray.from_host(np.ones((n, dim), np.float32))
    before_x = t.Pull(d_ids, note_rows=True)[1].to_host()
    _h2d(api, d_ids, y)
    assert t.Push(o, d_ids, d_g, 0.5, as_pulled=True) == 0
    assert np.array_equal(t.Pull(y)[1], before_y)
    assert np.array_equal(t.Pull(x)[1], before_x - np.float32(0.5))
    _h2d(api, d_ids, x)
    assert t.Pull(d_ids, note_rows=True)[0] == 0
    t.erase(x[:100])
    assert t.Push(o, d_ids, d_g, 0.5, as_pulled=True) == 12            # the erased ids are gone
    assert np.array_equal(t.Pull(x[100:])[1], before_x[100:] - np.float32(0.5) - np.float32(0.5))
    t.close()


@pytest.mark.parametrize("dim", [16, 32, 64])
def test_group_push_of_unique_ids_with_notes_equals_without(api, dim):
    rng = np.random.default_rng(7 + dim)
    o = api.Optim.create(api.OptimType.kAdagrad)
    counts = [3790, 0, 1, 9000, 64]
    ta = [api.SparseTable(dim, _init(api)) for _ in counts]
    tb = [api.SparseTable(dim, _init(api)) for _ in counts]
    ga, gb = api.TableGroup(ta), api.TableGroup(tb)
    off = ga._offsets(counts)
    total = int(off[-1])
    for step in range(3):
        per = [rng.permutation(np.arange(1, 20001, dtype=np.uint64))[:c] + np.uint64(step * 3000) for c in counts]
        d_ids = api.DeviceArray.from_host(np.concatenate(per))
        d_g = api.DeviceArray.from_host((rng.standard_normal((total, dim)) * 0.1).astype(np.float32))
        assert ga.CombinePull(d_ids, off, note_rows=True)[0] == 0
        assert gb.CombinePull(d_ids, off)[0] == 0
        assert ga.CombinePush(o, d_ids, off, d_g, 0.05, as_pulled=True) == 0
        assert gb.CombinePush(o, d_ids, off, d_g, 0.05) == 0
    for a, b, c in zip(ta, tb, counts):
        if c:
            _same_tables(api, a, b, [api.StateType.kStateSum])
    ga.close()
    gb.close()
