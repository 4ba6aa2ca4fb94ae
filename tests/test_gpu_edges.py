"""Edge cases of the id index and of the request sizes: ids built to collide, empty requests,
requests beyond what one launch addresses."""
import ctypes as C

import numpy as np
import pytest

from util import assert_close, make_optims, splitmix64

pytestmark = pytest.mark.gpu

M64 = (1 << 64) - 1


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def _unmix(h):
    """Inverse of the index's hash (the 64-bit finaliser x ^= x >> 33; x *= c1; x ^= x >> 33;
    x *= c2; x ^= x >> 33): every step is a bijection on 64-bit words."""
    c1, c2 = 0xFF51AFD7ED558CCD, 0xC4CEB9FE1A85EC53
    h ^= h >> 33
    h = (h * pow(c2, -1, 1 << 64)) & M64
    h ^= h >> 33
    h = (h * pow(c1, -1, 1 << 64)) & M64
    h ^= h >> 33
    return h


def _mix(x):
    c1, c2 = 0xFF51AFD7ED558CCD, 0xC4CEB9FE1A85EC53
    x ^= x >> 33
    x = (x * c1) & M64
    x ^= x >> 33
    x = (x * c2) & M64
    x ^= x >> 33
    return x


def test_unmix_is_the_inverse():
    for h in (0, 1, 0xDEADBEEF, M64, 0x0123456789ABCDEF):
        assert _mix(_unmix(h)) == h


def test_ids_that_all_probe_from_the_same_bucket(api, oracle):
    """600 ids whose hashes agree in their low 24 bits start from one bucket whatever the table's
    size (up to 2^26 slots): the index degenerates into one chain of 150 buckets. Every
    operation still has to agree with the oracle, through two growths of the table."""
    rng = np.random.default_rng(0)
    dim = 16
    low = 0xABCDE5
    crowd = np.array([_unmix((int(hi) << 24) | low) for hi in rng.integers(1, 1 << 39, size=600)], np.uint64)
    assert len(set(crowd.tolist())) == 600
    others = splitmix64(np.arange(6000, dtype=np.uint64))
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "5"})
    t = api.SparseTable(dim, gi, capacity_hint=64)
    ref = oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=5))
    o_ref, o_gpu = make_optims(oracle, api, 0, {})
    for part in range(3):                               # 200 colliding + 2000 ordinary ids per round
        ids = np.concatenate([crowd[part * 200:(part + 1) * 200], others[part * 2000:(part + 1) * 2000]])
        rng.shuffle(ids)
        rc, rows = t.Pull(np.concatenate([ids, ids[:50]]))        # with repeats in one request
        rc2, want = ref.pull(np.concatenate([ids, ids[:50]]))
        assert rc == 0 and rc2 == 0
        assert_close(rows, want, "pull round %d" % part, rtol=1e-6)
        g = (rng.integers(-64, 65, size=(ids.size, dim)) / 4096.0).astype(np.float32)
        assert t.Push(o_gpu, ids, g, 0.05) == 0 and ref.push(o_ref, ids, g, 0.05) == 0
        assert len(t) == len(ref)
    seen = np.concatenate([crowd, others])
    assert (t.lookup(seen) >= 0).all()
    never = np.array([_unmix((int(hi) << 24) | low) for hi in range(1 << 39, (1 << 39) + 100)], np.uint64)
    assert (t.lookup(never) == -1).all()                 # walks the whole chain and ends at an empty slot
    assert t.Push(o_gpu, never[:3], np.zeros((3, dim), np.float32), 0.05) == api.SPARSE_ID_NOT_EXIST
    assert_close(t.Pull(seen)[1], ref.pull(seen)[1], "after three rounds")
    # taking ids out of the middle of the chain must not cut off the ones behind them
    gone = crowd[100:400]
    assert t.erase(gone) == ref.erase(gone) == 300
    found, vals, _, _ = t.fetch(crowd)
    assert np.array_equal(found, ~np.isin(crowd, gone))
    keep = crowd[found]
    assert_close(vals[found], ref.pull(keep)[1], "chain after erase")
    # raw push of a request made of the colliding ids only
    raw = rng.choice(keep, size=5000)
    g = (rng.integers(-64, 65, size=(raw.size, dim)) / 4096.0).astype(np.float32)
    assert t.PushRaw(o_gpu, raw, g, 0.05) == 0
    u, gs = oracle.dedup_sum(raw, g)
    assert ref.push(o_ref, u, gs, 0.05) == 0
    assert_close(t.Pull(keep)[1], ref.pull(keep)[1], "raw push on the chain")


def test_empty_requests(api, oracle):
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "1"})
    t = api.SparseTable(8, gi)
    none = np.zeros(0, np.uint64)
    nog = np.zeros((0, 8), np.float32)
    _, o = make_optims(oracle, api, 1, {})
    assert t.Pull(none)[0] == 0 and t.Pull(none)[1].shape == (0, 8)
    assert t.Push(o, none, nog, 0.1) == 0 and t.PushRaw(o, none, nog, 0.1) == 0
    assert t.lookup(none).size == 0 and t.erase(none) == 0 and len(t) == 0
    assert t.fetch(none)[0].size == 0
    assert t.export()[0].size == 0
    u, inv = api.dedup(none)
    assert u.size == 0 and inv.size == 0
    assert t.PullPooled(none, np.zeros(1, np.int64))[1].shape == (0, 8)
    assert t.PushPooled(o, none, np.zeros(1, np.int64), nog, 0.1) == 0
    assert len(t) == 0
    d = api.DenseTable(np.zeros(0, np.float32))
    assert d.Pull()[0] == 0 and d.Push(o, np.zeros(0, np.float32), 0.1) == 0
    assert api.coo_to_dense(np.zeros(0, np.int64), np.zeros(0, np.float32), 5).tolist() == [0] * 5


def test_requests_beyond_one_launch_are_refused_up_front(api, oracle):
    """A launch addresses fewer than 2^32 work-items; larger requests return the capacity error
    before anything is read (the pointers here cover only a few elements)."""
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "1"})
    t = api.SparseTable(128, gi)                      # 32 lanes per id
    L = api.lib()
    ids = np.arange(4, dtype=np.uint64)
    buf = np.zeros((4, 128), np.float32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    _, o = make_optims(oracle, api, 0, {})
    huge = 1 << 27                                    # x 32 lanes = 2^32 work-items
    assert L.krk_sparse_pull(t.h, p(ids), huge, p(buf), 0) == api.E_CAPACITY
    assert L.krk_sparse_push(t.h, C.byref(o.raw), p(ids), huge, p(buf), 128, 0.1, 0) == api.E_CAPACITY
    assert L.krk_sparse_push_raw(t.h, C.byref(o.raw), p(ids), (1 << 28) + 1, p(buf), 128, 0.1, 0) == api.E_CAPACITY
    assert L.krk_sparse_lookup(t.h, p(ids), 1 << 30, p(buf), 0) == api.E_CAPACITY
    assert L.krk_sparse_pull(t.h, p(ids), -1, p(buf), 0) == api.E_ARGUMENT
    assert len(t) == 0 and t.Pull(ids)[0] == 0        # the table is untouched and usable


def test_page_locked_host_buffers_are_used_in_place(api, oracle):
    """Host pointers into page-locked memory are handed to the kernels as they are (no staging
    copy); pageable ones and misaligned ones are staged. All three must give the same table and the
    same replies, for a single table, a group and a dense table."""
    dim, n = 16, 5000
    rng = np.random.default_rng(3)
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "2"})
    ids = splitmix64(np.arange(n, dtype=np.uint64))
    g = (rng.integers(-64, 65, size=(n, dim)) / 256.0).astype(np.float32)
    o_ref, o_gpu = make_optims(oracle, api, 0, {})
    r = oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=2))
    _, want0 = r.pull(ids)
    assert r.push(o_ref, ids, g, 0.05) == 0
    _, want1 = r.pull(ids)

    def run(ids_a, g_a, out_a):
        t = api.SparseTable(dim, gi)
        assert t.Pull(ids_a, out=out_a)[0] == 0
        first = np.array(out_a)
        assert t.Push(o_gpu, ids_a, g_a, 0.05) == 0
        assert t.Pull(ids_a, out=out_a)[0] == 0
        return first, np.array(out_a)

    pageable = run(ids, g, np.empty((n, dim), np.float32))
    locked = run(api.pinned_copy(ids), api.pinned_copy(g), api.pinned_empty((n, dim), np.float32))
    # page-locked but off the 16-byte grid: staged like pageable memory
    raw_i = api.pinned_empty(n + 1, np.uint64)
    raw_g = api.pinned_empty(n * dim + 1, np.float32)
    raw_o = api.pinned_empty(n * dim + 1, np.float32)
    raw_i[1:] = ids
    raw_g[1:] = g.ravel()
    skewed = run(raw_i[1:], raw_g[1:].reshape(n, dim), raw_o[1:].reshape(n, dim))
    for got in (pageable, locked, skewed):
        assert_close(got[0], want0, "first pull", rtol=1e-6)
        assert_close(got[1], want1, "after push")
    assert np.array_equal(pageable[0], locked[0]) and np.array_equal(pageable[1], locked[1])
    assert np.array_equal(pageable[1], skewed[1])

    # a group and a dense table through page-locked buffers
    a, b = api.SparseTable(dim, gi), api.SparseTable(dim, gi)
    grp = api.TableGroup([a, b])
    off = [0, n // 2, n]
    p_ids, p_g, p_out = api.pinned_copy(ids), api.pinned_copy(g), api.pinned_empty((n, dim), np.float32)
    assert grp.CombinePull(p_ids, off, out=p_out)[0] == 0
    assert np.array_equal(np.array(p_out), pageable[0])
    assert grp.CombinePush(o_gpu, p_ids, off, p_g, 0.05) == 0
    assert grp.CombinePull(p_ids, off, out=p_out)[0] == 0
    assert np.array_equal(np.array(p_out), pageable[1])
    grp.close()
    w0 = rng.standard_normal(1000).astype(np.float32)
    d1, d2 = api.DenseTable(w0), api.DenseTable(api.pinned_copy(w0))
    gd = rng.standard_normal(1000).astype(np.float32)
    adam = api.Optim.create(api.OptimType.kAdam)
    assert d1.Push(adam, gd, 0.01) == 0 and d2.Push(adam, api.pinned_copy(gd), 0.01) == 0
    out2 = api.pinned_empty(1000, np.float32)
    assert d2.Pull(out=out2)[0] == 0
    assert np.array_equal(d1.Pull()[1], np.array(out2))
