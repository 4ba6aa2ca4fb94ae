"""Combined requests over several tables (Ps::CombinePullSparseTable / CombinePushSparseTable,
ps/ps_op.cc:370-387, 456-469) served by one launch, against the oracle looping over tables the
way the reference does. Shape of the reference's own test: emitter_test.cc:75-87, 112-158
(two tables, Constant init, SGD, combined pull and combined push)."""
import numpy as np
import pytest

from util import OPTIM_CASES, assert_close, make_optims, splitmix64, zipf_ids

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def test_emitter_test_combined_shape(api, oracle):
    """emitter_test.cc:75-87 and 134-158: CombinePull on two Constant tables, CombinePush with
    SGD, after == before - lr * grad."""
    v0, v1 = 7.5, -3.25
    t0 = api.SparseTable(100, api.Initializer.create(0, {"value": repr(v0)}))
    t1 = api.SparseTable(100, api.Initializer.create(0, {"value": repr(v1)}))
    g = api.TableGroup([t0, t1])
    ids = np.array([0, 1, 0, 1], dtype=np.uint64)
    off = [0, 2, 4]
    rc, vals = g.CombinePull(ids, off)
    assert rc == 0
    assert np.array_equal(vals[:2], np.full((2, 100), np.float32(v0)))
    assert np.array_equal(vals[2:], np.full((2, 100), np.float32(v1)))
    ids2 = np.array([2, 3, 2, 3], dtype=np.uint64)
    rc, before = g.CombinePull(ids2, off)
    rng = np.random.default_rng(0)
    grads = rng.standard_normal((4, 100)).astype(np.float32)
    lr = 0.625
    assert g.CombinePush(api.Optim.create(api.OptimType.kSGD), ids2, off, grads, lr) == 0
    rc, after = g.CombinePull(ids2, off)
    assert np.array_equal(after, before - np.float32(lr) * grads)
    # single-table calls on a member see the group's writes (same stream, same rows)
    assert np.array_equal(t1.Pull([2, 3])[1], after[2:])
    assert len(t0) == 4 and len(t1) == 4
    g.close()
    assert np.array_equal(t0.Pull([2, 3])[1], after[:2])      # tables outlive their group


@pytest.mark.parametrize("name,type_,conf", [c for c in OPTIM_CASES if c[0] in (
    "sgd_mom", "adagrad", "adam", "rmsprop_all")], ids=lambda v: v if isinstance(v, str) else None)
@pytest.mark.parametrize("dim,n_tables", [(16, 26), (30, 3), (64, 7), (128, 5)])
def test_group_matches_oracle_loop(api, oracle, name, type_, conf, dim, n_tables):
    """The Wide&Deep shape: n tables, one Zipf batch each, pull then push, several steps, with
    new ids arriving at every step (insert-on-pull inside the combined launch)."""
    rng = np.random.default_rng(dim + n_tables)
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "11"})
    tables = [api.SparseTable(dim, gi, capacity_hint=64) for _ in range(n_tables)]
    refs = [oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=11))
            for _ in range(n_tables)]
    grp = api.TableGroup(tables)
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    lr = 0.05
    for step in range(4):
        per = [np.unique(zipf_ids(rng, 1.05, 100000, int(rng.integers(1, 3000)))) for _ in range(n_tables)]
        if step == 2:
            per[1] = np.zeros(0, np.uint64)                   # a table with nothing in this request
        off = grp._offsets([p.size for p in per])
        ids = np.concatenate(per)
        grads = (rng.standard_normal((ids.size, dim)) * 0.1).astype(np.float32)
        rc, got = grp.CombinePull(ids, off)
        assert rc == 0
        want = np.concatenate([r.pull(p)[1] for r, p in zip(refs, per)])
        assert_close(got, want, "%s pull step %d" % (name, step))
        assert grp.CombinePush(o_gpu, ids, off, grads, lr) == 0
        for r, p, a, b in zip(refs, per, off[:-1], off[1:]):
            assert r.push(o_ref, p, grads[a:b], lr) == 0
    for t, r in zip(tables, refs):
        gid, gval, _, gsteps = t.export()
        rid, rval, _, rsteps = r.export()
        og, orr = np.argsort(gid), np.argsort(rid)
        assert np.array_equal(gid[og], rid[orr])
        assert_close(gval[og], rval[orr], name + " final weights")
        if type_ == 1:
            assert np.array_equal(gsteps[og], rsteps[orr])


@pytest.mark.parametrize("dim", [16, 6, 36, 64, 128])
def test_group_pulls_while_the_tables_are_being_filled(api, oracle, dim):
    """A combined pull of 8192 ids or more whose members' tables are being filled (new tables, or
    a pull before it that met many new ids) looks up and copies in one launch, queues the missing
    positions member by member and inserts them in a second one. Members of very different
    sizes, one of them empty, ids that repeat inside a member, the ids 0 and all ones, new ids at
    every step, then the same request twice (the second takes the fused kernel again): every
    pulled row as the oracle's, every table holding each id once."""
    rng = np.random.default_rng(dim)
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "17"})
    counts = [9000, 0, 1, 17, 4000, 300, 2500]
    tables = [api.SparseTable(dim, gi, capacity_hint=64) for _ in counts]
    refs = [oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=17)) for _ in counts]
    grp = api.TableGroup(tables)
    per = None
    for step in range(6):
        if step < 4:
            per = []
            for c in counts:
                ids = splitmix64(rng.integers(0, 6000 * (step + 1), size=c, dtype=np.uint64))
                if c > 100:
                    ids[:2] = np.array([0, 2**64 - 1], np.uint64)
                    ids[2:40] = ids[50]                      # one id many times in a row
                per.append(ids)
        off = grp._offsets([p.size for p in per])
        rc, got = grp.CombinePull(np.concatenate(per), off)
        assert rc == 0
        want = np.concatenate([r.pull(p)[1] for r, p in zip(refs, per) if p.size])
        assert_close(got, want, "dim %d, step %d" % (dim, step), rtol=1e-6)
        for t, r in zip(tables, refs):
            assert len(t) == len(r)
    for t, r in zip(tables, refs):
        gid = t.export()[0]
        assert np.array_equal(np.sort(gid), np.sort(r.export()[0]))
    grp.close()

def test_group_errors_and_async(api, oracle):
    gi = api.Initializer.create(0, {"value": "1"})
    a, b, c = (api.SparseTable(8, gi) for _ in range(3))
    with pytest.raises(api.KrakenHipError):
        api.TableGroup([a, api.SparseTable(16, gi)])          # unequal dimension
    grp = api.TableGroup([a, b, c])
    with pytest.raises(api.KrakenHipError):
        api.TableGroup([a])                                    # already a member
    ids = np.array([1, 2, 3, 1, 2, 3, 9], dtype=np.uint64)
    off = [0, 3, 6, 7]
    assert grp.CombinePull(ids, off)[0] == 0
    o = api.Optim.create(api.OptimType.kSGD)
    g = np.ones((7, 8), np.float32)
    bad = ids.copy()
    bad[4] = 77                                                # table b has never seen 77
    assert grp.CombinePush(o, bad, off, g, 0.5) == 12
    assert np.array_equal(a.Pull([1, 2, 3])[1], np.full((3, 8), np.float32(0.5)))   # other rows applied
    assert np.array_equal(b.Pull([1, 3])[1], np.full((2, 8), np.float32(0.5)))
    assert b.lookup([77])[0] == -1
    assert grp.CombinePush(o, ids, off, np.ones((7, 4), np.float32), 0.5) == 11
    assert grp.CombinePull(np.zeros(0, np.uint64), [0, 0, 0, 0])[0] == 0
    # device pointers, enqueue only
    d_ids = api.DeviceArray.from_host(ids)
    d_g = api.DeviceArray.from_host(g)
    rc, d_out = grp.CombinePull(d_ids, off, async_=True)
    assert rc == 0 and grp.CombinePush(o, d_ids, off, d_g, 0.25, async_=True) == 0
    assert grp.sync() == 0
    assert np.array_equal(d_out.to_host()[:3], np.full((3, 8), np.float32(0.5)))
    assert np.array_equal(c.Pull([9])[1], np.full((1, 8), np.float32(0.25)))
    grp.close()


def _dyadic(rng, shape):
    """Gradients whose sums are exact in fp32 in any order."""
    return (rng.integers(-64, 65, size=shape) / 256.0).astype(np.float32)


@pytest.mark.parametrize("name,type_,conf", [c for c in OPTIM_CASES if c[0] in (
    "sgd", "sgd_mom", "adagrad", "adam", "rmsprop_all")], ids=lambda v: v if isinstance(v, str) else None)
@pytest.mark.parametrize("dim,n_tables,per_table", [(16, 26, 8192), (30, 3, 500), (128, 5, 70_000)])
def test_group_push_raw_matches_dedup_sum_per_table(api, oracle, name, type_, conf, dim, n_tables, per_table):
    """Emitter::CombinePushSparseTable (worker/emitter.cc:552-606): repeated ids of every table
    are summed per (table, id) and each distinct row is updated once. The same id appears in
    several tables with different gradients; the members have different row capacities and,
    for one of them, a state column created by an earlier optimizer."""
    rng = np.random.default_rng(dim * n_tables)
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "21"})
    tables = [api.SparseTable(dim, gi, capacity_hint=64 << (i % 4)) for i in range(n_tables)]
    refs = [oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=21))
            for _ in range(n_tables)]
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    # member 1 already has RMSprop's columns: its record layout differs from the others'
    pre_ref, pre_gpu = make_optims(oracle, api, 2, {})
    first = np.arange(10, dtype=np.uint64)
    tables[1].Pull(first)
    refs[1].pull(first)
    g0 = _dyadic(rng, (10, dim))
    assert tables[1].Push(pre_gpu, first, g0, 0.125) == 0
    assert refs[1].push(pre_ref, first, g0, 0.125) == 0
    grp = api.TableGroup(tables)
    lr = 0.05
    for step in range(3):
        per = [zipf_ids(rng, 1.05, 100000, per_table if i != 2 or step != 1 else 0) for i in range(n_tables)]
        off = grp._offsets([p.size for p in per])
        ids = np.concatenate(per)
        grads = _dyadic(rng, (ids.size, dim))
        assert grp.CombinePull(ids, off)[0] == 0
        for r, p in zip(refs, per):
            r.pull(p)
        assert grp.CombinePushRaw(o_gpu, ids, off, grads, lr) == 0
        for r, p, a, b in zip(refs, per, off[:-1], off[1:]):
            u, gs = oracle.dedup_sum(p, grads[a:b])
            assert r.push(o_ref, u, gs, lr) == 0
    for i, (t, r) in enumerate(zip(tables, refs)):
        gid, gval, _, gsteps = t.export()
        rid, rval, _, rsteps = r.export()
        og, orr = np.argsort(gid), np.argsort(rid)
        assert np.array_equal(gid[og], rid[orr])
        assert_close(gval[og], rval[orr], "%s table %d" % (name, i), rtol=1e-5, atol=1e-7)
        if type_ == 1:
            assert np.array_equal(gsteps[og], rsteps[orr])    # one optimizer step per distinct id
    grp.close()


def test_group_push_raw_agrees_with_per_table_push_raw(api):
    """Random gradients, Adam, identical row numbering on both sides: the combined pipeline and
    krk_sparse_push_raw per table differ only in where tile borders fall in the sorted sequence,
    i.e. in how the fp32 additions of one row's gradients are grouped."""
    dim, n_tables, n = 32, 4, 30_000
    rng = np.random.default_rng(5)
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "4"})
    per = [zipf_ids(rng, 1.2, 50000, n) for _ in range(n_tables)]
    grads = [(rng.standard_normal((n, dim)) * 1e-2).astype(np.float32) for _ in range(n_tables)]
    o = api.Optim.create(api.OptimType.kAdam)
    solo = [api.SparseTable(dim, gi) for _ in range(n_tables)]
    grouped = [api.SparseTable(dim, gi) for _ in range(n_tables)]
    uniq = [np.unique(p) for p in per]
    for tabs in (solo, grouped):
        for t, u in zip(tabs, uniq):
            for k in range(u.size):
                t.Pull(u[k:k + 1])                             # one id per call: rows numbered in this order
    for a, b, u in zip(solo, grouped, uniq):
        assert np.array_equal(a.lookup(u), b.lookup(u))
    grp = api.TableGroup(grouped)
    off = grp._offsets([n] * n_tables)
    for step in range(2):
        for t, p, g in zip(solo, per, grads):
            assert t.PushRaw(o, p, g, 0.01) == 0
        assert grp.CombinePushRaw(o, np.concatenate(per), off, np.concatenate(grads), 0.01) == 0
    for i, (a, b, u) in enumerate(zip(solo, grouped, uniq)):
        assert_close(b.Pull(u)[1], a.Pull(u)[1], "table %d" % i, rtol=1e-5, atol=1e-7)
    grp.close()


def test_group_push_raw_errors(api):
    gi = api.Initializer.create(0, {"value": "1"})
    a, b = api.SparseTable(8, gi), api.SparseTable(8, gi)
    grp = api.TableGroup([a, b])
    ids = np.array([1, 2, 1, 1, 5, 5], dtype=np.uint64)
    off = [0, 4, 6]
    assert grp.CombinePull(ids, off)[0] == 0
    o = api.Optim.create(api.OptimType.kSGD)
    g = np.ones((6, 8), np.float32)
    assert grp.CombinePushRaw(o, ids, off, g, 0.5) == 0
    assert np.array_equal(a.Pull([1, 2])[1][:, 0], np.float32([1 - 1.5, 1 - 0.5]))
    assert np.array_equal(b.Pull([5])[1][:, 0], np.float32([0.0]))
    bad = ids.copy()
    bad[5] = 77                                                # b has never seen 77; 5 still gets its share
    assert grp.CombinePushRaw(o, bad, off, g, 0.5) == 12
    assert np.array_equal(b.Pull([5])[1][:, 0], np.float32([-0.5]))
    assert b.lookup([77])[0] == -1
    assert grp.CombinePushRaw(o, ids, off, np.ones((6, 4), np.float32), 0.5) == 11
    assert grp.CombinePushRaw(o, np.zeros(0, np.uint64), [0, 0, 0], np.zeros((0, 8), np.float32), 0.5) == 0
    assert grp.CombinePushRaw(api.Optim.create(api.OptimType.kSGD), ids, [0, 5, 4], g, 0.5) != 0
    grp.close()


@pytest.mark.parametrize("filler", [5, 9000])
def test_group_push_raw_adds_repeats_in_position_order(api, filler):
    """worker/emitter.cc:563-606 adds the gradients of a repeated (table, id) in the order the
    request lists them. 1e8 + 1 - 1e8 is 0 in that order and 1 in the other two, so the sort
    has to be stable: members of few ids take the one-workgroup-a-member sort, a member above
    8192 ids the radix sort over the whole request."""
    dim = 4
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "0.5"})
    a, b = api.SparseTable(dim, gi), api.SparseTable(dim, gi)
    first = np.array([7], np.uint64)
    a.Pull(first)                                   # row 0 of member 0: its key sorts first
    b.Pull(first)
    rest = np.arange(100, 100 + filler, dtype=np.uint64)
    a.Pull(rest)
    b.Pull(rest)
    grp = api.TableGroup([a, b])
    ids = np.concatenate([[7], rest[: filler // 2], [7], rest[filler // 2:], [7], [7, 7, 7]]).astype(np.uint64)
    off = grp._offsets([ids.size - 3, 3])
    g = np.zeros((ids.size, dim), np.float32)
    at = [0, 1 + filler // 2, ids.size - 4]         # the three positions of id 7 in member 0
    g[at[0]], g[at[1]], g[at[2]] = 1e8, 1.0, -1e8
    g[-3], g[-2], g[-1] = -1e8, 1e8, 1.0            # member 1: (-1e8 + 1e8) + 1 = 1
    sgd = api.Optim.create(api.OptimType.kSGD)
    assert grp.CombinePushRaw(sgd, ids, off, g, 1.0) == 0
    assert np.array_equal(a.Pull(first)[1], np.full((1, dim), 0.5, np.float32))     # 0.5 - 0
    assert np.array_equal(b.Pull(first)[1], np.full((1, dim), -0.5, np.float32))    # 0.5 - 1
    grp.close()
