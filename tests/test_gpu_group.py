"""Combined requests over several tables (Ps::CombinePullSparseTable / CombinePushSparseTable,
ps/ps_op.cc:370-387, 456-469) served by one launch, against the oracle looping over tables the
way the reference does. Shape of the reference's own test: emitter_test.cc:75-87, 112-158
(two tables, Constant init, SGD, combined pull and combined push)."""
import numpy as np
import pytest

from util import OPTIM_CASES, assert_close, make_optims, zipf_ids

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
@pytest.mark.parametrize("dim,n_tables", [(16, 26), (30, 3), (128, 5)])
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
