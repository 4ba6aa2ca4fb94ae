"""Worker-side dedup and the fused dedup + segment-reduce + update path against the oracle's
restatement of Emitter::PullSparseTableImpl / PushSparseTable (worker/emitter.cc:131-149,
510-531) followed by SparseTable::Push.

Bar: unique ids, their order and the inverse map exact; summed-and-updated values within 1e-5
relative of the reference order of additions (the GPU adds in a fixed tree, the reference in
position order), measured against the magnitude of the addends where sums cancel.
"""
import numpy as np
import pytest

from util import OPTIM_CASES, assert_close, make_optims, splitmix64, zipf_ids

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


@pytest.mark.parametrize("ids", [
    [5], [5, 5, 5, 5], [1, 2, 3, 4], [9, 1, 9, 2, 1, 9, 2**64 - 1, 0, 2**64 - 1],
])
def test_dedup_small(api, oracle, ids):
    ids = np.array(ids, dtype=np.uint64)
    u, inv = api.dedup(ids)
    ru, rinv = oracle.dedup(ids)
    assert np.array_equal(u, ru) and np.array_equal(inv, rinv)


@pytest.mark.parametrize("n", [1, 63, 1024, 8191, 8192, 8193])
@pytest.mark.parametrize("kind", ["distinct", "same", "pairs", "sentinels"])
def test_dedup_single_launch_boundaries(api, oracle, n, kind):
    """Requests of at most 8192 ids are deduplicated by one workgroup; 8193 ids take the path of
    large requests. Both must give the oracle's unique list (first-occurrence order) and inverse,
    for all-distinct ids (the table at its fullest), one id throughout, every id twice, and the
    two ids an index might mistake for markers (0 and all ones)."""
    rng = np.random.default_rng(n)
    if kind == "distinct":
        ids = rng.permutation(n).astype(np.uint64) * np.uint64(0x9E3779B97F4A7C15)
    elif kind == "same":
        ids = np.full(n, 77, np.uint64)
    elif kind == "pairs":
        ids = np.repeat(rng.permutation((n + 1) // 2).astype(np.uint64) + np.uint64(10), 2)[:n]
        rng.shuffle(ids)
    else:
        ids = rng.choice(np.array([0, 2**64 - 1, 5], np.uint64), size=n)
    u, inv = api.dedup(ids)
    ru, rinv = oracle.dedup(ids)
    assert np.array_equal(u, ru) and np.array_equal(inv, rinv)
    du, dinv, cnt = api.dedup(api.DeviceArray.from_host(ids))
    assert cnt == ru.size
    assert np.array_equal(du.to_host()[:cnt], ru) and np.array_equal(dinv.to_host(), rinv)


def test_dedup_empty(api):
    u, inv = api.dedup(np.zeros(0, np.uint64))
    assert u.size == 0 and inv.size == 0


# 31 / 32 and 127 / 128 workgroups of 1024 positions: below, at and between the sizes from which
# the first 8 or 32 workgroups claim their ids in a launch ahead of the others
@pytest.mark.parametrize("n,s,space", [(8192, 1.05, 10**6), (31 * 1024 + 7, 1.2, 10**5), (32 * 1024, 1.2, 10**5),
                                       (127 * 1024 + 1, 1.3, 10**6), (128 * 1024 + 1, 1.3, 10**6),
                                       (200_000, 1.3, 10**6), (1_000_000, 1.1, 10**7)])
def test_dedup_zipf_exact(api, oracle, n, s, space):
    rng = np.random.default_rng(n)
    ids = zipf_ids(rng, s, space, n)
    u, inv = api.dedup(ids)
    ru, rinv = oracle.dedup(ids)
    assert np.array_equal(u, ru)               # first-occurrence order, bit for bit
    assert np.array_equal(inv, rinv)
    assert np.array_equal(u[inv], ids)
    # device-resident variant
    d = api.DeviceArray.from_host(ids)
    du, dinv, cnt = api.dedup(d)
    assert cnt == ru.size
    assert np.array_equal(du.to_host()[:cnt], ru) and np.array_equal(dinv.to_host(), rinv)


def _dyadic_grads(rng, shape):
    """Gradients on a coarse binary grid: any order of fp32 additions gives the same bits, so
    the comparison isolates dedup + update from the (order-dependent) rounding of the sums."""
    return (rng.integers(-64, 65, size=shape).astype(np.float32) / np.float32(4096.0))


@pytest.mark.parametrize("name,type_,conf", [c for c in OPTIM_CASES if c[0] in (
    "sgd", "sgd_damp", "adagrad", "adam", "adam_amsgrad", "rmsprop", "rmsprop_all")],
    ids=lambda v: v if isinstance(v, str) else None)
@pytest.mark.parametrize("dim,n,s", [(16, 8192, 1.05), (128, 50_000, 1.3), (100, 3000, 1.3), (8, 300_000, 1.2)])
def test_push_raw_matches_dedup_sum_then_push(api, oracle, name, type_, conf, dim, n, s):
    rng = np.random.default_rng(n + dim)
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "9"})
    t = api.SparseTable(dim, gi)
    r = oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=9))
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    lr = 0.05
    for step in range(3):
        ids = zipf_ids(rng, s, 10**6, n)
        g = _dyadic_grads(rng, (n, dim))
        assert t.Pull(ids)[0] == 0
        r.pull(ids)
        assert t.PushRaw(o_gpu, ids, g, lr) == 0
        u, gs = oracle.dedup_sum(ids, g)
        assert r.push(o_ref, u, gs, lr) == 0
    gid, gval, _, gsteps = t.export()
    rid, rval, _, rsteps = r.export()
    og, orr = np.argsort(gid), np.argsort(rid)
    assert np.array_equal(gid[og], rid[orr])
    if type_ == 1:
        assert np.array_equal(gsteps[og], rsteps[orr])       # one optimizer step per unique id
    assert_close(gval[og], rval[orr], "%s dim %d" % (name, dim), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dim,n,s", [(16, 8192, 1.05), (128, 100_000, 1.3), (32, 1_000_000, 1.1)])
def test_push_raw_sums_random_gradients(api, oracle, dim, n, s):
    """Random N(0, 1e-2) gradients, as in the benchmark configs. With thousands of duplicates per
    id the fp32 sum depends on the order of additions (position order in the reference, a fixed
    tree here), so both are held to the float64 sum: error <= 1e-5 relative plus 1e-6 of the
    absolute mass that was added."""
    rng = np.random.default_rng(n)
    ids = zipf_ids(rng, s, 10**6, n)
    g = (rng.standard_normal((n, dim)) * 1e-2).astype(np.float32)
    t = api.SparseTable(dim, api.Initializer.create(api.InitializerType.kConstant, {"value": "0"}))
    t.Pull(ids)
    lr = 0.5
    assert t.PushRaw(api.Optim.create(api.OptimType.kSGD), ids, g, lr) == 0
    u, inv = oracle.dedup(ids)
    exact = np.zeros((u.size, dim), np.float64)
    mass = np.zeros((u.size, dim), np.float64)
    np.add.at(exact, inv, g.astype(np.float64))
    np.add.at(mass, inv, np.abs(g.astype(np.float64)))
    want = -lr * exact
    tol = 1e-5 * np.abs(want) + 1e-6 * lr * mass + 1e-9
    got = t.Pull(u)[1].astype(np.float64)
    assert (np.abs(got - want) <= tol).all(), float((np.abs(got - want) / tol).max())
    _, ref_sum = oracle.dedup_sum(ids, g)
    assert (np.abs(-lr * ref_sum.astype(np.float64) - want) <= tol).all()


def test_push_raw_single_hot_id_and_all_distinct(api, oracle):
    """The extremes of the segmented reduction: one run spanning every tile, no runs at all,
    and a hundred long runs."""
    dim = 32
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "1"})
    o_ref, o_gpu = make_optims(oracle, api, 3, {})
    rng = np.random.default_rng(7)
    for ids in (np.full(70_000, 12345, dtype=np.uint64),
                splitmix64(np.arange(70_000, dtype=np.uint64)),
                np.repeat(splitmix64(np.arange(100, dtype=np.uint64)), 700),
                np.tile(splitmix64(np.arange(100, dtype=np.uint64)), 700)):
        t = api.SparseTable(dim, gi)
        r = oracle.SparseTable(dim, oracle.init(oracle.INIT_CONSTANT, 1.0))
        g = _dyadic_grads(rng, (ids.size, dim))
        t.Pull(ids)
        r.pull(ids)
        assert t.PushRaw(o_gpu, ids, g, 0.5) == 0
        u, gs = oracle.dedup_sum(ids, g)
        assert r.push(o_ref, u, gs, 0.5) == 0
        rc, got = t.Pull(u)
        _, want = r.pull(u)
        assert np.array_equal(got, want)                       # exact sums, exact SGD
        # the same request on the same table state gives the same bits again
        g2 = (rng.standard_normal((ids.size, dim)) * 1e-2).astype(np.float32)
        a = api.SparseTable(dim, gi)
        b = api.SparseTable(dim, gi)
        for x in (a, b):
            for k in u[:200]:
                x.Pull([k])                                    # one id per call: same row numbers
            x.Pull(ids)
            assert x.PushRaw(o_gpu, ids, g2, 0.5) == 0
        if u.size <= 200:
            assert np.array_equal(a.Pull(u)[1], b.Pull(u)[1])


def test_push_raw_missing_id_and_width(api, oracle):
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "2"})
    t = api.SparseTable(8, gi)
    t.Pull([1, 2, 3])
    o = api.Optim.create(api.OptimType.kSGD)
    g = np.ones((5, 8), np.float32)
    assert t.PushRaw(o, [1, 1, 2, 77, 77], g, 0.25) == 12
    rc, rows = t.Pull([1, 2, 3])
    assert np.array_equal(rows[:, 0], np.float32([2 - 0.5, 2 - 0.25, 2]))
    assert t.lookup([77])[0] == -1
    assert t.PushRaw(o, [1, 2], np.ones((2, 4), np.float32), 0.1) == 11
    assert t.PushRaw(o, [], np.zeros((0, 8), np.float32), 0.1) == 0


@pytest.mark.parametrize("dim", [1, 6, 16, 128])
@pytest.mark.parametrize("n,s,space", [(1, 1.05, 10), (9, 1.05, 4), (8192, 1.05, 10**6), (300_000, 1.3, 10**6)])
def test_dedup_sum_standalone(api, oracle, dim, n, s, space):
    """Emitter::PushSparseTable's dedup + sum as a call of its own: unique ids, inverse map and
    (on a binary grid, where the order of additions cannot matter) the summed rows all exact."""
    rng = np.random.default_rng(dim * 1000 + n)
    ids = zipf_ids(rng, s, space, n)
    g = (rng.integers(-64, 65, size=(n, dim)) / 4096.0).astype(np.float32)
    u, inv, sums = api.dedup_sum(ids, g)
    ru, rs = oracle.dedup_sum(ids, g)
    _, rinv = oracle.dedup(ids)
    assert np.array_equal(u, ru) and np.array_equal(inv, rinv)
    assert np.array_equal(sums, rs)
    # the pull side's re-expansion (worker/emitter.cc:162-182) undoes the dedup
    rc, back = api.expand_rows(sums, inv)
    assert rc == 0 and np.array_equal(back, rs[rinv])


def test_dedup_sum_random_gradients_and_device_arrays(api, oracle):
    rng = np.random.default_rng(77)
    n, dim = 500_000, 32
    ids = zipf_ids(rng, 1.2, 10**6, n)
    g = rng.standard_normal((n, dim)).astype(np.float32)
    d_u, d_inv, d_sums, count = api.dedup_sum(api.DeviceArray.from_host(ids), api.DeviceArray.from_host(g))
    ru, rinv = oracle.dedup(ids)
    assert count == ru.size
    assert np.array_equal(d_u.to_host()[:count], ru) and np.array_equal(d_inv.to_host(), rinv)
    exact = np.zeros((count, dim), np.float64)
    np.add.at(exact, rinv, g.astype(np.float64))
    mass = np.zeros((count, dim), np.float64)
    np.add.at(mass, rinv, np.abs(g).astype(np.float64))
    got = d_sums.to_host()[:count]
    # fp32 summation in a fixed tree: error bounded by a few ulps of the summed magnitudes
    assert (np.abs(got - exact) <= 4e-7 * mass + 1e-30).all()
    rc, d_back = api.expand_rows(d_sums, d_inv)
    assert rc == 0 and np.array_equal(d_back.to_host(), got[rinv])
    bad = rinv.copy()
    bad[5] = count + 3
    rc, _ = api.expand_rows(got, bad)
    assert rc == api.E_ARGUMENT


@pytest.mark.parametrize("dim", [5, 16, 64])
@pytest.mark.parametrize("shape", ["one_id", "one_bucket", "long_and_short", "boundary"])
def test_push_raw_short_path_extremes(api, oracle, dim, shape):
    """Requests of at most 8192 ids take the two-launch path (one workgroup per bucket of rows, LDS
    sort, runs above 64 positions shared out over the workgroup). Its corners, against the oracle's
    dedup + sum + push: 8192 copies of one id (one run that fills the bucket), 8192 distinct rows that
    all fall into one bucket (the workgroup's arrays at their fullest), long runs next to short ones
    at an odd row width, and the same ids as a request of 8192 and of 8193 (the second takes the
    path of large requests). Dyadic gradients: exact whatever the order of additions. Random
    gradients: the long runs are added as per-lane-group stretches combined in a fixed tree, not
    strictly in position order, so they are held to the float64 sum."""
    rng = np.random.default_rng(dim * 10 + len(shape))
    gi = api.Initializer.create(api.InitializerType.kConstant, {"value": "1"})
    t = api.SparseTable(dim, gi)
    r = oracle.SparseTable(dim, oracle.init(oracle.INIT_CONSTANT, 1.0))
    o_ref, o_gpu = make_optims(oracle, api, 0, {})          # Adagrad: a non-linear update
    if shape == "one_id":
        requests = [np.full(8192, 4242, np.uint64)]
    elif shape == "one_bucket":
        pool = splitmix64(np.arange(300_000, dtype=np.uint64))
        t.Pull(pool)
        r.pull(pool)
        rows = t.lookup(pool)
        same = pool[rows % 32 == 0][:8192]                    # the short path's buckets are row mod 8..32
        assert same.size == 8192
        requests = [same]
    elif shape == "long_and_short":
        hot = splitmix64(np.arange(5, dtype=np.uint64))
        ids = np.concatenate([np.repeat(hot, [3000, 900, 65, 64, 63]), splitmix64(np.arange(100, 4200, dtype=np.uint64))])
        requests = [ids[rng.permutation(ids.size)]]
    else:
        base = zipf_ids(rng, 1.05, 10**5, 8193)
        requests = [base[:8192], base]
    for ids in requests:
        t.Pull(ids)
        r.pull(ids)
        for grads in (_dyadic_grads(rng, (ids.size, dim)),
                      (rng.standard_normal((ids.size, dim)) * 1e-2).astype(np.float32)):
            assert t.PushRaw(o_gpu, ids, grads, 0.05) == 0
            u, gs = oracle.dedup_sum(ids, grads)
            assert r.push(o_ref, u, gs, 0.05) == 0
            got, want = t.Pull(u)[1], r.pull(u)[1]
            if grads is not None and np.array_equal(grads * 4096, np.round(grads * 4096)):
                assert_close(got, want, "%s dim %d, dyadic" % (shape, dim), rtol=1e-6, atol=1e-7)
            else:
                # the two orders of fp32 additions differ by a few ulps of the mass that was added
                assert_close(got, want, "%s dim %d, random" % (shape, dim), rtol=1e-5, atol=1e-6)
    # SGD makes the sum itself visible: against the float64 sum of the long runs
    if shape in ("one_id", "long_and_short"):
        ids = requests[0]
        grads = (rng.standard_normal((ids.size, dim)) * 1e-2).astype(np.float32)
        before = t.Pull(np.unique(ids))[1].astype(np.float64)
        assert t.PushRaw(api.Optim.create(api.OptimType.kSGD), ids, grads, 1.0) == 0
        u, inv = np.unique(ids, return_inverse=True)
        exact = np.zeros((u.size, dim), np.float64)
        mass = np.zeros((u.size, dim), np.float64)
        np.add.at(exact, inv, grads.astype(np.float64))
        np.add.at(mass, inv, np.abs(grads).astype(np.float64))
        after = t.Pull(u)[1].astype(np.float64)
        assert (np.abs((before - after) - exact) <= 4e-7 * mass + 2e-7 * np.abs(before) + 1e-30).all()
