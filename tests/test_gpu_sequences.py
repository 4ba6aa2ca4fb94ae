"""Random sequences of table operations against the oracle table: pulls with new and old ids,
pushes of unique ids, pushes with repeats, pooled pulls and pushes, erases, imports, a trip
through a checkpoint file and a change of optimizer mid-way (new state columns on a populated
table). After every operation that returns rows they are compared; at the end every row, state
and counter. What the single-purpose tests cover one by one is covered here in combination."""
import numpy as np
import pytest

from util import assert_close, make_optims, splitmix64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def _dyadic(rng, shape):
    return (rng.integers(-32, 33, size=shape) / 1024.0).astype(np.float32)


# The optimizers a sequence switches between. SGD with momentum tells a row's first update by a
# flag that RMSprop with momentum does not set (the reference looks for the buffer in the row's
# state map, and a model has one optimizer, so the two never meet on a table): a sequence draws
# from a family that holds one of them.
FAMILIES = [[(3, {}), (0, {}), (1, {}), (2, {"momentum": 0.5})],
            [(3, {}), (0, {}), (1, {}), (3, {"momentum": 0.9, "dampening": 0.25}), (2, {})]]


@pytest.mark.parametrize("seed", range(120))
def test_random_operation_sequences(api, oracle, tmp_path, seed):
    _table_sequence(api, oracle, tmp_path, seed, [4, 5, 16, 32, 64, 72, 128])


@pytest.mark.parametrize("seed", range(12))
def test_random_operation_sequences_on_wide_rows(api, oracle, tmp_path, seed):
    """Rows wider than one pass of a wavefront (more than 256 floats): every kernel walks them in
    chunks, and a row's step counter must advance once, after its last chunk."""
    _table_sequence(api, oracle, tmp_path, 500 + seed, [260, 1000, 1030])


def _table_sequence(api, oracle, tmp_path, seed, dims):
    rng = np.random.default_rng(1000 + seed)
    dim = int(rng.choice(dims))
    space = int(rng.choice([300, 5000, 200000]))
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.05", "seed": str(seed)})
    oi = oracle.init(oracle.INIT_NORMAL, 0.0, 0.05, seed=seed)
    t = api.SparseTable(dim, gi, capacity_hint=int(rng.choice([0, 64, 4096])))
    r = oracle.SparseTable(dim, oi)
    used = set()
    OPTIMS = FAMILIES[seed % 2]
    type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    lr = 0.03125

    def some_ids(n, known_only=False):
        if known_only:
            pool = np.fromiter(used, np.uint64, len(used))
            return rng.choice(pool, size=min(n, pool.size), replace=True) if pool.size else pool
        ids = splitmix64(rng.integers(0, space, size=n).astype(np.uint64))
        if n and rng.random() < 0.25:
            ids[rng.integers(n)] = np.uint64(2**64 - 1)        # the id that equals the index's empty marker
        if n and rng.random() < 0.25:
            ids[rng.integers(n)] = np.uint64(0)
        return ids

    log = []
    for step in range(60):
        op = rng.choice(["pull", "pull", "push", "push_raw", "pooled", "erase", "load", "file", "optim", "fetch",
                         "route"])
        log.append(op)
        n = int(rng.choice([1, 7, 300, 3000]))
        if op == "pull":
            ids = some_ids(n)
            rc, got = t.Pull(ids)
            assert rc == 0
            assert_close(got, r.pull(ids)[1], "step %d pull" % step, rtol=1e-5, atol=1e-7)
            used.update(ids.tolist())
        elif op == "push" and used:
            ids = np.unique(some_ids(n, known_only=True))
            g = _dyadic(rng, (ids.size, dim))
            assert t.Push(o_gpu, ids, g, lr) == 0 and r.push(o_ref, ids, g, lr) == 0
        elif op == "push_raw" and used:
            ids = some_ids(n, known_only=True)
            g = _dyadic(rng, (ids.size, dim))
            assert t.PushRaw(o_gpu, ids, g, lr) == 0
            u, gs = oracle.dedup_sum(ids, g)
            assert r.push(o_ref, u, gs, lr) == 0
        elif op == "pooled" and dim <= 256:
            bags = int(rng.choice([1, 5, 200]))
            # bag sizes whose mean ratio is a power of two: every gradient sum stays exact, so the
            # optimizers (Adam above all, whose step is g / |g| on a fresh row) see identical inputs
            lengths = rng.choice([0, 1, 2, 4], size=bags)
            off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
            ids = some_ids(int(off[-1]))
            mode = str(rng.choice(["sum", "mean"]))
            w = (2.0 ** rng.integers(-2, 2, size=ids.size)).astype(np.float32) if rng.random() < 0.5 else None
            rc, got = t.PullPooled(ids, off, mode, 0.5, weights=w)
            assert rc == 0
            u, inv = oracle.dedup(ids)
            rows = r.pull(u)[1][inv] if ids.size else np.zeros((0, dim), np.float32)
            if w is not None:
                rows = rows * w[:, None]                       # pytorch/jagged_embedding.py:44-45
            assert_close(got, oracle.jagged_forward(rows, off, mode, 0.5), "step %d pooled pull" % step,
                         rtol=1e-5, atol=1e-6)
            used.update(ids.tolist())
            bg = _dyadic(rng, (bags, dim))
            assert t.PushPooled(o_gpu, ids, off, bg, lr, mode=mode, weights=w) == 0
            if ids.size:
                vg = oracle.jagged_backward(off, bg, mode)
                if w is not None:
                    vg = vg * w[:, None]
                u2, gs = oracle.dedup_sum(ids, vg)
                assert r.push(o_ref, u2, gs, lr) == 0
        elif op == "erase" and used:
            gone = np.unique(np.concatenate([some_ids(n, known_only=True)[: max(1, n // 3)], some_ids(3)]))
            assert t.erase(gone) == r.erase(gone)
            used.difference_update(gone.tolist())
        elif op == "route" and used:
            # a cluster change (ps/ps.cc:92-109): a ring of a few nodes, this server keeps its share
            nodes = int(rng.integers(1, 5))
            ring = sorted((int(h), int(k) % nodes) for k, h in enumerate(
                rng.integers(0, 2**63, size=3 * nodes, dtype=np.int64).astype(np.uint64) * np.uint64(2)))
            table_id, me = int(rng.integers(0, 1000)), int(rng.integers(0, nodes))
            live = r.export()[0]
            owners = oracle.route_owners(ring, table_id, live)
            mine = t.select_routed(table_id, ring, me)
            assert np.array_equal(np.sort(mine), np.sort(live[owners == me]))
            gone = t.select_routed(table_id, ring, me, owned=False)
            assert np.array_equal(np.sort(gone), np.sort(live[owners != me]))
            if rng.random() < 0.5:
                assert t.erase(gone) == r.erase(gone) == gone.size
                used.difference_update(gone.tolist())
        elif op == "load":
            ids = np.unique(some_ids(min(n, 300)))
            vals = _dyadic(rng, (ids.size, dim))
            t.load(ids, vals)
            r.load(ids, vals)
            used.update(ids.tolist())
        elif op == "file" and used:
            path = str(tmp_path / ("t%d.sparse" % step))
            assert t.save(path, 1, "t") == 0
            t2 = api.SparseTable(dim, gi)
            rc, taken = t2.load_file(path, 1, "t")
            assert rc == 0 and taken == len(r)
            t = t2
        elif op == "optim":
            type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
            o_ref, o_gpu = make_optims(oracle, api, type_, conf)
        elif op == "fetch" and used:
            ids = np.concatenate([some_ids(n, known_only=True), some_ids(5)])
            found, vals, _, _ = t.fetch(ids)
            rf, rv = r.fetch(ids)
            assert np.array_equal(found, rf)
            assert_close(vals[found], rv[rf], "step %d fetch" % step, rtol=1e-5, atol=1e-7)
        assert len(t) == len(r), (step, log)

    gid, gval, _, gsteps = t.export()
    rid, rval, _, rsteps = r.export()
    og, orr = np.argsort(gid), np.argsort(rid)
    assert np.array_equal(gid[og], rid[orr]), log
    assert_close(gval[og], rval[orr], "final weights after %s" % log, rtol=2e-5, atol=1e-6)
    assert np.array_equal(gsteps[og], rsteps[orr]), log        # Adam's per-row counts
    for st in range(1, 8):
        gs = t.export(state_type=st)[2]
        rs = r.export(state_type=st)[2]
        assert_close(gs[og], rs[orr], "final state %d" % st, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("seed", range(40))
def test_random_sequences_on_a_group(api, oracle, seed):
    """Combined pulls and pushes (unique ids and with repeats) interleaved with the members' own
    calls, erases and imports, which move rows and add columns under the group's feet."""
    rng = np.random.default_rng(7000 + seed)
    dim = int(rng.choice([4, 6, 16, 32]))
    n_tables = int(rng.choice([1, 2, 5, 26]))
    space = int(rng.choice([200, 20000]))
    tables, refs = [], []
    for m in range(n_tables):
        tables.append(api.SparseTable(dim, api.Initializer.create(
            api.InitializerType.kNormal, {"stddev": "0.05", "seed": str(seed * 100 + m)}),
            capacity_hint=int(rng.choice([0, 2048]))))
        refs.append(oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.05, seed=seed * 100 + m)))
    grp = api.TableGroup(tables)
    used = [set() for _ in range(n_tables)]
    OPTIMS = FAMILIES[seed % 2]
    type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    lr = 0.03125

    def ids_for(m, n, known_only):
        if known_only:
            pool = np.fromiter(used[m], np.uint64, len(used[m]))
            return rng.choice(pool, size=min(n, pool.size), replace=True) if pool.size else pool
        return splitmix64(rng.integers(0, space, size=n).astype(np.uint64))

    log = []
    for step in range(40):
        op = str(rng.choice(["cpull", "cpull", "cpush", "cpush_raw", "pull", "push_raw", "erase", "load", "optim"]))
        log.append(op)
        sizes = [int(rng.choice([0, 1, 40, 900])) for _ in range(n_tables)]
        if op == "cpull":
            per = [ids_for(m, sizes[m], False) for m in range(n_tables)]
            off = grp._offsets([p.size for p in per])
            rc, got = grp.CombinePull(np.concatenate(per), off)
            assert rc == 0
            want = np.concatenate([r.pull(p)[1] for r, p in zip(refs, per)])
            assert_close(got, want, "step %d combined pull" % step, rtol=1e-5, atol=1e-7)
            for m in range(n_tables):
                used[m].update(per[m].tolist())
        elif op in ("cpush", "cpush_raw"):
            per = [ids_for(m, sizes[m], True) for m in range(n_tables)]
            if op == "cpush":
                per = [np.unique(p) for p in per]
            off = grp._offsets([p.size for p in per])
            g = _dyadic(rng, (int(off[-1]), dim))
            ids = np.concatenate(per) if off[-1] else np.zeros(0, np.uint64)
            assert grp.CombinePush(o_gpu, ids, off, g, lr, raw=(op == "cpush_raw")) == 0
            for r, p, a, b in zip(refs, per, off[:-1], off[1:]):
                if p.size:
                    u, gs = oracle.dedup_sum(p, g[a:b])
                    assert r.push(o_ref, u, gs, lr) == 0
        else:
            m = int(rng.integers(n_tables))
            t, r = tables[m], refs[m]
            if op == "pull":
                ids = ids_for(m, sizes[m] + 1, False)
                assert_close(t.Pull(ids)[1], r.pull(ids)[1], "step %d member pull" % step, rtol=1e-5, atol=1e-7)
                used[m].update(ids.tolist())
            elif op == "push_raw" and used[m]:
                ids = ids_for(m, sizes[m] + 1, True)
                g = _dyadic(rng, (ids.size, dim))
                assert t.PushRaw(o_gpu, ids, g, lr) == 0
                u, gs = oracle.dedup_sum(ids, g)
                assert r.push(o_ref, u, gs, lr) == 0
            elif op == "erase" and used[m]:
                gone = np.unique(ids_for(m, sizes[m] // 3 + 1, True))
                assert t.erase(gone) == r.erase(gone)
                used[m].difference_update(gone.tolist())
            elif op == "load":
                ids = np.unique(ids_for(m, 50, False))
                vals = _dyadic(rng, (ids.size, dim))
                t.load(ids, vals)
                r.load(ids, vals)
                used[m].update(ids.tolist())
            elif op == "optim":
                type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
                o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    for m, (t, r) in enumerate(zip(tables, refs)):
        gid, gval, _, gsteps = t.export()
        rid, rval, _, rsteps = r.export()
        og, orr = np.argsort(gid), np.argsort(rid)
        assert np.array_equal(gid[og], rid[orr]), (m, log)
        assert_close(gval[og], rval[orr], "table %d after %s" % (m, log), rtol=2e-5, atol=1e-6)
        assert np.array_equal(gsteps[og], rsteps[orr]), (m, log)
        for st in range(1, 8):
            assert_close(t.export(state_type=st)[2][og], r.export(state_type=st)[2][orr],
                         "table %d state %d" % (m, st), rtol=2e-5, atol=1e-6)
    grp.close()


@pytest.mark.parametrize("seed", range(30))
def test_random_sequences_on_a_dense_table(api, oracle, tmp_path, seed):
    """Dense and COO gradients, optimizer changes and trips through a *.dense file, against the
    oracle's dense table."""
    rng = np.random.default_rng(9000 + seed)
    n = int(rng.choice([1, 7, 256, 1000, 40000]))
    w0 = (rng.standard_normal(n) * 0.1).astype(np.float32)
    t, r = api.DenseTable(w0), oracle.DenseTable(w0)
    OPTIMS = FAMILIES[seed % 2]
    type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    for step in range(25):
        op = str(rng.choice(["push", "push", "coo", "empty_coo", "file", "optim", "pull"]))
        if op == "push":
            g = _dyadic(rng, n)
            assert t.Push(o_gpu, g, 0.0625) == 0 and r.push(o_ref, g, 0.0625) == 0
        elif op == "coo":
            k = int(rng.integers(1, max(2, n // 3 + 1)))
            idx = np.sort(rng.choice(n, size=min(k, n), replace=False)).astype(np.int64)
            val = _dyadic(rng, idx.size)
            assert t.PushCoo(o_gpu, idx, val, 0.0625) == 0 and r.push_coo(o_ref, idx, val, 0.0625) == 0
        elif op == "empty_coo":
            # ps/optim/adam.cc:26-29 : success without touching state or the step counter
            e_i, e_v = np.zeros(0, np.int64), np.zeros(0, np.float32)
            assert t.PushCoo(o_gpu, e_i, e_v, 0.0625) == 0 and r.push_coo(o_ref, e_i, e_v, 0.0625) == 0
        elif op == "file":
            path = str(tmp_path / ("d%d.dense" % step))
            assert t.save(path, 5, "d") == 0
            rc, t, tid, name, shape = api.DenseTable.from_file(path)
            assert rc == 0 and tid == 5 and name == "d"
        elif op == "optim":
            type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
            o_ref, o_gpu = make_optims(oracle, api, type_, conf)
        assert_close(t.Pull()[1], r.pull(), "step %d %s" % (step, op), rtol=2e-5, atol=1e-6)
        assert t.steps == r.steps
    for st in range(1, 8):
        want = r.state(st)
        got = t.state(st)
        if want is None:
            assert got is None or not np.any(got)
        else:
            assert_close(got, want, "state %d" % st, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("seed", range(30))
def test_random_sequences_enqueued_without_waiting(api, oracle, seed):
    """The same operations through device pointers with KRK_ASYNC: nothing waits until the end,
    tables start tiny so that they grow (records, index, new state columns) while earlier
    launches are still queued, and every reply is checked after the final sync."""
    rng = np.random.default_rng(12000 + seed)
    dim = int(rng.choice([4, 16, 32]))
    space = int(rng.choice([500, 100000]))
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.05", "seed": str(seed)})
    t = api.SparseTable(dim, gi, capacity_hint=int(rng.choice([0, 16])))
    r = oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.05, seed=seed))
    OPTIMS = FAMILIES[seed % 2]
    type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    used = np.zeros(0, np.uint64)
    pending = []          # (device output, expected rows, what)
    keep = []             # device inputs stay alive until the sync
    for step in range(30):
        op = str(rng.choice(["pull", "pull", "push", "push_raw", "pooled", "optim"]))
        n = int(rng.choice([1, 50, 2000, 20000]))
        if op == "pull":
            ids = splitmix64(rng.integers(0, space, size=n).astype(np.uint64))
            d_ids = api.DeviceArray.from_host(ids)
            rc, d_out = t.Pull(d_ids, async_=True)
            assert rc == 0
            pending.append((d_out, r.pull(ids)[1], "step %d pull" % step))
            keep.append(d_ids)
            used = np.union1d(used, ids)
        elif op in ("push", "push_raw") and used.size:
            ids = rng.choice(used, size=min(n, used.size), replace=(op == "push_raw"))
            g = _dyadic(rng, (ids.size, dim))
            d_ids, d_g = api.DeviceArray.from_host(ids), api.DeviceArray.from_host(g)
            assert t.Push(o_gpu, d_ids, d_g, 0.03125, async_=True, raw=(op == "push_raw")) == 0
            u, gs = oracle.dedup_sum(ids, g)
            assert r.push(o_ref, u, gs, 0.03125) == 0
            keep += [d_ids, d_g]
        elif op == "pooled":
            bags = int(rng.choice([1, 30, 3000]))
            lengths = rng.choice([0, 1, 2, 4], size=bags)
            off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
            ids = splitmix64(rng.integers(0, space, size=int(off[-1])).astype(np.uint64))
            d_ids, d_off = api.DeviceArray.from_host(ids), api.DeviceArray.from_host(off)
            rc, d_out = t.PullPooled(d_ids, d_off, "mean", 0.25, async_=True)
            assert rc == 0
            u, inv = oracle.dedup(ids)
            rows = r.pull(u)[1][inv] if ids.size else np.zeros((0, dim), np.float32)
            pending.append((d_out, oracle.jagged_forward(rows, off, "mean", 0.25), "step %d pooled" % step))
            used = np.union1d(used, ids)
            bg = _dyadic(rng, (bags, dim))
            d_bg = api.DeviceArray.from_host(bg)
            assert t.PushPooled(o_gpu, d_ids, d_off, d_bg, 0.03125, mode="mean", async_=True) == 0
            if ids.size:
                u2, gs = oracle.dedup_sum(ids, oracle.jagged_backward(off, bg, "mean"))
                assert r.push(o_ref, u2, gs, 0.03125) == 0
            keep += [d_ids, d_off, d_bg]
        elif op == "optim":
            type_, conf = OPTIMS[int(rng.integers(len(OPTIMS)))]
            o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    assert t.sync() == 0
    for d_out, want, what in pending:
        assert_close(d_out.to_host(), want, what, rtol=1e-5, atol=1e-6)
    gid, gval, _, gsteps = t.export()
    rid, rval, _, rsteps = r.export()
    og, orr = np.argsort(gid), np.argsort(rid)
    assert np.array_equal(gid[og], rid[orr])
    assert_close(gval[og], rval[orr], "final weights", rtol=2e-5, atol=1e-6)
    assert np.array_equal(gsteps[og], rsteps[orr])


@pytest.mark.parametrize("seed", range(20))
def test_random_sequences_of_the_threshold_codec(api, oracle, seed):
    """Many steps of one DenseBag with awkward gradients (all zeros, all equal, a few huge values,
    subnormals, signed zeros) and a life span that makes thresholds go stale: indices, values,
    threshold, residual and step count equal the oracle's at every step."""
    rng = np.random.default_rng(15000 + seed)
    n = int(rng.choice([256, 257, 1000, 4096, 70001]))
    life_span = int(rng.choice([1, 2, 3, 1000]))
    eta = float(rng.choice([0.1, 0.5, 0.75, 0.99]))
    bag, ref = api.DenseBag(n), oracle.DctState(n)
    for step in range(10):
        kind = str(rng.choice(["normal", "normal", "zeros", "equal", "spikes", "tiny", "negzero"]))
        if kind == "normal":
            g = rng.standard_normal(n).astype(np.float32)
        elif kind == "zeros":
            g = np.zeros(n, np.float32)
        elif kind == "equal":
            g = np.full(n, np.float32(rng.choice([-1.5, 0.25])))
        elif kind == "spikes":
            g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
            g[rng.choice(n, size=5, replace=False)] = np.float32(1e30)
        elif kind == "tiny":
            g = (rng.standard_normal(n) * 1e-42).astype(np.float32)       # subnormal
        else:
            g = np.where(rng.random(n) < 0.5, np.float32(-0.0), np.float32(0.0)).astype(np.float32)
        idx, val = bag.MaybeToCoo(life_span, eta, g)
        ridx, rval = ref.compress(g, life_span=life_span, eta=eta, exact_select=True)
        assert bag.tau == ref.tau, (step, kind)
        assert np.array_equal(idx, ridx), (step, kind)
        assert np.array_equal(val.view(np.uint32), rval.view(np.uint32)), (step, kind)
        assert np.array_equal(bag.residual.view(np.uint32), ref.residual.view(np.uint32)), (step, kind)
        assert bag.step == ref.step
        assert np.array_equal(api.coo_to_dense(idx, val, n), oracle.coo_to_dense(ridx, rval, n))
