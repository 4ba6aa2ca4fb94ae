"""Several host threads calling one table at once, the way Station worker threads call a
SparseTable (kraken/rpc/station.cc:177-180, default --thread_nums=2). The reference serialises
per slot with a unique lock for Pull and Push alike (ps/sparse_table.cc:48,88) and a dense Push
takes a unique lock (ps/dense_table.cc:40): whatever the interleaving, every update is applied
exactly once. Gradients lie on a binary grid and the optimizer is plain SGD, so the final table
does not depend on the order in which the threads' pushes land and can be compared exactly."""
import threading

import numpy as np
import pytest

from util import splitmix64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def test_concurrent_pull_push_on_one_table(api, oracle):
    dim, n_threads, steps, batch = 16, 4, 25, 4096
    t = api.SparseTable(dim, api.Initializer.create(api.InitializerType.kConstant, {"value": "1"}),
                        capacity_hint=64)          # small: growth happens under contention too
    sgd = api.Optim.create(api.OptimType.kSGD)
    work = []
    for k in range(n_threads):
        rng = np.random.default_rng(100 + k)
        per = []
        for _ in range(steps):
            ids = np.unique(splitmix64(rng.integers(0, 20000, size=batch, dtype=np.uint64)))
            g = rng.integers(-8, 9, size=(ids.size, dim)).astype(np.float32) / np.float32(64.0)
            per.append((ids, g))
        work.append(per)
    errors = []

    def worker(k):
        try:
            for ids, g in work[k]:
                rc, rows = t.Pull(ids)
                assert rc == 0 and rows.shape == (ids.size, dim)
                assert t.Push(sgd, ids, g, 0.5) == 0
        except Exception as e:       # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    # the same requests, one after the other, on the oracle
    r = oracle.SparseTable(dim, oracle.init(oracle.INIT_CONSTANT, 1.0))
    o = oracle.optim(oracle.SGD)
    for per in work:
        for ids, g in per:
            r.pull(ids)
            assert r.push(o, ids, g, 0.5) == 0
    rid, rval, _, _ = r.export()
    gid, gval, _, _ = t.export()
    og, orr = np.argsort(gid), np.argsort(rid)
    assert np.array_equal(gid[og], rid[orr])
    assert np.array_equal(gval[og], rval[orr])


def test_concurrent_dense_pushes(api, oracle):
    n = 10_000
    w0 = np.zeros(n, np.float32)
    t = api.DenseTable(w0)
    sgd = api.Optim.create(api.OptimType.kSGD)
    grads = [(np.random.default_rng(k).integers(-8, 9, size=n) / 64.0).astype(np.float32) for k in range(8)]

    def worker(k):
        for _ in range(20):
            assert t.Push(sgd, grads[k], 0.25) == 0
            t.Pull()

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    want = -0.25 * 20 * np.sum(np.stack(grads).astype(np.float64), axis=0)
    assert np.array_equal(t.Pull()[1].astype(np.float64), want)


def test_group_calls_and_member_calls_from_several_threads(api, oracle):
    """Two threads issue combined requests on a group while two others call its member tables
    directly (pulls that insert, pushes with repeats, a checkpoint-style fetch): the group's lock
    and the members' locks must serialise them without losing an update or deadlocking."""
    dim, n_tables, steps = 8, 5, 20
    init = api.Initializer.create(api.InitializerType.kConstant, {"value": "1"})
    tables = [api.SparseTable(dim, init, capacity_hint=32) for _ in range(n_tables)]
    grp = api.TableGroup(tables)
    sgd = api.Optim.create(api.OptimType.kSGD)

    def requests(seed, combined):
        rng = np.random.default_rng(seed)
        out = []
        for _ in range(steps):
            if combined:
                per = [splitmix64(rng.integers(0, 3000, size=int(rng.integers(0, 400)), dtype=np.uint64))
                       for _ in range(n_tables)]
                g = rng.integers(-8, 9, size=(sum(p.size for p in per), dim)).astype(np.float32) / np.float32(64)
                out.append((per, g))
            else:
                m = int(rng.integers(n_tables))
                ids = splitmix64(rng.integers(0, 3000, size=int(rng.integers(1, 400)), dtype=np.uint64))
                g = rng.integers(-8, 9, size=(ids.size, dim)).astype(np.float32) / np.float32(64)
                out.append((m, ids, g))
        return out

    work = [requests(1, True), requests(2, True), requests(3, False), requests(4, False)]
    errors = []

    def combined_worker(reqs):
        try:
            for per, g in reqs:
                off = grp._offsets([p.size for p in per])
                ids = np.concatenate(per) if off[-1] else np.zeros(0, np.uint64)
                assert grp.CombinePull(ids, off)[0] == 0
                assert grp.CombinePushRaw(sgd, ids, off, g, 0.5) == 0
        except Exception as e:
            errors.append(e)

    def member_worker(reqs):
        try:
            for m, ids, g in reqs:
                assert tables[m].Pull(ids)[0] == 0
                assert tables[m].PushRaw(sgd, ids, g, 0.5) == 0
                found, _, _, _ = tables[m].fetch(ids[:10])
                assert found.all()
        except Exception as e:
            errors.append(e)

    threads = [threading.Thread(target=combined_worker, args=(work[0],)),
               threading.Thread(target=combined_worker, args=(work[1],)),
               threading.Thread(target=member_worker, args=(work[2],)),
               threading.Thread(target=member_worker, args=(work[3],))]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
        assert not th.is_alive(), "a thread is stuck"
    assert not errors, errors
    refs = [oracle.SparseTable(dim, oracle.init(oracle.INIT_CONSTANT, 1.0)) for _ in range(n_tables)]
    o = oracle.optim(oracle.SGD)
    for reqs in work[:2]:
        for per, g in reqs:
            at = 0
            for r, p in zip(refs, per):
                r.pull(p)
                if p.size:
                    u, gs = oracle.dedup_sum(p, g[at:at + p.size])
                    assert r.push(o, u, gs, 0.5) == 0
                at += p.size
    for reqs in work[2:]:
        for m, ids, g in reqs:
            refs[m].pull(ids)
            u, gs = oracle.dedup_sum(ids, g)
            assert refs[m].push(o, u, gs, 0.5) == 0
    for t, r in zip(tables, refs):
        rid, rval, _, _ = r.export()
        gid, gval, _, _ = t.export()
        og, orr = np.argsort(gid), np.argsort(rid)
        assert np.array_equal(gid[og], rid[orr])
        assert np.array_equal(gval[og], rval[orr])
    grp.close()
