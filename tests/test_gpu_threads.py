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
