"""Per-kernel timings of the table engine at the sizes of the benchmark configurations.

    python -m kraken_amd.microbench [lines] [copy] [tables] [raw] [combined] [host] [pooled] [codec] [dense] [dense_group]
                                    [dct2] [hooks] [legs]

Every figure is the average of back-to-back launches between two HIP events recorded on the
stream the kernels run on, with inputs resident in HBM; bandwidths are algorithmic bytes
(stated per line) over that time. With no argument all sections run (about a minute). This is
the program the rocprofv3 summaries of the individual kernels are taken from.
"""
import gc
import sys
import time

import numpy as np

from . import api
from .workloads import splitmix64, zipf_ranks


def timed(owner, fn, reps=10, sync=None):
    """Average seconds per call of fn between two events on owner's stream (None: null stream)."""
    sync = sync or (owner.sync if owner is not None else api.synchronize)
    fn()
    sync()
    # a collection of the interpreter's garbage in the middle of ten calls stalls the host for
    # longer than the calls take on the device, and the stream runs dry: collect before, not during
    gc.collect()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        e0, e1 = api.Event(), api.Event()
        e0.record(owner)
        for _ in range(reps):
            fn()
        e1.record(owner)
        sync()
    finally:
        if was_enabled:
            gc.enable()
    return e0.elapsed_ms(e1) / reps * 1e-3


def prefill(t, rows, dim, chunk=1 << 22):
    scratch = api.DeviceArray((min(chunk, rows), dim), np.float32)
    t.reserve(rows + rows // 8)
    for lo in range(0, rows, chunk):
        d = api.DeviceArray.from_host(splitmix64(np.arange(lo, min(lo + chunk, rows), dtype=np.uint64)))
        t.Pull(d, out=scratch, async_=True)
        t.sync()
        d.free()
    scratch.free()


def tables():
    print("# lookup / pull / push of U unique resident ids, table of 4e6 rows")
    print("#   bytes: lookup 20U, pull U(8+8D), push U(8+4D+8D(1+S)) (+16U Adam)")
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "0"})
    rows = 4 * 10**6
    for dim, u, optim_name in ((16, 98_600, "adagrad"), (16, 10**6, "adagrad"), (32, 10**6, "adagrad"),
                               (64, 10**6, "adagrad"), (128, 10**6, "adagrad"), (32, 10**6, "adam")):
        t = api.SparseTable(dim, init, capacity_hint=rows)
        prefill(t, rows, dim)
        rng = np.random.default_rng(0)
        sets = []
        for _ in range(4):
            ids = splitmix64(rng.choice(rows, size=u, replace=False).astype(np.uint64))
            sets.append((api.DeviceArray.from_host(ids),
                         api.DeviceArray.from_host((rng.standard_normal((u, dim)) * 1e-2).astype(np.float32)),
                         api.DeviceArray((u, dim), np.float32), api.DeviceArray(u, np.int32)))
        o = api.Optim.create({"adagrad": 0, "adam": 1}[optim_name])
        S = {"adagrad": 1, "adam": 2}[optim_name]
        k = [0]

        def nxt():
            k[0] += 1
            return sets[k[0] % 4]

        def lookup():
            d_ids, _, _, d_rows = nxt()
            api.lib().krk_sparse_lookup(t.h, api._ptr(d_ids), u, api._ptr(d_rows), api.DEVICE_PTRS | api.ASYNC)

        def pull():
            d_ids, _, d_out, _ = nxt()
            t.Pull(d_ids, out=d_out, async_=True)

        def push():
            d_ids, d_g, _, _ = nxt()
            t.Push(o, d_ids, d_g, 0.01, async_=True)

        tl, tp, tq = timed(t, lookup, 20), timed(t, pull, 20), timed(t, push, 20)
        bl, bp = 20 * u, u * (8 + 8 * dim)
        bq = u * (8 + 4 * dim + 8 * dim * (1 + S) + (16 if optim_name == "adam" else 0))
        print("dim %3d U %8d %-7s | lookup %7.1f us %5.0f GB/s | pull %7.1f us %5.0f GB/s | push %7.1f us %5.0f GB/s"
              % (dim, u, optim_name, tl * 1e6, bl / tl / 1e9, tp * 1e6, bp / tp / 1e9, tq * 1e6, bq / tq / 1e9),
              flush=True)
        for s in sets:
            for a in s:
                a.free()
        t.close()


def inserts():
    """Pulls that insert: every id new (a cold start), and 5 % of a million ids new. A request of
    262 144 ids or more runs as two launches (rows numbered once per workgroup of the second); a
    smaller one inserts inside the fused kernel, one addition to the row counter per wavefront."""
    print("# pulls that insert rows (each call brings ids the table has not seen); the same ids again: resident")
    for dim in (16, 64, 128):
        for n in (98_600, 1 << 20):
            init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "3"})
            t = api.SparseTable(dim, init, capacity_hint=1 << 20)
            t.reserve(6 * n + 1024)
            out = api.DeviceArray((n, dim), np.float32)
            e0, e1 = api.Event(), api.Event()
            cold = []
            for i in range(5):
                d = api.DeviceArray.from_host(splitmix64(np.arange(i * n, (i + 1) * n, dtype=np.uint64) + np.uint64(12345)))
                e0.record(t)
                assert t.Pull(d, out=out, async_=True)[0] == 0
                e1.record(t)
                assert t.sync() == 0
                cold.append(e0.elapsed_ms(e1) * 1e3)
                if i < 4:
                    d.free()
            warm = timed(t, lambda: t.Pull(d, out=out, async_=True), 5)
            print("dim %3d n %8d | every id new %7.1f us (median of calls 2 to 5) | resident %7.1f us"
                  % (dim, n, float(np.median(cold[1:])), warm * 1e6), flush=True)
            d.free()
            out.free()
            t.close()
    dim, n, rows = 128, 1 << 20, 4 * 10**6
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "3"})
    t = api.SparseTable(dim, init, capacity_hint=rows)
    prefill(t, rows, dim)
    t.reserve(rows + n)
    rng = np.random.default_rng(8)
    out = api.DeviceArray((n, dim), np.float32)
    e0, e1 = api.Event(), api.Event()
    some = []
    for i in range(6):
        ids = splitmix64(rng.integers(0, rows, size=n, dtype=np.uint64))
        where = rng.choice(n, size=n // 20, replace=False)
        ids[where] = splitmix64(np.uint64(1 << 40) + np.arange(i * (n // 20), (i + 1) * (n // 20), dtype=np.uint64))
        d = api.DeviceArray.from_host(ids)
        e0.record(t)
        assert t.Pull(d, out=out, async_=True)[0] == 0
        e1.record(t)
        assert t.sync() == 0
        some.append(e0.elapsed_ms(e1) * 1e3)
        d.free()
    print("dim %3d n %8d | 5 %% of the ids new %7.1f us (median of calls 2 to 6)" % (dim, n, float(np.median(some[1:]))),
          flush=True)
    out.free()
    t.close()
    # a combined request over 26 tables keeps the fused kernel: its additions spread over 26 counters
    dim, per = 16, 3792
    tables = [api.SparseTable(dim, init, capacity_hint=1 << 16) for _ in range(26)]
    for t in tables:
        t.reserve(8 * per)
    group = api.TableGroup(tables)
    n = 26 * per
    off = api.TableGroup._offsets([per] * 26)
    out = api.DeviceArray((n, dim), np.float32)
    cold = []
    for i in range(5):
        d = api.DeviceArray.from_host(splitmix64(np.arange(i * n, (i + 1) * n, dtype=np.uint64) + np.uint64(999)))
        e0.record(group)
        assert group.CombinePull(d, off, out=out, async_=True)[0] == 0
        e1.record(group)
        assert group.sync() == 0
        cold.append(e0.elapsed_ms(e1) * 1e3)
        if i < 4:
            d.free()
    warm = timed(group, lambda: group.CombinePull(d, off, out=out, async_=True), 5)
    print("dim %3d n %8d over 26 tables, one combined pull | every id new %7.1f us (median of calls 2 to 5) | "
          "resident %7.1f us" % (dim, n, float(np.median(cold[1:])), warm * 1e6), flush=True)
    d.free()
    out.free()
    group.close()
    for t in tables:
        t.close()


def raw():
    print("# push_raw (dedup + duplicate-gradient sum + update fused) and stand-alone dedup of N ids")
    print("#   bytes: U(8+4D+8D(1+S)) + 8N + 4DN")
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01"})
    for dim, space, n, s, optim in ((16, 10**6, 8192, 1.05, 0), (16, 10**6, 212_992, 1.05, 0),
                                    (128, 2 * 10**7, 1 << 20, 1.3, 2), (32, 10**7, 2_000_000, 1.1, 1)):
        rng = np.random.default_rng(0)
        t = api.SparseTable(dim, init, capacity_hint=min(space, 3 * 10**7))
        ids = splitmix64(zipf_ranks(rng, s, space, n))
        u = np.unique(ids).size
        d_ids = api.DeviceArray.from_host(ids)
        d_g = api.DeviceArray.from_host((rng.standard_normal((n, dim)) * 1e-2).astype(np.float32))
        d_out = api.DeviceArray((n, dim), np.float32)
        t.Pull(d_ids, out=d_out, async_=True)
        assert t.sync() == 0
        o = api.Optim.create(optim, {"alpha": "0.9"} if optim == 2 else {})
        S = {0: 1, 1: 2, 2: 1}[optim]
        dt = timed(t, lambda: t.PushRaw(o, d_ids, d_g, 0.01, async_=True))
        dp = timed(t, lambda: t.Pull(d_ids, out=d_out, async_=True))
        alg = u * (8 + 4 * dim + 8 * dim * (1 + S)) + 8 * n + 4 * dim * n
        uids, inv = api.DeviceArray(n, np.uint64), api.DeviceArray(n, np.int64)
        cnt = api.C.c_int64()

        def dedup():
            api.lib().krk_dedup(api._ptr(d_ids), n, api._ptr(uids), api._ptr(inv), api.C.byref(cnt),
                                api.DEVICE_PTRS)
        dd = timed(None, dedup, 5)
        print("dim %3d N %8d U %7d zipf %.2f | push_raw %7.1f us %5.0f GB/s | pull of the N ids %7.1f us | "
              "dedup (blocking call) %7.1f us" % (dim, n, u, s, dt * 1e6, alg / dt / 1e9, dp * 1e6, dd * 1e6),
              flush=True)
        if n <= 8192:
            def both(noted):
                t.Pull(d_ids, out=d_out, async_=True, note_rows=noted)
                t.PushRaw(o, d_ids, d_g, 0.01, async_=True, as_pulled=noted)
            plain, noted = timed(t, lambda: both(False)), timed(t, lambda: both(True))
            print("                                       | pull + push_raw of the same ids %7.1f us, with the pull's "
                  "row notes %7.1f us" % (plain * 1e6, noted * 1e6), flush=True)
        for a in (d_ids, d_g, d_out, uids, inv):
            a.free()
        t.close()


def combined():
    print("# Wide&Deep step with the worker side on the device: 26 tables of 1e6 rows, 8192 Zipf 1.05 ids")
    print("# per table with repeats, dim 16, Adagrad")
    n_tables, space, batch, dim = 26, 10**6, 8192, 16
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01"})
    rng = np.random.default_rng(0)
    tables = [api.SparseTable(dim, init, capacity_hint=space) for _ in range(n_tables)]
    for t in tables:
        prefill(t, space, dim)
    grp = api.TableGroup(tables)
    per = [splitmix64(zipf_ranks(rng, 1.05, space, batch)) for _ in range(n_tables)]
    off = grp._offsets([batch] * n_tables)
    n = n_tables * batch
    u = sum(np.unique(p).size for p in per)
    d_ids = api.DeviceArray.from_host(np.concatenate(per))
    d_one = [api.DeviceArray.from_host(p) for p in per]
    d_g = api.DeviceArray.from_host((rng.standard_normal((n, dim)) * 1e-2).astype(np.float32))
    d_g1 = api.DeviceArray.from_host((rng.standard_normal((batch, dim)) * 1e-2).astype(np.float32))
    d_out = api.DeviceArray((n, dim), np.float32)
    o = api.Optim.create(api.OptimType.kAdagrad)
    print("ids %d, distinct (table, id) pairs %d" % (n, u), flush=True)

    def per_table():
        for t, d in zip(tables, d_one):
            t.PushRaw(o, d, d_g1, 0.01, async_=True)

    def both(noted):
        grp.CombinePull(d_ids, off, out=d_out, async_=True, note_rows=noted)
        grp.CombinePushRaw(o, d_ids, off, d_g, 0.01, async_=True, as_pulled=noted)

    for name, fn in (
            ("combined pull of all ids", lambda: grp.CombinePull(d_ids, off, out=d_out, async_=True)),
            ("combined push with repeats", lambda: grp.CombinePushRaw(o, d_ids, off, d_g, 0.01, async_=True)),
            ("pull + push of the same ids", lambda: both(False)),
            ("the same with the pull's row notes", lambda: both(True)),
            ("push_raw table by table (26 calls)", per_table)):
        print("%-36s %8.1f us" % (name, timed(grp, fn, 10) * 1e6), flush=True)
    grp.close()
    for t in tables:
        t.close()


def host():
    print("# the same step through host pointers (blocking calls, pageable numpy arrays): what a server")
    print("# that receives its requests in host memory pays, copies over PCIe included")
    import time
    n_tables, space, dim = 26, 10**6, 16
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01"})
    rng = np.random.default_rng(0)
    tables = [api.SparseTable(dim, init, capacity_hint=space) for _ in range(n_tables)]
    for t in tables:
        prefill(t, space, dim)
    grp = api.TableGroup(tables)
    per = [np.unique(splitmix64(zipf_ranks(rng, 1.05, space, 8192))) for _ in range(n_tables)]
    off = grp._offsets([p.size for p in per])
    ids = np.concatenate(per)
    grads = (rng.standard_normal((ids.size, dim)) * 1e-2).astype(np.float32)
    out = np.empty((ids.size, dim), np.float32)
    o = api.Optim.create(api.OptimType.kAdagrad)
    p_ids, p_grads, p_out = api.pinned_copy(ids), api.pinned_copy(grads), api.pinned_empty(out.shape, np.float32)
    for name, fn in (("combined pull, pageable", lambda: grp.CombinePull(ids, off, out=out)),
                     ("combined push, pageable", lambda: grp.CombinePush(o, ids, off, grads, 0.01)),
                     ("combined pull, page-locked", lambda: grp.CombinePull(p_ids, off, out=p_out)),
                     ("combined push, page-locked", lambda: grp.CombinePush(o, p_ids, off, p_grads, 0.01))):
        fn()
        t0 = time.perf_counter()
        for _ in range(20):
            fn()
        dt = (time.perf_counter() - t0) / 20
        print("%-28s %d unique rows  %8.1f us  %.2e rows/s" % (name, ids.size, dt * 1e6, ids.size / dt), flush=True)
    # one table's request of 8192 ids, as arrays and in the reference's wire layout
    t = tables[0]
    one = per[0]
    g1 = grads[:one.size]
    rc, reply = t.PullWire(one)
    p_reply = api.pinned_empty(reply.size, np.uint8)
    p_one = api.pinned_copy(one)
    for name, fn in (("pull [n, dim], pageable", lambda: t.Pull(one)),
                     ("pull, wire layout, pageable", lambda: t.PullWire(one, reply=reply)),
                     ("pull, wire layout, page-locked", lambda: t.PullWire(p_one, reply=p_reply)),
                     ("push [n, dim], pageable", lambda: t.Push(o, one, g1, 0.01)),
                     ("push, wire layout, pageable", lambda: t.PushWire(o, one, reply, 1e-6)),
                     ("push, wire layout, page-locked", lambda: t.PushWire(o, p_one, p_reply, 1e-6))):
        fn()
        t0 = time.perf_counter()
        for _ in range(50):
            fn()
        dt = (time.perf_counter() - t0) / 50
        print("%-32s %d rows  %8.1f us" % (name, one.size, dt * 1e6), flush=True)
    grp.close()
    for t in tables:
        t.close()


def pooled():
    print("# multi-hot field of the DeepFM shape: 65536 samples x 13 fields, 1..20 ids per bag, dim 32,")
    print("# table of 1e7 rows, Zipf 1.1")
    space, dim, samples = 10**7, 32, 65536
    rng = np.random.default_rng(0)
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "3"})
    t = api.SparseTable(dim, init, capacity_hint=space)
    prefill(t, space, dim)
    bags = samples * 13
    lengths = rng.integers(1, 21, size=bags)
    off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
    n = int(off[-1])
    d_ids = api.DeviceArray.from_host(splitmix64(zipf_ranks(rng, 1.1, space, n)))
    d_off = api.DeviceArray.from_host(off)
    d_g = api.DeviceArray.from_host((rng.standard_normal((bags, dim)) * 1e-3).astype(np.float32))
    d_out = api.DeviceArray((bags, dim), np.float32)
    d_rows = api.DeviceArray((n, dim), np.float32)
    opt = api.Optim.create(api.OptimType.kAdam)
    print("bags %d ids %d" % (bags, n), flush=True)
    for name, fn in (
            ("pull of every id -> [n, dim]", lambda: t.Pull(d_ids, out=d_rows, async_=True)),
            ("pooled pull (mean) -> [bags, dim]", lambda: t.PullPooled(d_ids, d_off, "mean", out=d_out, async_=True)),
            ("push_raw of [n, dim] gradients", lambda: t.PushRaw(opt, d_ids, d_rows, 1e-3, async_=True)),
            ("pooled push (mean)", lambda: t.PushPooled(opt, d_ids, d_off, d_g, 1e-3, mode="mean", async_=True)),
            ("pooled push (sum)", lambda: t.PushPooled(opt, d_ids, d_off, d_g, 1e-3, mode="sum", async_=True))):
        print("%-36s %8.1f us" % (name, timed(t, fn, 5) * 1e6), flush=True)
    t.close()
    # the same field over a table that starts empty: each step draws its own ids
    t = api.SparseTable(dim, init, capacity_hint=space)
    t.reserve(space + space // 8)
    e0, e1 = api.Event(), api.Event()
    steps = []
    for i in range(6):
        d = api.DeviceArray.from_host(splitmix64(zipf_ranks(rng, 1.1, space, n)))
        rows_before = len(t)
        e0.record(t)
        assert t.PullPooled(d, d_off, "mean", out=d_out, async_=True)[0] == 0
        e1.record(t)
        assert t.sync() == 0
        steps.append("%.0f us (%d new rows)" % (e0.elapsed_ms(e1) * 1e3, len(t) - rows_before))
        d.free()
    print("pooled pull (mean), table empty at first, step by step: " + ", ".join(steps), flush=True)
    for a in (d_ids, d_off, d_g, d_out, d_rows):
        a.free()
    t.close()


def codec():
    print("# threshold codec, eta 0.75: bytes compress 12n + 12nnz, decode 4n + 16nnz")
    for n in (1 << 20, 4096 * 16384):
        rng = np.random.default_rng(1)
        d_g = api.DeviceArray.from_host(rng.standard_normal(n).astype(np.float32))
        bag = api.DenseBag(n)
        idx, val = api.DeviceArray(n, np.int64), api.DeviceArray(n, np.float32)
        nnz = bag.MaybeToCoo(1000, 0.75, d_g, idx, val)[2]
        dt = timed(bag, lambda: bag.MaybeToCoo(1000, 0.75, d_g, idx, val), 5, sync=api.synchronize)
        dense = api.DeviceArray(n, np.float32)

        def decode():
            api.lib().krk_coo_to_dense(api._ptr(idx), api._ptr(val), nnz, api._ptr(dense), n, api.DEVICE_PTRS)
        dd = timed(None, decode, 5)
        print("n %9d nnz %9d | compress (stale threshold) %7.1f us %5.0f GB/s | decode (blocking call) %7.1f us "
              "%5.0f GB/s" % (n, nnz, dt * 1e6, (12 * n + 12 * nnz) / dt / 1e9, dd * 1e6,
                              (4 * n + 16 * nnz) / dd / 1e9), flush=True)
        for a in (d_g, idx, val, dense):
            a.free()


def dense():
    print("# dense table, Adam: bytes 28P")
    for p in (150_000, 1 << 26):
        t = api.DenseTable(np.zeros(p, np.float32))
        o = api.Optim.create(api.OptimType.kAdam)
        g = api.DeviceArray.from_host(np.ones(p, np.float32))
        dt = timed(t, lambda: t.Push(o, g, 1e-3, async_=True), 50)
        print("P %9d | push %7.1f us %5.0f GB/s" % (p, dt * 1e6, 28 * p / dt / 1e9), flush=True)
        g.free()
        t.close()


def dense_group():
    print("# dense parameters of one model, Adam: 40 tables (2 x 150k, 6 x 16k, 32 x 64..2048) table by table and")
    print("# as one combined request (krk_dense_group_pull / _push)")
    rng = np.random.default_rng(0)
    sizes = [150_000, 150_000] + [16_384] * 6 + [int(x) for x in rng.integers(64, 2048, size=32)]
    tables = [api.DenseTable(np.zeros(n, np.float32)) for n in sizes]
    o = api.Optim.create(api.OptimType.kAdam)
    grads = [api.DeviceArray.from_host(np.ones(n, np.float32)) for n in sizes]
    outs = [api.DeviceArray(n, np.float32) for n in sizes]
    total = sum(sizes)

    def each_push():
        for t, g in zip(tables, grads):
            t.Push(o, g, 1e-3, async_=True)

    def each_pull():
        for t, d in zip(tables, outs):
            api.lib().krk_dense_pull(t.h, api._ptr(d), api.DEVICE_PTRS | api.ASYNC)

    def sync_each():
        for t in tables:
            t.sync()
    def wall(fn, reps=20):
        fn()
        sync_each()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        sync_each()
        return (time.perf_counter() - t0) / reps
    t_each_push, t_each_pull = wall(each_push), wall(each_pull)
    grp = api.DenseGroup(tables)
    d_g, d_out = api.DeviceArray.from_host(np.ones(total, np.float32)), api.DeviceArray(total, np.float32)
    t_push = timed(grp, lambda: grp.CombinePush(o, d_g, 1e-3, async_=True), 20)
    t_pull = timed(grp, lambda: grp.CombinePull(out=d_out, async_=True), 20)
    print("%d tables, %d parameters | push: one call a table %7.1f us (wall clock; the tables' streams run side by side), "
          "combined %6.1f us | pull: one call a table %7.1f us, combined %6.1f us" % (
              len(sizes), total, t_each_push * 1e6, t_push * 1e6, t_each_pull * 1e6, t_pull * 1e6), flush=True)
    grp.close()
    for t in tables:
        t.close()


def dct():
    print("# blockwise DCT-II, block 256, n = 4096 x 16384: 4 (n + n keep / 256) bytes; TFLOP/s counts the plain product's")
    print("#   2 n keep (the kernels fold the basis along its mirror symmetry and multiply in bf16 pieces at fp32 accuracy)")
    n = 4096 * 16384
    x = api.DeviceArray.from_host(np.random.default_rng(0).standard_normal(n).astype(np.float32))
    for keep in (64, 128, 256):
        y = api.DeviceArray((n // 256, keep), np.float32)
        back = api.DeviceArray(n, np.float32)
        fl = api.DEVICE_PTRS | api.ASYNC
        for name, fn in (
                ("forward", lambda: api.lib().krk_dct2_forward(api._ptr(x), api._ptr(y), n, keep, fl)),
                ("inverse", lambda: api.lib().krk_dct2_inverse(api._ptr(y), api._ptr(back), n, keep, fl))):
            dt = timed(None, fn, 10)
            print("keep %3d %s | %7.1f us %6.1f TFLOP/s %5.0f GB/s" % (
                keep, name, dt * 1e6, 2.0 * n * keep / dt / 1e12, 4.0 * (n + n // 256 * keep) / dt / 1e9), flush=True)
        y.free()
        back.free()


def hooks():
    print("# routing on the device: a ring of 8 nodes x 64 virtual nodes (blocking calls, device ids)")
    rng = np.random.default_rng(3)
    hashes = np.sort(rng.integers(0, 1 << 63, size=8 * 64, dtype=np.uint64) * np.uint64(2))
    ring = [(int(h), int(i % 8)) for i, h in enumerate(hashes)]
    for n in (98_600, 1_000_000):
        d_ids = api.DeviceArray.from_host(splitmix64(np.arange(n, dtype=np.uint64)))
        rh = np.ascontiguousarray([h for h, _ in ring], dtype=np.uint64)
        rn = np.ascontiguousarray([i for _, i in ring], dtype=np.uint64)
        owner, perm = api.DeviceArray(n, np.uint64), api.DeviceArray(n, np.int64)
        node_ids, counts, m = np.empty(8, np.uint64), np.empty(8, np.int64), api.C.c_int64()

        def call():
            rc = api.lib().krk_route_ids(7, api._ptr(rh), api._ptr(rn), len(ring), api._ptr(d_ids), n,
                                         api._ptr(owner), api._ptr(perm), api._ptr(node_ids), api._ptr(counts), 8,
                                         api.C.byref(m), api.DEVICE_PTRS)
            assert rc == 0 and m.value == 8
        call()
        t0 = time.perf_counter()
        reps = 10
        for _ in range(reps):
            call()
        dt = (time.perf_counter() - t0) / reps
        owner.free()
        perm.free()
        print("route %8d ids to their nodes (owner per id, stable partition) %8.1f us" % (n, dt * 1e6), flush=True)
        d_ids.free()
    init = api.Initializer.create(api.InitializerType.kConstant, {"value": "0"})
    rows = 10_000_000
    t = api.SparseTable(16, init, capacity_hint=rows)
    prefill(t, rows, 16)
    rh = np.ascontiguousarray([h for h, _ in ring], dtype=np.uint64)
    rn = np.ascontiguousarray([i for _, i in ring], dtype=np.uint64)
    d_sel, count = api.DeviceArray(rows, np.uint64), api.C.c_int64()

    def select():
        rc = api.lib().krk_sparse_select_routed(t.h, 7, api._ptr(rh), api._ptr(rn), len(ring), 3, 1, api._ptr(d_sel),
                                                rows, api.C.byref(count), api.DEVICE_PTRS)
        assert rc == 0
    select()
    t0 = time.perf_counter()
    for _ in range(5):
        select()
    dt = (time.perf_counter() - t0) / 5
    print("select the rows of one node among %d rows (%d selected, ids left on the device) %8.1f us" % (
        rows, count.value, dt * 1e6), flush=True)
    d_sel.free()
    t.close()


def copy():
    nbytes = 1 << 30
    a, b = api.DeviceArray(nbytes // 4, np.float32), api.DeviceArray(nbytes // 4, np.float32)
    api.lib().krk_memset(api._ptr(a), 1, nbytes)
    dt = timed(None, lambda: api.lib().krk_stream_copy(api._ptr(b), api._ptr(a), nbytes), 20)
    print("# plain copy of 1 GiB: %.1f us, %.0f GB/s read + write" % (dt * 1e6, 2 * nbytes / dt / 1e9), flush=True)


def lines():
    """Random 128-byte lines (krk_hbm_probe_lines) out of regions of growing size, twice: as the
    launches come (a launch's lines then fall on pages that were not touched for a while), and
    with four million lines of the same region touched just before each timed run, which leaves
    the region's address translations in the GPU's translation caches."""
    print("# random independent 128-byte lines out of the first R bytes of one 16 GiB allocation")
    print("#   cold: launch after launch of n lines; warm: 4M lines of the region touched before the timed launches")
    region_max = 1 << 34
    big = api.DeviceArray(region_max // 4, np.float32)
    api.lib().krk_memset(api._ptr(big), 1, region_max)
    api.synchronize()
    salt = [1]

    def probe(rmw, region, n):
        salt[0] += 1
        rc = api.lib().krk_hbm_probe_lines(rmw, api._ptr(big), region, n, salt[0] * 0x9E3779B97F4A7C15 % (1 << 64))
        assert rc == 0

    for region in (1 << 25, 1 << 28, 1 << 30, 1 << 32, 1 << 34):
        for n in (98_600, 1 << 20):
            cells = []
            for rmw in (0, 1):
                cold = timed(None, lambda: probe(rmw, region, n), 10)
                for _ in range(3):
                    probe(0, region, 1 << 22)
                warm = timed(None, lambda: probe(rmw, region, n), 10)
                cells.append("%s cold %6.1f us warm %6.1f us %5.1f G lines/s" % (
                    "read + write" if rmw else "read", cold * 1e6, warm * 1e6, n / warm / 1e9))
            print("R %6d MB n %8d | %s | %s" % (region >> 20, n, cells[0], cells[1]), flush=True)
    big.free()


# ---------------------------------------------------------------------------------------------
# The legs bench.py reports under "secondary": each returns a dict of figures. Times are HIP
# events around back-to-back launches on the stream the kernels run on, inputs resident in HBM.
# ---------------------------------------------------------------------------------------------
HBM_PEAK = 8.0e12
MFMA_F32_PEAK = 157.3e12


def _leg(ms, nbytes=None, flops=None, **more):
    out = {"ms": ms}
    if nbytes is not None:
        out.update(algorithmic_bytes=float(nbytes), achieved_gbs=nbytes / (ms * 1e-3) / 1e9,
                   frac=nbytes / (ms * 1e-3) / HBM_PEAK, bound="hbm")
    if flops is not None:
        out.update(flops=float(flops), achieved_tflops=flops / (ms * 1e-3) / 1e12,
                   frac=flops / (ms * 1e-3) / MFMA_F32_PEAK, bound="mfma")
    out.update(more)
    return out


def _states(optim_name):
    return {"adagrad": 1, "adam": 2, "rmsprop": 1}[optim_name]


def pull_bytes_expanded(n, u, dim):
    """Pull with the re-expansion on the device: ids in, each distinct row read once, n rows out."""
    return 8 * n + 4 * dim * u + 4 * dim * n


def push_raw_bytes(n, u, dim, states, adam=False):
    """Push with the dedup on the device: ids and one gradient row per position in, one fused
    read-modify-write per distinct row."""
    return u * (8 + 4 * dim + 8 * dim * (1 + states) + (16 if adam else 0)) + 8 * n + 4 * dim * n


def worker_boundary_leg(cfg, tables, group, optim, lr, n_batches=8, reps=20):
    """The Wide&Deep step as the worker holds it: every table's ids with their repeats. One
    combined pull of all N ids and one combined push that dedups, sums the gradients of equal
    ids and updates (worker/emitter.cc:185-283, 552-632 + ps/sparse_table.cc:33-108)."""
    from .workloads import make_batches
    dim = cfg["dim"]
    batches = make_batches(cfg, n_batches, seed=11, unique=False)
    dev, n_ids, n_unique = [], [], []
    for per_table in batches:
        off = api.TableGroup._offsets([ids.size for ids, _ in per_table])
        ids = np.concatenate([ids for ids, _ in per_table])
        g = np.concatenate([g for _, g in per_table])
        dev.append((api.DeviceArray.from_host(ids), api.DeviceArray.from_host(g), off))
        n_ids.append(ids.size)
        n_unique.append(sum(np.unique(i).size for i, _ in per_table))
    d_out = api.DeviceArray((max(n_ids), dim), np.float32)
    k = [0]

    def pull():
        k[0] += 1
        d_ids, _, off = dev[k[0] % n_batches]
        assert group.CombinePull(d_ids, off, out=d_out, async_=True)[0] == 0

    def push():
        k[0] += 1
        d_ids, d_g, off = dev[k[0] % n_batches]
        assert group.CombinePushRaw(optim, d_ids, off, d_g, lr, async_=True) == 0

    def step(noted):
        # the worker's sequence: the rows of a batch's ids, then the gradients of the same ids
        k[0] += 1
        d_ids, d_g, off = dev[k[0] % n_batches]
        assert group.CombinePull(d_ids, off, out=d_out, async_=True, note_rows=noted)[0] == 0
        assert group.CombinePushRaw(optim, d_ids, off, d_g, lr, async_=True, as_pulled=noted) == 0

    def noting_pull():
        k[0] += 1
        d_ids, _, off = dev[k[0] % n_batches]
        assert group.CombinePull(d_ids, off, out=d_out, async_=True, note_rows=True)[0] == 0

    t_pull, t_push, t_plain, t_step, t_noting = (timed(group, f, reps) for f in (
        pull, push, lambda: step(False), lambda: step(True), noting_pull))
    n, u, S = float(np.mean(n_ids)), float(np.mean(n_unique)), _states(cfg["optim"])
    b_pull, b_push = pull_bytes_expanded(n, u, dim), push_raw_bytes(n, u, dim, S)
    for d in dev:
        d[0].free()
        d[1].free()
    d_out.free()
    return {"workload": "wide_deep, ids with repeats: %d tables x %d ids, dim %d, %s" % (
                cfg["tables"], cfg["batch"], dim, cfg["optim"]),
            "ids_per_step": n, "distinct_rows_per_step": u,
            # step: the push reuses the rows the pull noted (KRK_NOTE_ROWS / KRK_IDS_AS_PULLED)
            "step": _leg(t_step * 1e3, b_pull + b_push),
            "step_ids_looked_up_twice": _leg(t_plain * 1e3, b_pull + b_push),
            "group_pull": _leg(t_pull * 1e3, b_pull),
            "group_push_raw": _leg(t_push * 1e3, b_push),
            # what the push adds to a step whose pull noted the rows: the flagged step less the noting pull
            "group_push_raw_ids_as_pulled": _leg((t_step - t_noting) * 1e3, b_push),
            "group_pull_noting_rows": _leg(t_noting * 1e3, b_pull), "ids_per_s": n / t_step}


def _single_table(cfg, seed, extra_rows=0):
    from .workloads import table_ids
    dim = cfg["dim"]
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": str(seed)})
    t = api.SparseTable(dim, init, capacity_hint=min(cfg["space"], 4 * 10**6))
    chunk = 1 << 22
    scratch = api.DeviceArray((min(chunk, cfg["space"]), dim), np.float32)
    t.reserve(cfg["space"] + cfg["space"] // 8 + extra_rows)
    for lo in range(0, cfg["space"], chunk):
        d = api.DeviceArray.from_host(table_ids(cfg, 0, lo, min(lo + chunk, cfg["space"])))
        t.Pull(d, out=scratch, async_=True)
        assert t.sync() == 0
        d.free()
    scratch.free()
    return t


def deepfm_leg(n_batches=3, reps=6):
    """cfg3: one table of 1e8 resident rows, dim 32, Adam; a step's 2.56M ids (Zipf 1.1) with
    their repeats: pull of all ids, push_raw (dedup + sum + update), and the same step at the
    server boundary (unique ids: pull + fused push)."""
    from .workloads import WORKLOADS, raw_batch
    cfg = WORKLOADS["deepfm"]
    dim, n = cfg["dim"], cfg["batch"]
    t = _single_table(cfg, seed=0)
    rng = np.random.default_rng(21)
    o = api.Optim.create(api.OptimType.kAdam)
    d_g = api.DeviceArray.from_host(rng.standard_normal((n, dim), dtype=np.float32) * np.float32(1e-3))
    d_out = api.DeviceArray((n, dim), np.float32)
    raw, uniq, us = [], [], []
    for _ in range(n_batches):
        ids = raw_batch(rng, cfg)
        u = np.unique(ids)
        rng.shuffle(u)
        raw.append(api.DeviceArray.from_host(ids))
        uniq.append(api.DeviceArray.from_host(u))
        us.append(u.size)
    k = [0]

    def nxt(arrs):
        k[0] += 1
        return arrs[k[0] % n_batches]

    def chk(rc):
        assert (rc[0] if isinstance(rc, tuple) else rc) == 0

    t_pull_all = timed(t, lambda: chk(t.Pull(nxt(raw), out=d_out, async_=True)), reps)
    t_push_raw = timed(t, lambda: chk(t.PushRaw(o, nxt(raw), d_g, 1e-3, async_=True)), reps)

    def unique_step():
        d = nxt(uniq)
        chk(t.Pull(d, out=d_out, async_=True))
        chk(t.Push(o, d, d_g, 1e-3, async_=True))
    t_unique = timed(t, unique_step, reps)
    u = float(np.mean(us))
    out = {"workload": "deepfm: 1 table, 1e8 resident rows, dim 32, Zipf 1.1, %d ids a step, Adam" % n,
           "ids_per_step": n, "distinct_rows_per_step": u,
           "pull_all_ids": _leg(t_pull_all * 1e3, pull_bytes_expanded(n, u, dim)),
           "push_raw": _leg(t_push_raw * 1e3, push_raw_bytes(n, u, dim, 2, adam=True)),
           "unique_boundary_step": _leg(t_unique * 1e3, u * (16 + 4 * dim * (2 + 1 + 2 * 3) + 16)),
           "unique_rows_per_s": u / t_unique}
    for a in raw + uniq + [d_g, d_out]:
        a.free()
    t.close()
    return out


def dup_heavy_leg(steps=8, warm=2):
    """cfg4: one table of 2e7 resident rows, dim 128, 1 048 576 Zipf(1.3) ids a step of which 5 %
    are ids the table has never seen (every timed step has its own), RMSprop (alpha 0.9) and
    Adagrad as separate passes. A step = pull of all ids (inserting and initialising the unseen
    ones) + push_raw."""
    from .workloads import WORKLOADS, raw_batch, splitmix64
    cfg = WORKLOADS["dup_heavy"]
    dim, n = cfg["dim"], cfg["batch"]
    total_steps = 2 * (steps + warm)
    fresh_per_step = n // 20
    t = _single_table(cfg, seed=0, extra_rows=total_steps * fresh_per_step)
    rng = np.random.default_rng(31)
    d_g = api.DeviceArray.from_host(rng.standard_normal((n, dim), dtype=np.float32) * np.float32(1e-2))
    d_out = api.DeviceArray((n, dim), np.float32)
    batches, us = [], []
    for i in range(total_steps):
        ids = raw_batch(rng, cfg)
        where = rng.choice(n, size=fresh_per_step, replace=False)
        # ids beyond the key space: never drawn by the Zipf ranks, new to the table at their step
        ids[where] = splitmix64(np.uint64(cfg["space"]) + np.arange(i * fresh_per_step, (i + 1) * fresh_per_step,
                                                                    dtype=np.uint64))
        batches.append(api.DeviceArray.from_host(ids))
        us.append(np.unique(ids).size)
    out = {"workload": "dup_heavy: 1 table, 2e7 resident rows, dim 128, Zipf 1.3, %d ids a step, 5 %% unseen" % n,
           "ids_per_step": n, "distinct_rows_per_step": float(np.mean(us))}
    e = [api.Event() for _ in range(3)]
    nxt = 0
    for name, o in (("rmsprop", api.Optim.create(api.OptimType.kRMSprop, {"alpha": "0.9"})),
                    ("adagrad", api.Optim.create(api.OptimType.kAdagrad))):
        pulls, pushes, u_timed = [], [], []
        for s in range(warm + steps):
            d = batches[nxt]
            e[0].record(t)
            assert t.Pull(d, out=d_out, async_=True)[0] == 0
            e[1].record(t)
            assert t.PushRaw(o, d, d_g, 1e-3, async_=True) == 0
            e[2].record(t)
            assert t.sync() == 0
            if s >= warm:
                pulls.append(e[0].elapsed_ms(e[1]))
                pushes.append(e[1].elapsed_ms(e[2]))
                u_timed.append(us[nxt])
            nxt += 1
        u = float(np.mean(u_timed))
        tp, tq = float(np.median(pulls)), float(np.median(pushes))
        b_pull, b_push = pull_bytes_expanded(n, u, dim), push_raw_bytes(n, u, dim, 1)
        out[name] = {"step": _leg(tp + tq, b_pull + b_push), "pull_with_inserts": _leg(tp, b_pull),
                     "push_raw": _leg(tq, b_push), "ids_per_s": n / ((tp + tq) * 1e-3)}
    for a in batches + [d_g, d_out]:
        a.free()
    t.close()
    return out


def codec_leg(reps=5):
    """cfg5 through the reference's emitter (worker/dct_emitter.cc:16-43): the error-feedback
    threshold codec on a fp32 [4096, 16384] N(0, 1) gradient, eta 0.75, life_span 1000. The first
    call selects the threshold, the timed ones run with it; decode = CooToDense. A second bag
    with life_span 1 re-selects its threshold at every call: what a selecting step costs warm
    (the very first call of a process also pays for its work space and is not what is timed)."""
    n = 4096 * 16384
    rng = np.random.default_rng(5)
    g = rng.standard_normal(n, dtype=np.float32)
    d_g = api.DeviceArray.from_host(g)
    bag = api.DenseBag(n)
    idx, val = api.DeviceArray(n, np.int64), api.DeviceArray(n, np.float32)
    nnz = bag.MaybeToCoo(1000, 0.75, d_g, idx, val)[2]
    api.synchronize()
    dense = api.DeviceArray(n, np.float32)
    assert api.lib().krk_coo_to_dense(api._ptr(idx), api._ptr(val), nnz, api._ptr(dense), n, api.DEVICE_PTRS) == 0
    # decode(coo) + residual restores the gradient exactly (the first call starts from a zero residual)
    back = dense.to_host() + bag.residual
    err = float(np.max(np.abs(back - g)))
    kept = dense.to_host()
    kept_err = float(np.max(np.abs(kept[kept != 0] - g[kept != 0]))) if nnz else 0.0
    nnz2 = [nnz]

    def compress():
        nnz2[0] = bag.MaybeToCoo(1000, 0.75, d_g, idx, val)[2]
    t_c = timed(bag, compress, reps, sync=api.synchronize)
    # every call selects: the residual grows from call to call, the count of kept entries with it
    sel = api.DenseBag(n)
    idx_sel, val_sel = api.DeviceArray(n, np.int64), api.DeviceArray(n, np.float32)
    nnz_sel = [0]

    def select():
        nnz_sel[0] = sel.MaybeToCoo(1, 0.75, d_g, idx_sel, val_sel)[2]
    t_select = timed(sel, select, reps, sync=api.synchronize)
    sel.close()
    idx_sel.free()
    val_sel.free()

    def decode():
        assert api.lib().krk_coo_to_dense(api._ptr(idx), api._ptr(val), nnz2[0], api._ptr(dense), n,
                                          api.DEVICE_PTRS) == 0
    t_d = timed(None, decode, reps)
    out = {"workload": "threshold codec, fp32 [4096, 16384] N(0,1), eta 0.75, life_span 1000",
           "n": n, "nnz_first_call": nnz, "nnz_timed_calls": nnz2[0],
           "compress_selecting_threshold": _leg(t_select * 1e3, 16 * n + 12 * nnz_sel[0]),
           "compress": _leg(t_c * 1e3, 12 * n + 12 * nnz2[0]),
           "decode": _leg(t_d * 1e3, 4 * n + 16 * nnz2[0]),
           "max_abs_error_of_kept_values": kept_err,
           "max_abs_error_decode_plus_residual_vs_gradient": err,
           "max_rel_error": 0.0 if err == 0.0 and kept_err == 0.0 else err / float(np.max(np.abs(g)))}
    for a in (d_g, idx, val, dense):
        a.free()
    bag.close()
    return out


def dct2_leg(reps=10):
    """cfg5 through the blockwise DCT-II (block 256; no reference counterpart): forward and inverse
    at keep 64 (the emitter's retention 1 - eta = 0.25) and keep 256 (round trip). Errors: the
    coefficients of the first 4096 blocks against scipy.fft.dct(norm="ortho") in float64, relative
    to the largest coefficient, and the keep-256 round trip against the input."""
    import scipy.fft
    n = 4096 * 16384
    x = np.random.default_rng(0).standard_normal(n, dtype=np.float32)
    d_x = api.DeviceArray.from_host(x)
    out = {"workload": "blockwise DCT-II, block 256, fp32 [4096, 16384] N(0,1)", "n": n}
    fl = api.DEVICE_PTRS | api.ASYNC
    for keep in (64, 256):
        y = api.DeviceArray((n // 256, keep), np.float32)
        back = api.DeviceArray(n, np.float32)
        tf = timed(None, lambda: api.lib().krk_dct2_forward(api._ptr(d_x), api._ptr(y), n, keep, fl), reps)
        ti = timed(None, lambda: api.lib().krk_dct2_inverse(api._ptr(y), api._ptr(back), n, keep, fl), reps)
        # Bytes the transform has to move against the HBM peak: memory is what every width waits
        # for (the kernels fold the basis along its mirror symmetry and multiply in bf16 pieces at
        # fp32 accuracy: 6 x n keep / 2 bf16 multiply-adds, a fifth of the matrix pipe's time at
        # keep 256). flops_plain_product is what a plain fp32 product would be charged, 2 n keep.
        nbytes = 4.0 * (n + n // 256 * keep)
        rec = {"forward": _leg(tf * 1e3, nbytes=nbytes), "inverse": _leg(ti * 1e3, nbytes=nbytes)}
        for r in rec.values():
            r.update(flops_plain_product=2.0 * n * keep,
                     plain_product_tflops=2.0 * n * keep / (r["ms"] * 1e-3) / 1e12)
        coeff = y.to_host()[:4096].astype(np.float64)
        want = scipy.fft.dct(x[:4096 * 256].reshape(4096, 256).astype(np.float64), type=2, norm="ortho")[:, :keep]
        rec["max_rel_error_vs_scipy"] = float(np.max(np.abs(coeff - want)) / np.max(np.abs(want)))
        if keep == 256:
            rt = back.to_host()
            rec["max_rel_error_round_trip"] = float(np.max(np.abs(rt - x)) / np.max(np.abs(x)))
        out["keep_%d" % keep] = rec
        y.free()
        back.free()
    d_x.free()
    return out


def legs():
    import json
    from .workloads import WORKLOADS
    for fn in (deepfm_leg, dup_heavy_leg, codec_leg, dct2_leg):
        print(fn.__name__, json.dumps(fn()), flush=True)


SECTIONS = {"legs": legs, "lines": lines, "copy": copy, "tables": tables, "inserts": inserts, "raw": raw, "combined": combined, "host": host, "pooled": pooled, "codec": codec, "dense": dense, "dense_group": dense_group, "dct2": dct, "hooks": hooks}


def main(argv):
    rc = api.lib().krk_runtime_init(0)
    if rc != 0:
        raise RuntimeError("no usable GPU: " + api.lib().krk_last_error_string().decode())
    # `legs` (the bench's secondary legs as json lines) only runs when it is named
    for name in argv or [n for n in SECTIONS if n != "legs"]:
        SECTIONS[name]()


if __name__ == "__main__":
    main(sys.argv[1:])
