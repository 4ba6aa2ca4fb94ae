"""Per-kernel timings of the table engine at the sizes of the benchmark configurations.

    python -m kraken_amd.microbench [lines] [copy] [tables] [raw] [combined] [host] [pooled] [codec] [dense] [dct2] [hooks]

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


def splitmix64(x):
    with np.errstate(over="ignore"):
        z = np.asarray(x, dtype=np.uint64) + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def zipf_ranks(rng, s, space, size):
    w = 1.0 / np.arange(1, space + 1, dtype=np.float64) ** s
    cdf = np.cumsum(w)
    cdf /= cdf[-1]
    return np.searchsorted(cdf, rng.random(size)).astype(np.uint64)


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

    for name, fn in (
            ("combined pull of all ids", lambda: grp.CombinePull(d_ids, off, out=d_out, async_=True)),
            ("combined push with repeats", lambda: grp.CombinePushRaw(o, d_ids, off, d_g, 0.01, async_=True)),
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


def dct():
    print("# blockwise DCT-II, block 256, n = 4096 x 16384: 2 n keep flop, 4 (n + n keep / 256) bytes")
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


SECTIONS = {"lines": lines, "copy": copy, "tables": tables, "raw": raw, "combined": combined, "host": host, "pooled": pooled, "codec": codec, "dense": dense, "dct2": dct, "hooks": hooks}


def main(argv):
    rc = api.lib().krk_runtime_init(0)
    if rc != 0:
        raise RuntimeError("no usable GPU: " + api.lib().krk_last_error_string().decode())
    for name in argv or list(SECTIONS):
        SECTIONS[name]()


if __name__ == "__main__":
    main(sys.argv[1:])
