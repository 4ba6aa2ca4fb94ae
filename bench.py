"""Benchmark of the sparse-table hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload wide_deep|deepfm|dup_heavy]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM: for every sparse table, pull the batch's unique ids and push one gradient row per
unique id (Adagrad), then one dense Adam push. The default workload is the Wide&Deep shape:
26 tables, 1e6 possible ids each drawn Zipf(1.05) and hashed with splitmix64, dim 16 fp32,
batch 8192 per table, Adagrad lr 0.05 with initial accumulator 0.1, plus a dense table of
150 000 fp32 parameters under Adam.

Timing: all timed blocks of K steps are enqueued back to back; HIP events recorded on the stream
the sparse kernels run on separate the blocks (the last one after that stream has been made to
wait for the dense table's), and the host waits once, at the end. `ms_per_step` is the median
block's span / K, so it does not depend on how often the host drains the queue; the figure with a
host drain after every block is carried as `ms_per_step_host_drained`, and the step whose push is
told that its ids are the pull's (KRK_NOTE_ROWS / KRK_IDS_AS_PULLED: no second look-up) as
`ms_per_step_ids_as_pulled`. `value` comes from the plain step.

Prints ONE JSON line. `value` is unique rows pulled and pushed per second over the whole job.
`roofline` prices the dominant kernel (the fused Adagrad push) at its algorithmic bytes,
U * (8 + 4D + 16D) per launch, against 8 TB/s; `line_floor_us` next to every `us_per_launch` is
what the kernel's count of random 128-byte lines costs at the line rates measured in the same
run, plus one empty launch, and `lines_and_streams_us` adds the ids and gradient rows the
kernel streams in or the pulled rows it streams out at the streaming rates of the same run.
`secondary` holds the other configurations (ids with their repeats at
the worker boundary, DeepFM, the duplicate-heavy shape, the codec and the blockwise DCT), each
with its own algorithmic bytes or flops. `cpu_baseline` times the CPU oracle (a restatement of
the reference's table path; the checker, never the product) on the host cores of the same
machine on a bounded sample of the same workload.
"""
import argparse
import concurrent.futures
import gc
import hashlib
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from kraken_amd.workloads import WORKLOADS, make_batches, table_ids  # noqa: E402

HBM_PEAK_GBS = 8000.0
T_START = time.perf_counter()

# ---------------------------------------------------------------------------------------------
# Figures that hardware counters gave for the dominant kernel (HBM bytes per launch from
# FETCH_SIZE and WRITE_SIZE scaled by the plain copy kernel, L2 hit rate). Counters cannot be read
# from inside this process, so the summaries under profiles/ carry them in a machine-readable
# block, together with a hash of the kernel sources they were measured at:
#
#     <!-- bench-figures
#     {"workload": "wide_deep", "dim": 16, "kernel": "...", "traffic": 45.4e6,
#      "tcc_hit_rate": 0.456, "kernel_sources": "<sha of the sources at measuring time>"}
#     -->
#
# The bench line repeats them with their source file and says so when the sources have changed.
# ---------------------------------------------------------------------------------------------
KERNEL_SOURCES = ("sparse_table.hip", "sparse_internal.h", "krk_internal.h")


def kernel_sources_hash(names=KERNEL_SOURCES):
    h = hashlib.sha256()
    for n in names:
        with open(os.path.join(ROOT, "kraken_amd", "csrc", n), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profile_figures():
    """Every bench-figures block under profiles/ -> {(workload, dim): figures + "source"}."""
    out = {}
    pdir = os.path.join(ROOT, "profiles")
    if not os.path.isdir(pdir):
        return out
    for name in sorted(os.listdir(pdir)):
        if not name.endswith(".md"):
            continue
        with open(os.path.join(pdir, name)) as f:
            text = f.read()
        for m in re.finditer(r"<!-- bench-figures\s*(.*?)-->", text, re.S):
            for line in m.group(1).strip().splitlines():
                line = line.strip()
                if not line:
                    continue
                fig = json.loads(line)
                fig["source"] = "profiles/" + name
                out[(fig["workload"], int(fig["dim"]))] = fig
    return out


def attach_counter_figures(roofline, workload, dim):
    fig = profile_figures().get((workload, dim))
    if not fig:
        return
    roofline["traffic"] = fig["traffic"]
    roofline["tcc_hit_rate"] = fig.get("tcc_hit_rate")
    roofline["traffic_kernel"] = fig.get("kernel")
    roofline["traffic_source"] = fig["source"] + " (hardware counters of an earlier run of this command)"
    roofline["traffic_kernel_sources"] = fig.get("kernel_sources")
    roofline["traffic_stale"] = fig.get("kernel_sources") != kernel_sources_hash()


def gpu_optim(api, name):
    if name == "adagrad":
        return api.Optim.create(api.OptimType.kAdagrad, {"initial_accumulator": "0.1"})
    if name == "adam":
        return api.Optim.create(api.OptimType.kAdam)
    return api.Optim.create(api.OptimType.kRMSprop, {"alpha": "0.9"})


def state_arrays(name):
    return {"adagrad": 1, "adam": 2, "rmsprop": 1}[name]


def _percentiles(xs):
    xs = np.sort(np.asarray(xs, np.float64))
    return float(np.median(xs)), float(xs[int(0.1 * (xs.size - 1))]), float(xs[int(np.ceil(0.9 * (xs.size - 1)))])


def lines_per_row(dim, states, word):
    """128-byte lines one row costs: (read only by the pull, read only by the push, read and
    written back by the push). The index bucket is one line either way; a record's weights take
    ceil(4 D / 128) lines, the whole record (weights, state arrays, the 64-bit word's sector)
    ceil(bytes / 128)."""
    w_lines = -(-4 * dim // 128)
    rec_bytes = 4 * dim * (1 + states) + (64 if word else 0)
    return 1 + w_lines, 1, -(-rec_bytes // 128)


def run_gpu(cfg, steps, warmup, blocks=30, n_batches=32, with_worker_leg=False, drained_blocks=8,
            noted_blocks=10):
    """Builds the workload's tables, fills their key space and times `blocks` blocks of `steps`
    steps each between events on the stream the sparse kernels run on. -> dict of figures."""
    import ctypes as C
    from kraken_amd import api
    L = api.lib()
    rc = L.krk_runtime_init(0)
    if rc != 0:
        raise RuntimeError("no usable GPU: " + L.krk_last_error_string().decode())
    dim = cfg["dim"]
    batches = make_batches(cfg, n_batches, seed=1)
    init = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": "0"})
    tables = [api.SparseTable(dim, init, capacity_hint=min(cfg["space"], 4 * 10**6))
              for _ in range(cfg["tables"])]
    optim = gpu_optim(api, cfg["optim"])
    lr = 0.05 if cfg["optim"] == "adagrad" else 1e-3
    dense = None
    if cfg["dense"]:
        rng = np.random.default_rng(2)
        dense = api.DenseTable((rng.standard_normal(cfg["dense"]) * 0.01).astype(np.float32))
        dense_opt = api.Optim.create(api.OptimType.kAdam)
        d_dense_g = [api.DeviceArray.from_host((rng.standard_normal(cfg["dense"]) * 1e-3).astype(np.float32))
                     for _ in range(n_batches)]
    # inputs and outputs live in HBM before the clock starts: per batch the ids and gradient
    # rows of all tables concatenated, the way one combined request carries them
    dev = []
    for per_table in batches:
        off = api.TableGroup._offsets([ids.size for ids, _ in per_table])
        ids = np.concatenate([ids for ids, _ in per_table])
        g = np.concatenate([g for _, g in per_table])
        dev.append((api.DeviceArray.from_host(ids), api.DeviceArray.from_host(g),
                    api.DeviceArray((ids.size, dim), np.float32), off, ids.size))

    # steady state: every id of the key space is resident before timing, so a step's rows come
    # from HBM-sized tables (the hot head of the Zipf draw stays in cache, the tail does not)
    chunk = 1 << 22
    scratch = api.DeviceArray((min(chunk, cfg["space"]), dim), np.float32)
    for ti, t in enumerate(tables):
        # an eighth of headroom, as a table that grew by doubling has: one filled to the last
        # row would publish its row count after every launch to decide about growing
        t.reserve(cfg["space"] + cfg["space"] // 8)
        for lo in range(0, cfg["space"], chunk):
            d = api.DeviceArray.from_host(table_ids(cfg, ti, lo, min(lo + chunk, cfg["space"])))
            t.Pull(d, out=scratch, async_=True)
            t.sync()
            d.free()
    scratch.free()
    single = len(tables) == 1
    group = None if single else api.TableGroup(tables)
    owner = tables[0] if single else group          # whose stream the step's launches run on

    # The step's three calls through the C ABI, arguments converted once: a C++ server thread
    # pays no argument marshalling either. several tables: one combined request per step (one
    # launch each way); a single table is called directly.
    flags = api.DEVICE_PTRS | api.ASYNC
    o_raw = C.byref(optim.raw)
    calls = []
    for i in range(n_batches):
        d_ids, d_g, d_out, off, n = dev[i]
        p_ids, p_g, p_out = C.c_void_p(d_ids.ptr), C.c_void_p(d_g.ptr), C.c_void_p(d_out.ptr)
        if single:
            pull = (L.krk_sparse_pull, (tables[0].h, p_ids, n, p_out, flags))
            push = (L.krk_sparse_push, (tables[0].h, o_raw, p_ids, n, p_g, dim, lr, flags))
        else:
            p_off = off.ctypes.data_as(C.c_void_p)
            pull = (L.krk_group_pull, (group.h, p_ids, p_off, p_out, flags))
            push = (L.krk_group_push, (group.h, o_raw, p_ids, p_off, p_g, dim, lr, flags))
        dpush = None
        if dense is not None:
            dpush = (L.krk_dense_push, (dense.h, C.byref(dense_opt.raw), C.c_void_p(d_dense_g[i].ptr),
                                        cfg["dense"], 1e-3, flags))
        # the same two calls with the push told that its ids are the pull's (a second figure,
        # not the headline: the pull then notes every position's row and the push skips its look-up)
        noted_pull = (pull[0], pull[1][:-1] + (flags | api.NOTE_ROWS,))
        noted_push = (push[0], push[1][:-1] + (flags | api.IDS_AS_PULLED,))
        calls.append((pull, push, dpush, noted_pull, noted_push))

    def step(i, noted=False):
        pull, push, dpush = calls[i % n_batches][3 if noted else 0], calls[i % n_batches][4 if noted else 1], \
            calls[i % n_batches][2]
        rc = pull[0](*pull[1]) | push[0](*push[1])
        if dpush is not None:
            rc |= dpush[0](*dpush[1])
        if rc:
            raise RuntimeError("step failed: " + L.krk_last_error_string().decode())

    def sync_all():
        rc = owner.sync()
        if rc != 0:
            raise RuntimeError("sparse tables reported error %d" % rc)
        if dense is not None:
            dense.sync()
        api.synchronize()

    for i in range(n_batches):
        step(i)
    sync_all()
    for i in range(warmup):
        step(i)
    sync_all()
    rows_per_step = float(np.mean([dev[i % n_batches][4] for i in range(steps)]))
    marks = [api.Event() for _ in range(blocks + 1)]
    dense_done = api.Event()
    # the interpreter's garbage is collected between phases, not inside one: a collection stalls
    # the host for longer than several steps take on the device
    gc.collect()
    gc.disable()
    try:
        # 1. every block enqueued behind the one before, events in between, one wait at the end.
        #    An untimed block goes first so that the queue is never empty while the clock runs.
        t0 = time.perf_counter()
        for i in range(steps):
            step(i)
        marks[0].record(owner)
        for b in range(blocks):
            for i in range(steps):
                step(i)
            if b == blocks - 1 and dense is not None:
                # the span ends when the dense table's stream has finished too
                dense_done.record(dense)
                dense_done.wait(owner)
            marks[b + 1].record(owner)
        t1 = time.perf_counter()
        sync_all()
        per_step = [marks[b].elapsed_ms(marks[b + 1]) * 1e-3 / steps for b in range(blocks)]
        enqueue_s = (t1 - t0) / ((blocks + 1) * steps)
        gc.collect()
        # 2. the same blocks with the host waiting for every queue after each of them: what a
        #    caller that drains after K steps sees (the waits' cost is spread over K steps)
        drained = []
        for b in range(drained_blocks):
            t0 = time.perf_counter()
            for i in range(steps):
                step(i)
            sync_all()
            drained.append((time.perf_counter() - t0) / steps)
            gc.collect()
        # 3. as 1., with KRK_NOTE_ROWS on the pull and KRK_IDS_AS_PULLED on the push
        noted_marks = [api.Event() for _ in range(noted_blocks + 1)]
        for i in range(steps if noted_blocks else 0):
            step(i, True)
        noted_marks[0].record(owner)
        for b in range(noted_blocks):
            for i in range(steps):
                step(i, True)
            if b == noted_blocks - 1 and dense is not None:
                dense_done.record(dense)
                dense_done.wait(owner)
            noted_marks[b + 1].record(owner)
        sync_all()
        noted = [noted_marks[b].elapsed_ms(noted_marks[b + 1]) * 1e-3 / steps for b in range(noted_blocks)]
    finally:
        gc.enable()
    noted_med = float(np.median(noted)) if noted else float("nan")
    med, p10, p90 = _percentiles(per_step)
    drained_med = float(np.median(drained)) if drained else None
    print("dim %d: %.2f us/step between events (p10 %.2f, p90 %.2f; %d blocks of %d steps), %.2f us/step with a "
          "host drain per block, host enqueue %.1f us/step; %.2f us/step when the push reuses the pull's rows" % (
              dim, med * 1e6, p10 * 1e6, p90 * 1e6, blocks, steps, (drained_med or 0) * 1e6, enqueue_s * 1e6,
              noted_med * 1e6),
          file=sys.stderr)

    # the two kernels of the step: M back-to-back launches on the owner's stream, bracketed by
    # HIP events recorded on that stream
    S = state_arrays(cfg["optim"])
    e0, e1 = api.Event(), api.Event()
    reps = 50 if cfg["batch"] < 10**6 else 10
    timed = {}
    for kind in (1, 0):
        samples = []
        for trial in range(6):
            e0.record(owner)
            for j in range(reps):
                c = calls[j % n_batches][kind]
                c[0](*c[1])
            e1.record(owner)
            owner.sync()
            if trial:
                samples.append(e0.elapsed_ms(e1) / reps)
        timed[kind] = float(np.median(samples))
    push_ms, pull_ms = timed[1], timed[0]
    u = float(np.mean([dev[j % n_batches][4] for j in range(reps)]))
    extra = 16 if cfg["optim"] == "adam" else 0
    push_bytes = u * (8 + 4 * dim + 8 * dim * (1 + S) + extra)
    pull_bytes = u * (8 + 8 * dim)
    wide = 32 <= dim <= 128 and dim % 4 == 0
    pull_lines, push_read_lines, push_rmw_lines = lines_per_row(dim, S, cfg["optim"] == "adam")
    roofline = {
        "bound": "hbm",
        "kernel": "%spush%s_kernel<%s>" % ("" if single else "group_", "_wide" if wide and dim <= 64 else "",
                                            cfg["optim"]),
        "achieved": push_bytes / (push_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": push_bytes / (push_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
        "bytes_per_launch": push_bytes, "us_per_launch": push_ms * 1e3,
        "lines_per_row": {"read": push_read_lines, "read_and_written_back": push_rmw_lines},
        "pull_kernel": {"achieved": pull_bytes / (pull_ms * 1e-3) / 1e9, "us_per_launch": pull_ms * 1e3,
                        "bytes_per_launch": pull_bytes,
                        "frac": pull_bytes / (pull_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        "lines_per_row": {"read": pull_lines}},
        "rows_per_launch": u,
    }
    per_row = 16 + 4 * dim * (2 + 1 + 2 * (1 + S)) + extra
    res = {
        "value": rows_per_step / med, "ms_per_step": med * 1e3, "ms_per_step_p10": p10 * 1e3,
        "ms_per_step_p90": p90 * 1e3, "blocks": blocks, "rows_per_step": rows_per_step,
        "ms_per_step_host_drained": drained_med * 1e3 if drained_med else None,
        # KRK_NOTE_ROWS on the pull, KRK_IDS_AS_PULLED on the push: the worker's pull-then-push of
        # one batch with the second look-up of the ids left out. Not what `value` is computed from.
        "ms_per_step_ids_as_pulled": noted_med * 1e3 if noted else None,
        "frac_whole_step_ids_as_pulled": rows_per_step / noted_med * (16 + 4 * dim * (2 + 1 + 2 * (1 + S)) + (
            16 if cfg["optim"] == "adam" else 0)) / 1e9 / HBM_PEAK_GBS if noted else None,
        "host_enqueue_us_per_step": enqueue_s * 1e6,
        "algorithmic_bytes_per_row": per_row,
        "achieved_gbs_whole_step": rows_per_step / med * per_row / 1e9,
        "frac_whole_step": rows_per_step / med * per_row / 1e9 / HBM_PEAK_GBS,
        "roofline": roofline, "batches": batches,
    }
    if with_worker_leg and group is not None:
        from kraken_amd import microbench
        try:
            res["worker_boundary"] = microbench.worker_boundary_leg(cfg, tables, group, optim, lr)
        except Exception as e:   # a secondary leg never takes the headline down with it
            res["worker_boundary"] = {"error": repr(e)}
    # give the memory back before the next configuration is built
    if group is not None:
        group.close()
    for t in tables:
        t.close()
    if dense is not None:
        dense.close()
    for d in dev:
        for a in d[:3]:
            a.free()
    return res


def add_line_floors(roofline, ceil, dim):
    """line_floor_us: the kernel's random lines at the line rates this run measured (read-only
    lines at the read rate, lines written back at the read-modify-write rate) + one empty launch:
    a bound. lines_and_streams_us adds what the kernel streams besides (ids and gradient rows
    read, pulled rows written) at the streaming rates of the same run: an estimate of a launch in
    which the scattered lines and the streams take turns at the memory."""
    rd = ceil["random_lines"]["random_line_read_%d" % (1 << 22)]["lines_per_s"]
    rmw = ceil["random_lines"]["random_line_rmw_%d" % (1 << 22)]["lines_per_s"]
    empty = ceil["empty_launch_us"]
    u = roofline["rows_per_launch"]
    lp = roofline["lines_per_row"]
    roofline["line_floor_us"] = (u * lp["read"] / rd + u * lp["read_and_written_back"] / rmw) * 1e6 + empty
    roofline["lines_and_streams_us"] = roofline["line_floor_us"] + u * (8 + 4 * dim) / (ceil["read_ceiling"] * 1e9) * 1e6
    pk = roofline["pull_kernel"]
    pk["line_floor_us"] = u * pk["lines_per_row"]["read"] / rd * 1e6 + empty
    pk["lines_and_streams_us"] = pk["line_floor_us"] + (u * 8 / (ceil["read_ceiling"] * 1e9) +
                                                          u * 4 * dim / (ceil["write_ceiling"] * 1e9)) * 1e6
    return roofline["line_floor_us"] + pk["line_floor_us"]


def run_cpu(cfg, batches, budget_s=20.0, threads=1, n_tables=4, prefill_cap=2 * 10**6):
    """The oracle on the host, in process: the first n_tables tables of the workload with their
    key space resident (up to prefill_cap rows each), same ids, gradients and optimizer."""
    from oracle import binding as oracle
    dim = cfg["dim"]
    n_tables = min(n_tables, cfg["tables"])
    tables = [oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=0))
              for _ in range(n_tables)]
    for ti, t in enumerate(tables):
        for lo in range(0, min(cfg["space"], prefill_cap), 1 << 20):
            t.pull(table_ids(cfg, ti, lo, min(lo + (1 << 20), cfg["space"], prefill_cap)))
    if cfg["optim"] == "adagrad":
        o = oracle.optim(oracle.ADAGRAD)
        lr = 0.05
    elif cfg["optim"] == "adam":
        o = oracle.optim(oracle.ADAM)
        lr = 1e-3
    else:
        o = oracle.optim(oracle.RMSPROP, alpha=0.9)
        lr = 1e-3
    dense = None
    if cfg["dense"]:
        rng = np.random.default_rng(2)
        dense = oracle.DenseTable((rng.standard_normal(cfg["dense"]) * 0.01).astype(np.float32))
        dg = (rng.standard_normal(cfg["dense"]) * 1e-3).astype(np.float32)
        do = oracle.optim(oracle.ADAM)

    def one_table(args):
        t, ids, g = args
        t.pull(ids, mt=True)
        t.push(o, ids, g, lr, mt=True)
        return ids.size

    pool = concurrent.futures.ThreadPoolExecutor(max_workers=threads) if threads > 1 else None

    def step(i):
        work = [(t, ids, g) for t, (ids, g) in zip(tables, batches[i % len(batches)])]
        n = sum(pool.map(one_table, work)) if pool else sum(one_table(w) for w in work)
        if dense is not None:
            dense.push(do, dg, 1e-3)
        return n

    for i in range(2):                 # untimed warm-up (also inserts ids past prefill_cap)
        step(i)
    rows, steps = 0, 0
    t0 = time.perf_counter()
    while True:
        rows += step(steps)
        steps += 1
        if time.perf_counter() - t0 > budget_s or steps >= 200:
            break
    dt = time.perf_counter() - t0
    if pool:
        pool.shutdown()
    return rows / dt, steps


def copy_calibration(nbytes=1 << 30, reps=20):
    """The plain 1 GiB device-to-device copy kernel that hardware byte counters are scaled by."""
    from kraken_amd import api
    L = api.lib()
    if L.krk_runtime_init(0) != 0:
        raise RuntimeError("no usable GPU: " + L.krk_last_error_string().decode())
    a = api.DeviceArray(nbytes // 4, np.float32)
    b = api.DeviceArray(nbytes // 4, np.float32)
    L.krk_memset(api._ptr(a), 1, nbytes)
    for _ in range(3):
        L.krk_stream_copy(api._ptr(b), api._ptr(a), nbytes)
    api.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        L.krk_stream_copy(api._ptr(b), api._ptr(a), nbytes)
    api.synchronize()
    dt = (time.perf_counter() - t0) / reps
    a.free()
    b.free()
    return {"kernel": "stream_copy_kernel", "bytes_read": nbytes, "bytes_written": nbytes,
            "us_per_launch": dt * 1e6, "copy_gbs_read_plus_write": 2 * nbytes / dt / 1e9}


def hbm_ceilings(nbytes=1 << 31, verbose=False):
    """What this GPU's memory delivers to the simplest kernels, measured now: streaming read, fill
    and copy (best over unroll x non-temporal x workgroup count, HIP events on the null stream
    around 5 launches), random independent 128-byte lines over a 16 GiB region, read only and
    read-modify-write (the table kernels' access pattern without their index), each timed right
    after heavy traffic, and an empty launch. GB/s."""
    from kraken_amd import api
    L = api.lib()
    if L.krk_runtime_init(0) != 0:
        raise RuntimeError("no usable GPU: " + L.krk_last_error_string().decode())
    a = api.DeviceArray(nbytes // 4, np.float32)
    b = api.DeviceArray(nbytes // 4, np.float32)
    L.krk_memset(api._ptr(a), 1, nbytes)
    L.krk_memset(api._ptr(b), 2, nbytes)
    e0, e1 = api.Event(), api.Event()

    def timed(fn, reps=5):
        fn()
        e0.record(None)
        for _ in range(reps):
            fn()
        e1.record(None)
        return e0.elapsed_ms(e1) / reps * 1e-3

    best = {}
    table = []
    for kind, name, moved in ((0, "read", nbytes), (1, "write", nbytes), (2, "copy", 2 * nbytes)):
        for unroll in (1, 2, 4, 8):
            for nt in (0, 1):
                for blocks in (256, 512, 1024, 4096):
                    def run():
                        rc = L.krk_hbm_probe(kind, unroll, nt, blocks, api._ptr(b), api._ptr(a), nbytes)
                        if rc:
                            raise RuntimeError(L.krk_last_error_string().decode())
                    gbs = moved / timed(run) / 1e9
                    table.append((name, unroll, nt, blocks, gbs))
                    if gbs > best.get(name, (0,))[0]:
                        best[name] = (gbs, {"unroll": unroll, "nontemporal": nt, "workgroups": blocks})
    a.free()
    b.free()
    region = 1 << 34
    big = api.DeviceArray(region // 4, np.float32)
    L.krk_memset(api._ptr(big), 1, region)
    lines = {}
    salt = [1]

    def probe(n, kind):
        salt[0] += 1
        rc = L.krk_hbm_probe_lines(kind, api._ptr(big), region, n, salt[0] * 0x9E3779B97F4A7C15 % (1 << 64))
        if rc:
            raise RuntimeError(L.krk_last_error_string().decode())

    for n in (98600, 1 << 20, 1 << 22):
        for rmw, name in ((0, "random_line_read"), (1, "random_line_rmw")):
            # A sequence of nothing but small launches runs slower than the same launches right after
            # heavy traffic (98.6k lines over 16 GiB: 9-10 us against 4-4.5 us): the figure to hold a
            # table kernel against is the second, so every timing follows three 4M-line launches.
            for _ in range(3):
                probe(1 << 22, 0)
            sec = timed(lambda: probe(n, rmw), reps=10)
            lines["%s_%d" % (name, n)] = {"us_per_launch": sec * 1e6, "lines_per_s": n / sec,
                                          "gbs": n * 128 * (2 if rmw else 1) / sec / 1e9}
    empty_us = timed(lambda: probe(1, 0), reps=50) * 1e6     # one workgroup that reads one line
    big.free()
    out = {
        "read_ceiling": best["read"][0], "read_variant": best["read"][1],
        "write_ceiling": best["write"][0], "write_variant": best["write"][1],
        "copy_ceiling": best["copy"][0], "copy_variant": best["copy"][1],
        "random_line_read_ceiling": lines["random_line_read_%d" % (1 << 22)]["gbs"],
        "random_line_rmw_ceiling": lines["random_line_rmw_%d" % (1 << 22)]["gbs"],
        "random_lines": lines, "empty_launch_us": empty_us, "unit": "GB/s",
    }
    if verbose:
        out["stream_table"] = [dict(kind=k, unroll=u, nontemporal=nt, workgroups=bl, gbs=g)
                               for k, u, nt, bl, g in table]
    return out


def host_description():
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        affinity = len(os.sched_getaffinity(0))
    except AttributeError:
        affinity = os.cpu_count()
    return {"nproc": os.cpu_count(), "usable_cpus": affinity, "cpu_model": model,
            "pinning": "none (threads float over the usable cpus)"}


def secondary_legs(budget_s):
    """The other configurations, each a function of kraken_amd.microbench that returns a dict.
    A leg is skipped, and the line says so, when the run would pass its wall-clock budget."""
    from kraken_amd import microbench
    # the streaming legs first: after the 51 GB table of the DeepFM leg has come and gone the same
    # codec launches measure 8 % slower (the state the allocator leaves the device memory in)
    legs = (("codec", microbench.codec_leg, 20.0),
            ("dct2", microbench.dct2_leg, 15.0),
            ("deepfm", microbench.deepfm_leg, 45.0),
            ("dup_heavy", microbench.dup_heavy_leg, 60.0))
    out = {}
    for name, fn, estimate_s in legs:
        spent = time.perf_counter() - T_START
        if spent + estimate_s > budget_s:
            out[name] = {"skipped": "wall-clock budget: %.0f s spent, leg estimated at %.0f s, budget %.0f s" % (
                spent, estimate_s, budget_s)}
            continue
        t0 = time.perf_counter()
        try:
            out[name] = fn()
        except Exception as e:
            out[name] = {"error": repr(e)}
        out[name]["leg_wall_s"] = time.perf_counter() - t0
        gc.collect()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--blocks", type=int, default=30,
                    help="timed blocks of --steps steps each; the line carries their median, p10 and p90")
    ap.add_argument("--noted-blocks", type=int, default=10,
                    help="blocks of the second figure (push told that its ids are the pull's); 0 leaves it "
                         "out, as the committed profiles of the plain step do")
    ap.add_argument("--workload", default="wide_deep", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-dims", action="store_true", help="skip the dim 32 / dim 64 legs of the default workload")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the secondary legs (worker boundary, DeepFM, duplicate-heavy, codec, DCT)")
    ap.add_argument("--budget-s", type=float, default=270.0,
                    help="wall-clock budget of the whole run: a secondary leg that would pass it is skipped")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the plain 1 GiB streaming-copy kernel (hardware byte counters are "
                         "scaled by what they read for it) and print its bandwidth")
    ap.add_argument("--ceilings", action="store_true",
                    help="only measure the streaming and random-line ceilings (every variant listed)")
    args = ap.parse_args()
    if args.copy_calibration:
        print(json.dumps(copy_calibration()))
        return
    if args.ceilings:
        print(json.dumps(hbm_ceilings(verbose=True)))
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    cfg = WORKLOADS[args.workload]
    default = args.workload == "wide_deep"
    secondary = default and not args.no_secondary
    r = run_gpu(cfg, args.steps, args.warmup, blocks=args.blocks, with_worker_leg=secondary,
                noted_blocks=args.noted_blocks)
    batches = r.pop("batches")
    roofline = r.pop("roofline")
    ceil = hbm_ceilings()
    roofline["ceilings"] = ceil
    # the push reads and writes random lines: its honest ceiling is the random-line one
    roofline["frac_of_random_line_rmw_ceiling"] = roofline["achieved"] / ceil["random_line_rmw_ceiling"]
    roofline["copy_ceiling"] = ceil["copy_ceiling"]
    roofline["frac_of_copy_ceiling"] = roofline["achieved"] / ceil["copy_ceiling"]
    step_floor = add_line_floors(roofline, ceil, cfg["dim"])
    attach_counter_figures(roofline, args.workload, cfg["dim"])
    dim = cfg["dim"]
    line = {
        "metric": "sparse pull+push unique-rows/sec (%s, dim %d fp32)" % (cfg["optim"], dim),
        "value": r["value"], "unit": "unique-rows/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": r["ms_per_step"], "ms_per_step_p10": r["ms_per_step_p10"],
        "ms_per_step_p90": r["ms_per_step_p90"], "timed_blocks": r["blocks"],
        "timing": "HIP events between blocks on the sparse kernels' stream, blocks enqueued back to back",
        "ms_per_step_host_drained": r["ms_per_step_host_drained"],
        "ms_per_step_ids_as_pulled": r["ms_per_step_ids_as_pulled"],
        "frac_whole_step_ids_as_pulled": r["frac_whole_step_ids_as_pulled"],
        "host_enqueue_us_per_step": r["host_enqueue_us_per_step"],
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "tables": cfg["tables"], "dim": dim,
                   "ids_per_table_per_step": cfg["batch"], "id_space": cfg["space"],
                   "zipf_s": cfg["s"], "optimizer": cfg["optim"], "dense_params": cfg["dense"],
                   "unique_rows_per_step": r["rows_per_step"],
                   "boundary": "unique ids (server boundary), inputs resident in HBM"},
        "algorithmic_bytes_per_row": r["algorithmic_bytes_per_row"],
        "achieved_gbs_whole_step": r["achieved_gbs_whole_step"],
        "frac_whole_step": r["frac_whole_step"],
        "line_floor_us_whole_step": step_floor,
        "roofline": roofline,
    }
    worker = r.pop("worker_boundary", None)
    if default and not args.no_dims:
        by_dim = {}
        for d in (32, 64):
            c2 = dict(cfg, dim=d)
            r2 = run_gpu(c2, args.steps, args.warmup, blocks=args.blocks, noted_blocks=args.noted_blocks)
            r2.pop("batches")
            r2["line_floor_us_whole_step"] = add_line_floors(r2["roofline"], ceil, d)
            attach_counter_figures(r2["roofline"], args.workload, d)
            by_dim[str(d)] = r2
        line["by_dim"] = by_dim
    if secondary:
        sec = {"worker_boundary": worker} if worker is not None else {}
        sec.update(secondary_legs(args.budget_s - (0 if args.no_cpu else 30.0)))
        line["secondary"] = sec
    if not args.no_cpu:
        host = host_description()
        ncpu = min(16, host["usable_cpus"] or 1)
        # three points: one caller thread, the reference server's default of two
        # (ps_server_main.cc:6), and eight (its eight slot locks bound the concurrency)
        v1, s1 = run_cpu(cfg, batches, budget_s=7.0, threads=1)
        v2, s2 = run_cpu(cfg, batches, budget_s=7.0, threads=min(2, ncpu))
        threads = min(8, ncpu)
        v8, s8 = run_cpu(cfg, batches, budget_s=7.0, threads=threads)
        line["cpu_baseline"] = {
            "value": v2, "unit": "unique-rows/s", "cores": min(2, ncpu), "kind": "port",
            "threads_1": v1, "threads_2": v2, "threads_%d" % threads: v8, "host": host,
            "sample": "first 4 of the workload's %d tables with their key space resident, %d steps in all "
                      "(same ids, gradients, optimizer) through the CPU oracle in process; value = the "
                      "reference server's default of 2 caller threads" % (cfg["tables"], s1 + s2 + s8),
        }
    line["wall_s"] = time.perf_counter() - T_START
    print(json.dumps(line))


if __name__ == "__main__":
    main()
