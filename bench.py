"""Benchmark of the sparse-table hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload wide_deep|deepfm|dup_heavy]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM: for every sparse table, pull the batch's unique ids and push one gradient row per
unique id (Adagrad), then one dense Adam push. The default workload is the Wide&Deep shape:
26 tables, 1e6 possible ids each drawn Zipf(1.05) and hashed with splitmix64, dim 16 fp32,
batch 8192 per table, Adagrad lr 0.05 with initial accumulator 0.1, plus a dense table of
150 000 fp32 parameters under Adam.

Prints ONE JSON line. `value` is unique rows pulled and pushed per second over the whole job.
`roofline` prices the dominant kernel (the fused Adagrad push) at its algorithmic bytes,
U * (8 + 4D + 16D) per launch, against 8 TB/s. `cpu_baseline` times the CPU oracle (a
restatement of the reference's table path; the checker, never the product) on the host cores of
the same machine on a bounded sample of the same workload.
"""
import argparse
import concurrent.futures
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the dominant kernel from hardware counters (FETCH_SIZE and WRITE_SIZE,
# each scaled by what it reads for the plain 1 GiB copy kernel); the runs and their commands are
# summarised in profiles/wide_deep_adagrad_d16_hbm_counters.md. Counters cannot be read from
# inside this script, so the figure is carried here for the workload it was measured on.
COUNTER_TRAFFIC_BYTES = {"wide_deep": 45.3e6}

WORKLOADS = {
    # name: tables, id space, zipf s, dim, ids per table per step, optimizer, dense params
    "wide_deep": dict(tables=26, space=10**6, s=1.05, dim=16, batch=8192, optim="adagrad",
                      dense=150_000, prefill=0),
    "wide_deep_d32": dict(tables=26, space=10**6, s=1.05, dim=32, batch=8192, optim="adagrad",
                          dense=150_000, prefill=0),
    "deepfm": dict(tables=1, space=10**8, s=1.1, dim=32, batch=65536 * 39, optim="adam", dense=0,
                   prefill=0),
    "dup_heavy": dict(tables=1, space=2 * 10**7, s=1.3, dim=128, batch=131072 * 8, optim="rmsprop",
                      dense=0, prefill=0),
}


def make_batches(cfg, n_batches, seed):
    """Per batch and table: unique hashed ids (the server boundary sees unique ids,
    worker/emitter.cc:131-149) and one gradient row per unique id."""
    from util import zipf_ranks, splitmix64
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n_batches):
        per_table = []
        for t in range(cfg["tables"]):
            ranks = zipf_ranks(rng, cfg["s"], cfg["space"], cfg["batch"])
            ids = np.unique(splitmix64(ranks + np.uint64(t) * np.uint64(cfg["space"])))
            rng.shuffle(ids)
            g = (rng.standard_normal((ids.size, cfg["dim"])) * 1e-2).astype(np.float32)
            per_table.append((ids, g))
        out.append(per_table)
    return out


def gpu_optim(api, name):
    if name == "adagrad":
        return api.Optim.create(api.OptimType.kAdagrad, {"initial_accumulator": "0.1"})
    if name == "adam":
        return api.Optim.create(api.OptimType.kAdam)
    return api.Optim.create(api.OptimType.kRMSprop, {"alpha": "0.9"})


def state_arrays(name):
    return {"adagrad": 1, "adam": 2, "rmsprop": 1}[name]


def table_ids(cfg, t, lo, hi):
    """Every id table t can ever see, in rank order: the hashed Zipf ranks lo..hi-1."""
    from util import splitmix64
    return splitmix64(np.arange(lo, hi, dtype=np.uint64) + np.uint64(t) * np.uint64(cfg["space"]))


def run_gpu(cfg, steps, warmup, n_batches=32):
    from kraken_amd import api
    rc = api.lib().krk_runtime_init(0)
    if rc != 0:
        raise RuntimeError("no usable GPU: " + api.lib().krk_last_error_string().decode())
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

    # several tables: one combined request per step (one launch each way); a single table
    # is called directly, as a server with one sparse table would
    def pull(d_ids, off, d_out):
        if single:
            tables[0].Pull(d_ids, out=d_out, async_=True)
        else:
            group.CombinePull(d_ids, off, out=d_out, async_=True)

    def push(d_ids, off, d_g):
        if single:
            tables[0].Push(optim, d_ids, d_g, lr, async_=True)
        else:
            group.CombinePush(optim, d_ids, off, d_g, lr, async_=True)

    def step(i):
        d_ids, d_g, d_out, off, _ = dev[i % n_batches]
        pull(d_ids, off, d_out)
        push(d_ids, off, d_g)
        if dense is not None:
            dense.Push(dense_opt, d_dense_g[i % n_batches], 1e-3, async_=True)

    def sync_all():
        rc = owner.sync()
        if rc != 0:
            raise RuntimeError("sparse tables reported error %d" % rc)
        if dense is not None:
            dense.sync()
        api.synchronize()

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
    for i in range(n_batches):
        step(i)
    sync_all()
    for i in range(warmup):
        step(i)
    sync_all()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    t_enq = time.perf_counter() - t0
    sync_all()
    dt = time.perf_counter() - t0
    print("host enqueue %.1f us/step, drained %.1f us/step" % (t_enq / steps * 1e6, dt / steps * 1e6),
          file=sys.stderr)
    rows = sum(dev[i % n_batches][4] for i in range(steps))

    # dominant kernel: the fused push over all tables of the request. M back-to-back launches
    # on the group's stream, bracketed by HIP events recorded on that stream.
    S = state_arrays(cfg["optim"])
    e0, e1 = api.Event(), api.Event()
    reps = 50 if cfg["batch"] < 10**6 else 10
    for kind in ("push", "pull"):
        for timed in (False, True):
            if timed:
                e0.record(owner)
            for j in range(reps):
                d_ids, d_g, d_out, off, _ = dev[j % n_batches]
                if kind == "push":
                    push(d_ids, off, d_g)
                else:
                    pull(d_ids, off, d_out)
            if timed:
                e1.record(owner)
            owner.sync()
        ms = e0.elapsed_ms(e1) / reps
        u = float(np.mean([dev[j % n_batches][4] for j in range(reps)]))
        if kind == "push":
            push_ms, push_u = ms, u
        else:
            pull_ms, pull_u = ms, u
    extra = 16 if cfg["optim"] == "adam" else 0
    push_bytes = push_u * (8 + 4 * dim + 8 * dim * (1 + S) + extra)
    pull_bytes = pull_u * (8 + 8 * dim)
    roofline = {
        "bound": "hbm", "kernel": "%spush_kernel<%s,4>" % ("" if single else "group_", cfg["optim"]),
        "achieved": push_bytes / (push_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": push_bytes / (push_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
        "bytes_per_launch": push_bytes, "us_per_launch": push_ms * 1e3,
        "pull_kernel": {"achieved": pull_bytes / (pull_ms * 1e-3) / 1e9, "us_per_launch": pull_ms * 1e3,
                        "bytes_per_launch": pull_bytes},
    }
    return dt, rows, roofline, batches


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
    """A plain device-to-device copy of known size: the measured bandwidth ceiling."""
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
    return {"kernel": "stream_copy_kernel", "bytes_read": nbytes, "bytes_written": nbytes,
            "us_per_launch": dt * 1e6, "copy_gbs_read_plus_write": 2 * nbytes / dt / 1e9}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="wide_deep", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run the plain 1 GiB streaming-copy kernel (hardware byte counters are "
                         "scaled by what they read for it) and print its bandwidth")
    args = ap.parse_args()
    if args.copy_calibration:
        print(json.dumps(copy_calibration()))
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    cfg = WORKLOADS[args.workload]
    dt, rows, roofline, batches = run_gpu(cfg, args.steps, args.warmup)
    # the same achieved figure against what a plain copy kernel moves on this very box
    ceiling = copy_calibration(nbytes=1 << 30, reps=10)["copy_gbs_read_plus_write"]
    roofline["copy_ceiling"] = ceiling
    roofline["frac_of_copy_ceiling"] = roofline["achieved"] / ceiling
    value = rows / dt
    dim = cfg["dim"]
    S = state_arrays(cfg["optim"])
    per_row = 16 + 4 * dim * (2 + 1 + 2 * (1 + S)) + (16 if cfg["optim"] == "adam" else 0)
    roofline["traffic"] = COUNTER_TRAFFIC_BYTES.get(args.workload)
    line = {
        "metric": "sparse pull+push unique-rows/sec (%s, dim %d fp32)" % (cfg["optim"], dim),
        "value": value, "unit": "unique-rows/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "tables": cfg["tables"], "dim": dim,
                   "ids_per_table_per_step": cfg["batch"], "id_space": cfg["space"],
                   "zipf_s": cfg["s"], "optimizer": cfg["optim"], "dense_params": cfg["dense"],
                   "boundary": "unique ids (server boundary), inputs resident in HBM"},
        "algorithmic_bytes_per_row": per_row,
        "achieved_gbs_whole_step": value * per_row / 1e9,
        "roofline": roofline,
    }
    if not args.no_cpu:
        ncpu = min(16, os.cpu_count() or 1)
        # three points: one caller thread, the reference server's default of two
        # (ps_server_main.cc:6), and eight (its eight slot locks bound the concurrency)
        v1, s1 = run_cpu(cfg, batches, budget_s=8.0, threads=1)
        v2, s2 = run_cpu(cfg, batches, budget_s=8.0, threads=min(2, ncpu))
        threads = min(8, ncpu)
        v8, s8 = run_cpu(cfg, batches, budget_s=8.0, threads=threads)
        best, cores = max(((v1, 1), (v2, min(2, ncpu)), (v8, threads)))
        line["cpu_baseline"] = {
            "value": best, "unit": "unique-rows/s", "cores": cores, "kind": "port",
            "sample": "first 4 tables of the workload with their key space resident, %d steps "
                      "(same ids, gradients, optimizer) through the CPU oracle in process; "
                      "1 thread: %.3g rows/s, 2 threads: %.3g rows/s, %d threads: %.3g rows/s"
                      % (s1 + s2 + s8, v1, v2, threads, v8),
        }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
