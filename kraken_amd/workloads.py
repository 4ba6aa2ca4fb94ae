"""Synthetic inputs of the benchmark configurations: the generators the bench, the per-kernel
timings and the parity tests share, so that the GPU path and the CPU oracle are fed identical bytes.

Ids are splitmix64 of a Zipf rank (plus table * space, so that tables do not share ids); a batch is
generated on the host with numpy's seeded generator and copied to HBM before any clock starts.
"""
import numpy as np


def splitmix64(x):
    """Vectorised splitmix64 output function on uint64 arrays."""
    with np.errstate(over="ignore"):
        z = (np.asarray(x, dtype=np.uint64) + np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


_CDF_CACHE = {}


def zipf_ranks(rng, s, space, size):
    """Zipf(s) ranks in [0, space) by inverse-CDF on the truncated distribution."""
    key = (float(s), int(space))
    cdf = _CDF_CACHE.get(key)
    if cdf is None:
        w = 1.0 / np.arange(1, space + 1, dtype=np.float64) ** s
        cdf = np.cumsum(w)
        cdf /= cdf[-1]
        if space <= 2 * 10**7:       # larger tables (0.8 GB at 1e8) are not worth holding on to
            _CDF_CACHE.clear()
            _CDF_CACHE[key] = cdf
    return np.searchsorted(cdf, rng.random(size)).astype(np.uint64)


def zipf_ids(rng, s, space, size):
    """Ids of the benchmark configurations: splitmix64 of a Zipf rank."""
    return splitmix64(zipf_ranks(rng, s, space, size))


WORKLOADS = {
    # name: tables, id space, zipf s, dim, ids per table per step, optimizer, dense params
    "wide_deep": dict(tables=26, space=10**6, s=1.05, dim=16, batch=8192, optim="adagrad",
                      dense=150_000),
    "wide_deep_d32": dict(tables=26, space=10**6, s=1.05, dim=32, batch=8192, optim="adagrad",
                          dense=150_000),
    "deepfm": dict(tables=1, space=10**8, s=1.1, dim=32, batch=65536 * 39, optim="adam", dense=0),
    "dup_heavy": dict(tables=1, space=2 * 10**7, s=1.3, dim=128, batch=131072 * 8, optim="rmsprop",
                      dense=0),
    "dup_heavy_adagrad": dict(tables=1, space=2 * 10**7, s=1.3, dim=128, batch=131072 * 8,
                              optim="adagrad", dense=0),
}


def table_ids(cfg, t, lo, hi):
    """Every id table t can ever see, in rank order: the hashed Zipf ranks lo..hi-1."""
    return splitmix64(np.arange(lo, hi, dtype=np.uint64) + np.uint64(t) * np.uint64(cfg["space"]))


def raw_batch(rng, cfg, t=0):
    """One table's ids of one step as the worker sees them (repeats included)."""
    return splitmix64(zipf_ranks(rng, cfg["s"], cfg["space"], cfg["batch"]) +
                      np.uint64(t) * np.uint64(cfg["space"]))


def make_batches(cfg, n_batches, seed, unique=True, grad_scale=1e-2):
    """Per batch and table: (ids, gradient rows). unique: what the server boundary sees (unique
    ids in shuffled order, one gradient row each; worker/emitter.cc:131-149); otherwise what the
    worker holds (ids with their repeats, one gradient row per position)."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n_batches):
        per_table = []
        for t in range(cfg["tables"]):
            ids = raw_batch(rng, cfg, t)
            if unique:
                ids = np.unique(ids)
                rng.shuffle(ids)
            g = (rng.standard_normal((ids.size, cfg["dim"]), dtype=np.float32) * np.float32(grad_scale))
            per_table.append((ids, g))
        out.append(per_table)
    return out
