"""CPU-side checks of bench.py: it measures one GPU and says so when asked for more, the counter
figures it prints are read out of the summaries under profiles/ (with the hash of the kernel
sources they were measured at), and its byte and line counts are the ones the metric is defined by."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_counter_figures_are_read_from_the_committed_summaries():
    b = _bench()
    figs = b.profile_figures()
    for key in (("wide_deep", 16), ("wide_deep", 32), ("wide_deep", 64), ("dup_heavy", 128), ("deepfm", 32)):
        assert key in figs, key
        fig = figs[key]
        assert os.path.exists(os.path.join(ROOT, fig["source"]))
        assert fig["traffic"] > 0 and 0.0 < fig["tcc_hit_rate"] < 1.0
        assert len(fig["kernel_sources"]) == 16 and fig["kernel"]
    # what the bench line gets: the figure, where it is from, and whether the kernels changed since
    roofline = {}
    b.attach_counter_figures(roofline, "wide_deep", 16)
    assert roofline["traffic"] == figs[("wide_deep", 16)]["traffic"]
    assert roofline["traffic_source"].startswith("profiles/")
    assert roofline["traffic_stale"] == (figs[("wide_deep", 16)]["kernel_sources"] != b.kernel_sources_hash())
    none = {}
    b.attach_counter_figures(none, "no such workload", 16)
    assert none == {}


def test_algorithmic_bytes_per_row_of_the_headline_metric():
    # Adagrad pull + push per unique row = 16 + 28 D bytes: 464 at D = 16, 912 at 32, 1808 at 64
    b = _bench()
    for dim, want in ((16, 464), (32, 912), (64, 1808)):
        pull = 8 + 8 * dim
        push = 8 + 4 * dim + 8 * dim * (1 + b.state_arrays("adagrad"))
        assert pull + push == want


def test_lines_per_row():
    # bucket + the record's lines: Adagrad records are 128 / 256 / 512 bytes at dim 16 / 32 / 64
    b = _bench()
    assert b.lines_per_row(16, 1, False) == (2, 1, 1)
    assert b.lines_per_row(32, 1, False) == (2, 1, 2)
    assert b.lines_per_row(64, 1, False) == (3, 1, 4)
    assert b.lines_per_row(32, 2, True) == (2, 1, 4)      # Adam: 384 bytes + the word's sector


def test_workload_generators_live_in_the_package():
    b = _bench()
    from kraken_amd import workloads
    assert b.WORKLOADS is workloads.WORKLOADS and b.make_batches is workloads.make_batches
    import numpy as np
    cfg = dict(workloads.WORKLOADS["wide_deep"], tables=2, batch=256)
    uniq = workloads.make_batches(cfg, 1, seed=3)
    raw = workloads.make_batches(cfg, 1, seed=3, unique=False)
    for (u, gu), (r, gr) in zip(uniq[0], raw[0]):
        assert np.unique(u).size == u.size and gu.shape == (u.size, 16) and gu.dtype == np.float32
        assert r.size == 256 and gr.shape == (256, 16)
