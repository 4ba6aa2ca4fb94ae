"""CPU-side checks of bench.py: it measures one GPU and says so when asked for more, and every
counter figure it carries names a summary that exists under profiles/."""
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


def test_carried_counter_figures_point_at_committed_summaries():
    b = _bench()
    carried = list(b.COUNTER_FIGURES.items()) + [("dim %d" % d, v) for d, v in b.COUNTER_FIGURES_BY_DIM.items()]
    assert {"wide_deep", "dup_heavy", "deepfm"} <= set(b.COUNTER_FIGURES)
    for name, fig in carried:
        assert os.path.exists(os.path.join(ROOT, fig["source"])), (name, fig["source"])
        assert fig["traffic"] > 0 and 0.0 < fig["tcc_hit_rate"] < 1.0
    for name in b.COUNTER_FIGURES:
        assert name in b.WORKLOADS


def test_algorithmic_bytes_per_row_of_the_headline_metric():
    # Adagrad pull + push per unique row = 16 + 28 D bytes: 464 at D = 16, 912 at 32, 1808 at 64
    b = _bench()
    for dim, want in ((16, 464), (32, 912), (64, 1808)):
        pull = 8 + 8 * dim
        push = 8 + 4 * dim + 8 * dim * (1 + b.state_arrays("adagrad"))
        assert pull + push == want
