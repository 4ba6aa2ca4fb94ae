"""Shared helpers for the parity tests: seeded inputs and optimizer pairs."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

RTOL = 1e-5     # north-star tolerance for fp32 values
ATOL = 1e-7


# the workload generators live with the package: the bench and the tests draw the same inputs
from kraken_amd.workloads import splitmix64, zipf_ids, zipf_ranks  # noqa: E402,F401


OPTIM_CASES = [
    # (name, type index (info.h), conf) -- every flag combination of ps/optim/optim.cc:23-101
    ("sgd", 3, {}),
    ("sgd_wd", 3, {"weight_decay": 0.01}),
    ("sgd_mom", 3, {"momentum": 0.9}),
    ("sgd_nesterov", 3, {"momentum": 0.9, "nesterov": True}),
    ("sgd_damp", 3, {"momentum": 0.8, "dampening": 0.3, "weight_decay": 0.05}),
    ("adagrad", 0, {}),
    ("adagrad_wd", 0, {"weight_decay": 0.02, "eps": 1e-6}),
    ("adam", 1, {}),
    ("adam_wd", 1, {"weight_decay": 0.01, "beta1": 0.8, "beta2": 0.95, "eps": 1e-6}),
    ("adam_amsgrad", 1, {"amsgrad": True}),
    ("rmsprop", 2, {}),
    ("rmsprop_alpha", 2, {"alpha": 0.9, "weight_decay": 0.01}),
    ("rmsprop_centered", 2, {"centered": True}),
    ("rmsprop_mom", 2, {"momentum": 0.7}),
    ("rmsprop_all", 2, {"momentum": 0.7, "centered": True, "alpha": 0.95, "eps": 1e-6}),
]


def make_optims(oracle, api, type_, conf):
    """The same optimizer on both sides: oracle struct and the library's conf-string path."""
    o_ref = oracle.optim(type_, **conf)
    o_gpu = api.Optim.create(type_, {k: (str(v).lower() if isinstance(v, bool) else repr(v))
                                     for k, v in conf.items()})
    return o_ref, o_gpu


STATE_OF = {   # optimizer type -> state types worth comparing
    3: [1], 0: [2], 1: [3, 4, 5], 2: [6, 7, 1],
}


def assert_close(got, want, what="", rtol=RTOL, atol=ATOL):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    tol = atol + rtol * np.abs(want.astype(np.float64))
    bad = err > tol
    if bad.any():
        i = np.argmax(err - tol)
        raise AssertionError("%s: %d of %d differ; worst at %d: got %r want %r" % (
            what, int(bad.sum()), bad.size, i, got.ravel()[i], want.ravel()[i]))
