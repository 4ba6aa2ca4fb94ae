"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
parses optimizer/initializer confs like the reference, and refuses to run without a GPU."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    if not os.path.exists(a.LIB_PATH):
        from kraken_amd import build
        build.build(verbose=False)
    a.lib()
    return a


def test_every_declared_symbol_is_exported(api):
    header = open(os.path.join(ROOT, "include", "kraken_hip.h")).read()
    names = sorted(set(re.findall(r"\b(krk_[a-z0-9_]+)\s*\(", header)))
    assert len(names) > 40
    L = C.CDLL(api.LIB_PATH)
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    # and the binding knows every one of them
    assert not [n for n in names if n not in api.EXPORTS]


def test_flag_bits_of_the_binding_are_the_headers(api):
    """The call flags are single, distinct bits, and the ctypes binding carries the header's values."""
    header = open(os.path.join(ROOT, "include", "kraken_hip.h")).read()
    flags = {n: int(v, 16) for n, v in re.findall(r"#define (KRK_(?:DEVICE_PTRS|ASYNC|NOTE_ROWS|IDS_AS_PULLED)) (0x[0-9a-f]+)u", header)}
    assert flags == {"KRK_DEVICE_PTRS": api.DEVICE_PTRS, "KRK_ASYNC": api.ASYNC, "KRK_NOTE_ROWS": api.NOTE_ROWS,
                     "KRK_IDS_AS_PULLED": api.IDS_AS_PULLED}
    bits = sorted(flags.values())
    assert all(b and b & (b - 1) == 0 for b in bits) and len(set(bits)) == len(bits)


def test_optim_conf_parsing_matches_oracle_defaults(api, oracle):
    """Optim::Create (ps/optim/optim.cc:18-105): defaults and has_* flags."""
    for type_ in (0, 1, 2, 3):
        g = api.Optim.create(type_).raw
        r = oracle.optim(type_)
        for f in ("type", "has_weight_decay", "weight_decay", "has_momentum", "momentum",
                  "has_dampening", "dampening", "nesterov", "beta1", "beta2", "eps", "amsgrad",
                  "alpha", "centered"):
            assert getattr(g, f) == getattr(r, f), (type_, f)
        assert g.initial_accumulator == 0.0
    g = api.Optim.create(3, {"weight_decay": "0.5", "momentum": "0.9", "dampening": "0.1",
                             "nesterov": "TRUE", "eps": "3"}).raw
    assert (g.has_weight_decay, g.has_momentum, g.has_dampening, g.nesterov) == (1, 1, 1, 1)
    assert g.eps == np.float32(1e-8)                 # SGD has no eps key
    g = api.Optim.create(1, {"amsgrad": "1", "beta1": "oops", "beta2": "0.5"}).raw
    assert g.amsgrad == 1 and g.beta1 == np.float32(0.9) and g.beta2 == np.float32(0.5)
    g = api.Optim.create(2, {"centered": "yes", "alpha": "0.9"}).raw
    assert g.centered == 0 and g.alpha == np.float32(0.9)   # only "true"/"1" are true (utils.h:83-87)
    assert api.Optim.create(4) is None


def test_initializer_conf_parsing(api):
    """Initializer::Create (ps/initializer/initializer.cc:22-61) defaults and keys."""
    I = api.Initializer
    assert (I.create(0).raw.a, I.create(0, {"value": "2.5"}).raw.a) == (0.0, 2.5)
    u = I.create(1).raw
    assert (u.a, u.b) == (0.0, 1.0)
    n = I.create(2, {"mean": "1", "stddev": "0.01", "seed": "7"}).raw
    assert (n.a, n.b, n.seed) == (1.0, np.float32(0.01), 7)
    assert I.create(3).raw.a == 1.0 and I.create(4, {"gain": "2"}).raw.a == 2.0
    assert I.create(5) is None


def test_error_messages(api):
    L = api.lib()
    assert L.krk_error_message(0) == b"Success"
    assert L.krk_error_message(12) == b"SparseId not exist"
    assert L.krk_error_message(11) == b"Uncompatible gradient"


def test_no_gpu_fails_loudly(api):
    """Without a GPU every object constructor fails with a device error; nothing computes on CPU."""
    L = api.lib()
    cnt = C.c_int()
    try:
        hip = C.CDLL("libamdhip64.so")
        have_gpu = hip.hipGetDeviceCount(C.byref(cnt)) == 0 and cnt.value > 0
    except OSError:
        have_gpu = False
    if have_gpu:
        pytest.skip("a GPU is present")
    with pytest.raises(api.KrakenHipError) as e:
        api.SparseTable(8, api.Initializer.create(0))
    assert e.value.code == api.E_DEVICE
    with pytest.raises(api.KrakenHipError):
        api.DenseTable(np.zeros(4, np.float32))
    with pytest.raises(api.KrakenHipError):
        api.DenseBag(1024)
    with pytest.raises(api.KrakenHipError):
        api.dedup(np.arange(4, dtype=np.uint64))
