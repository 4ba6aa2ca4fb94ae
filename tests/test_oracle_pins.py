"""Pins the CPU oracle before anything is compared against it.

Sources of truth used here, none of which is the oracle's own formula retyped:
  * golden vectors produced by the reference's own header-only containers
    compiled in place (tests/golden/ref_containers.json);
  * the known-answer vectors held by the reference's unit tests
    (kraken/test/t/math_test.cc:323-382, kraken/test/worker/emitter_test.cc);
  * library optimizers (torch.optim on CPU, fp32) that the reference's headers
    cite as their definition (ps/optim/sgd.h:10, adagrad.h:11-12, adam.h:11-12,
    rmsprop.h:10-11);
  * brute force and invariants on small inputs.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# --------------------------------------------------------------------------- #
# hash + container vs the compiled reference
# --------------------------------------------------------------------------- #

def test_hash64_matches_reference_vectors(oracle):
    g = json.load(open(os.path.join(GOLDEN, "ref_containers.json")))
    L = oracle.lib()
    for k, h in g["hash64"]:
        assert L.kro_hash64(int(k)) == int(h)
    for a, b, h in g["hash64_pair"]:
        assert L.kro_hash64_pair(int(a), int(b)) == int(h)


def test_routing_ring_matches_reference_vectors(oracle):
    """Router::Hit(utils::Hash(table, id)) as ps/ps.cc:100, 306 call it, against rings the
    reference's own router built and answered (tests/golden/make_ref_router_vectors.py)."""
    L = oracle.lib()
    for case in json.load(open(os.path.join(GOLDEN, "ref_router.json"))):
        ring = [(int(h), int(n)) for h, n in case["ring"]]
        assert ring == sorted(ring) and len(ring) == 3 * len(case["nodes"])      # router.cc:12, 153-157
        rh = np.array([h for h, _ in ring], np.uint64)
        rn = np.array([n for _, n in ring], np.uint64)
        ph, pn = rh.ctypes.data_as(C.POINTER(C.c_uint64)), rn.ctypes.data_as(C.POINTER(C.c_uint64))
        for hv, owner in case["hits"]:
            assert L.kro_ring_hit(ph, pn, len(ring), int(hv)) == int(owner)
        ids = [int(i) for i, _ in case["ids"]]
        want = np.array([int(o) for _, o in case["ids"]], np.uint64)
        assert np.array_equal(oracle.route_owners(ring, case["table_id"], ids), want)
        if len(case["nodes"]) > 1:
            assert len(set(want.tolist())) > 1
    assert L.kro_ring_hit(None, None, 0, 5) == 2**64 - 1                          # router.cc:263-265


def test_routing_ring_matches_reference_live(oracle):
    """The same against the reference's router compiled in place, where that binary exists."""
    tool = os.path.join(os.path.dirname(__file__), "..", "oracle", "_ref", "ref_router")
    if not os.path.exists(tool):
        pytest.skip("oracle/_ref/ref_router is not built (no reference tree here)")
    import subprocess
    text = subprocess.check_output([tool, "99", "500", "n0", "n1", "n2", "n3"], text=True)
    ring, ids = [], []
    for line in text.splitlines():
        kind, a, b = line.split()
        if kind == "vnode":
            ring.append((int(a), int(b)))
        elif kind == "id":
            ids.append((int(a), int(b)))
    got = oracle.route_owners(ring, 99, [i for i, _ in ids])
    assert np.array_equal(got, np.array([o for _, o in ids], np.uint64))


def test_container_matches_reference_vectors(oracle):
    g = json.load(open(os.path.join(GOLDEN, "ref_containers.json")))["container"]
    ins = np.array([int(x) for x in g["inserted"]], dtype=np.uint64)
    vals = np.arange(ins.size * 2, dtype=np.float32).reshape(ins.size, 2)
    t = oracle.SparseTable(2, oracle.init(oracle.INIT_CONSTANT, 0.0))
    t.load(ins, vals)
    assert len(t) == g["fresh"]
    for k, s in zip(ins[:40], g["slots"]):
        assert oracle.lib().kro_hit_slot(int(k)) == s
    ids, v, _, _ = t.export()
    assert [str(int(x)) for x in ids] == g["export_order"]
    # duplicate inserts are rejected: the first value wins, as in SkipList::Insert
    first = {}
    for k, row in zip(ins, vals):
        first.setdefault(int(k), row[0])
    for k, row in zip(ids, v):
        assert row[0] == first[int(k)]
    for k, hit, col in zip(g["probe"], g["hit"], g["first_col"]):
        assert t.contains(int(k)) == bool(hit)
        if hit:
            assert first[int(k)] == col


def test_container_matches_reference_live(oracle):
    """Same comparison against the compiled reference itself, when it is built."""
    import ctypes as C
    L = oracle.ref_lib()
    if L is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(5)
    ids = rng.integers(0, 2**64, size=20000, dtype=np.uint64)
    ids[::7] = ids[::-7][: ids[::7].size]  # some duplicates
    vals = rng.standard_normal((ids.size, 3)).astype(np.float32)
    m = L.ref_map_create()
    fresh = L.ref_map_insert(m, ids.ctypes.data_as(C.POINTER(C.c_uint64)), ids.size,
                             vals.ctypes.data_as(C.POINTER(C.c_float)), 3)
    t = oracle.SparseTable(3, oracle.init(oracle.INIT_CONSTANT, 0.0))
    t.load(ids, vals)
    assert len(t) == fresh
    order = np.empty(ids.size, np.uint64)
    n = L.ref_map_keys(m, order.ctypes.data_as(C.POINTER(C.c_uint64)))
    eid, ev, _, _ = t.export()
    assert n == eid.size and np.array_equal(order[:n], eid)
    probe = np.concatenate([ids[:500], rng.integers(0, 2**64, size=500, dtype=np.uint64)])
    hit = np.empty(probe.size, np.uint8)
    got = np.zeros((probe.size, 3), np.float32)
    L.ref_map_find(m, probe.ctypes.data_as(C.POINTER(C.c_uint64)), probe.size,
                   hit.ctypes.data_as(C.POINTER(C.c_uint8)),
                   got.ctypes.data_as(C.POINTER(C.c_float)), 3)
    rc, rows = t.pull(probe[hit == 1])
    assert rc == 0 and np.array_equal(rows, got[hit == 1])
    for k, h in zip(probe[500:520], hit[500:520]):
        assert t.contains(int(k)) == bool(h)
    # SkipList::Remove through the clean-up walk of ps/ps.cc:92-109: same rows go, the rest keep
    # their order and their values
    L.ref_map_erase.restype = C.c_int64
    L.ref_map_erase.argtypes = [C.c_void_p, C.POINTER(C.c_uint64), C.c_int64]
    drop = np.concatenate([ids[::3], rng.integers(0, 2**64, size=300, dtype=np.uint64)])
    removed = L.ref_map_erase(m, drop.ctypes.data_as(C.POINTER(C.c_uint64)), drop.size)
    assert t.erase(drop) == removed
    n = L.ref_map_keys(m, order.ctypes.data_as(C.POINTER(C.c_uint64)))
    eid, ev, _, _ = t.export()
    assert n == eid.size == fresh - removed and np.array_equal(order[:n], eid)
    L.ref_map_find(m, probe.ctypes.data_as(C.POINTER(C.c_uint64)), probe.size,
                   hit.ctypes.data_as(C.POINTER(C.c_uint8)),
                   got.ctypes.data_as(C.POINTER(C.c_float)), 3)
    found, rows = t.fetch(probe)
    assert np.array_equal(found, hit == 1) and np.array_equal(rows[found], got[hit == 1])
    assert len(t) == n                                   # fetch inserts nothing
    L.ref_map_destroy(m)


def test_erase_and_fetch_against_a_python_dict(oracle):
    """No reference needed: the table is a map, erase and fetch are map operations."""
    rng = np.random.default_rng(6)
    ids = rng.integers(0, 5000, size=4000).astype(np.uint64)
    vals = rng.standard_normal((ids.size, 2)).astype(np.float32)
    t = oracle.SparseTable(2, oracle.init(oracle.INIT_CONSTANT, 0.0))
    t.load(ids, vals)
    model = {}
    for k, v in zip(ids.tolist(), vals):
        model.setdefault(k, v)
    for round_ in range(3):
        drop = rng.integers(0, 5000, size=700).astype(np.uint64)
        want = sum(1 for k in set(drop.tolist()) if k in model)
        assert t.erase(drop) == want
        for k in drop.tolist():
            model.pop(k, None)
        assert len(t) == len(model)
        probe = rng.integers(0, 5000, size=900).astype(np.uint64)
        found, rows = t.fetch(probe)
        for k, f, r in zip(probe.tolist(), found, rows):
            assert f == (k in model)
            if f:
                assert np.array_equal(r, model[k])
        eid, _, _, _ = t.export()
        assert sorted(eid.tolist()) == sorted(model)


# --------------------------------------------------------------------------- #
# codec known-answer vectors held by the reference's math_test.cc
# --------------------------------------------------------------------------- #

KAT6 = np.array([-1.0, 1.0, 2.0, 3.0, -4.0, -0.1], np.float32)
KAT10 = np.array([-1.0, 1.0, 2.0, 3.0, -4.0, -0.1, 0.001, 0.00001, 0.000001, 128], np.float32)


def test_kat_abs(oracle):            # math_test.cc:323-331
    assert np.array_equal(oracle.absf(KAT6), np.array([1, 1, 2, 3, 4, 0.1], np.float32))


def test_kat_topk(oracle):           # math_test.cc:333-341 : signed values, descending
    for hw in (1, 2, 8):
        got = oracle.topk(KAT6, 4, hw_threads=hw)
        assert np.array_equal(got, np.array([3.0, 2.0, 1.0, -0.1], np.float32))


def test_kat_take(oracle):           # math_test.cc:343-354
    got = oracle.take(KAT6, [0, 1, 3, 5])
    assert np.array_equal(got, np.array([-1.0, 1.0, 3.0, -0.1], np.float32))


def test_kat_tocoo_todense(oracle):  # math_test.cc:356-370
    idx, val = oracle.to_coo(KAT10, 0.01)
    assert np.array_equal(idx, [0, 1, 2, 3, 4, 5, 9])
    dense = oracle.coo_to_dense(idx, val, 10)
    expect = np.array([-1.0, 1.0, 2.0, 3.0, -4.0, -0.1, 0.0, 0.0, 0.0, 128], np.float32)
    assert np.array_equal(dense, expect)


def test_kat_ltkeep(oracle):         # math_test.cc:372-382
    got = oracle.lt_keep(KAT10, 0.01)
    expect = np.array([0, 0, 0, 0, 0, 0, 0.001, 0.00001, 0.000001, 0], np.float32)
    assert np.array_equal(got, expect)


def test_topk_against_sort_and_chunk_quirk(oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(4096).astype(np.float32)
    k = 1024
    # t_num divides n: chunked selection equals a full sort
    got = oracle.topk(x, k, hw_threads=4)
    assert np.array_equal(got, np.sort(x)[::-1][:k])
    # t_num = 3 does not divide 4096: the last 4096 % 3 = 1 element is never examined
    # (t/math.cc:573-586); make that element the maximum and watch it go missing.
    y = x.copy()
    y[-1] = 100.0
    got = oracle.topk(y, k, t_num=3)
    assert 100.0 not in got
    assert np.array_equal(got, np.sort(y[:-1])[::-1][:k])
    assert oracle.kth_largest_abs(y, 1) == 100.0


def test_codec_error_feedback_invariants(oracle):
    rng = np.random.default_rng(1)
    n = 4096
    s = oracle.DctState(n)
    assert oracle.DctState(100).compress(np.ones(100, np.float32)) == (None, None)  # n < 256
    e_prev = np.zeros(n, np.float32)
    for step in range(5):
        g = rng.standard_normal(n).astype(np.float32)
        idx, val = s.compress(g, life_span=2, eta=0.75)
        f = g + e_prev
        k = int(n * (1.0 - 0.75))
        if step % 2 == 0:
            tau = np.sort(np.abs(f))[::-1][k - 1]
            assert s.tau == tau
            assert idx.size >= k
        assert np.all(np.diff(idx) > 0)
        assert np.array_equal(val, f[idx])
        assert np.all(np.abs(val) >= s.tau)
        # decode + residual reproduces the corrected gradient exactly
        dense = oracle.coo_to_dense(idx, val, n)
        assert np.array_equal(dense + s.residual, f)
        assert np.all(np.abs(s.residual) < s.tau)
        e_prev = s.residual
    assert s.step == 5


# --------------------------------------------------------------------------- #
# optimizers vs the library definitions the reference's headers cite
# --------------------------------------------------------------------------- #

def _torch_run(make_opt, w0, grads, lr):
    torch = pytest.importorskip("torch")
    p = torch.nn.Parameter(torch.tensor(w0.copy()))
    opt = make_opt(torch, [p], lr)
    for g in grads:
        p.grad = torch.tensor(g.copy())
        opt.step()
    return p.detach().numpy().copy(), opt.state[p]


def _oracle_run(oracle, o, w0, grads, lr):
    v = oracle.Value(w0)
    for g in grads:
        assert v.update(o, g, lr) == 0
    return v


def _inputs(n=37, steps=6, seed=0):
    rng = np.random.default_rng(seed)
    w0 = rng.standard_normal(n).astype(np.float32)
    grads = [(rng.standard_normal(n) * 0.5).astype(np.float32) for _ in range(steps)]
    return w0, grads


RTOL = 2e-6   # a handful of fp32 roundings in a different association order
ATOL = 2e-7


@pytest.mark.parametrize("conf", [
    {}, {"weight_decay": 0.01}, {"momentum": 0.9}, {"momentum": 0.9, "nesterov": True},
    {"momentum": 0.8, "dampening": 0.3}, {"momentum": 0.9, "weight_decay": 0.1, "nesterov": True},
])
def test_sgd_vs_torch(oracle, conf):
    w0, grads = _inputs()
    lr = 0.05
    v = _oracle_run(oracle, oracle.optim(oracle.SGD, **conf), w0, grads, lr)
    w, st = _torch_run(lambda t, ps, lr: t.optim.SGD(
        ps, lr=lr, momentum=conf.get("momentum", 0.0), dampening=conf.get("dampening", 0.0),
        weight_decay=conf.get("weight_decay", 0.0), nesterov=conf.get("nesterov", False)),
        w0, grads, lr)
    np.testing.assert_allclose(v.val, w, rtol=RTOL, atol=ATOL)
    if "momentum" in conf:
        np.testing.assert_allclose(v.state(oracle.ST_MOMENTUM_BUFFER),
                                   st["momentum_buffer"].numpy(), rtol=RTOL, atol=ATOL)
    else:
        assert v.state(oracle.ST_MOMENTUM_BUFFER) is None


def test_sgd_plain_is_the_references_own_known_answer(oracle):
    """emitter_test.cc:51-63, 89-110: after == before - lr * g, to 4 ULP."""
    w0, grads = _inputs(100, 1, seed=3)
    lr = np.float32(0.37)
    v = _oracle_run(oracle, oracle.optim(oracle.SGD), w0, grads, float(lr))
    expect = w0 - lr * grads[0]
    assert np.array_equal(v.val, expect)


@pytest.mark.parametrize("conf", [{}, {"weight_decay": 0.05}, {"eps": 1e-6}])
def test_adagrad_vs_torch(oracle, conf):
    w0, grads = _inputs(seed=1)
    lr = 0.05
    o = oracle.optim(oracle.ADAGRAD, **conf)
    v = _oracle_run(oracle, o, w0, grads, lr)
    w, st = _torch_run(lambda t, ps, lr: t.optim.Adagrad(
        ps, lr=lr, initial_accumulator_value=0.0, eps=conf.get("eps", 1e-10),
        weight_decay=conf.get("weight_decay", 0.0)), w0, grads, lr)
    np.testing.assert_allclose(v.val, w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(v.state(oracle.ST_STATE_SUM), st["sum"].numpy(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("conf", [{}, {"weight_decay": 0.02}, {"beta1": 0.8, "beta2": 0.9, "eps": 1e-6}])
def test_adam_vs_torch(oracle, conf):
    w0, grads = _inputs(seed=2, steps=8)
    lr = 1e-2
    o = oracle.optim(oracle.ADAM, **conf)
    v = _oracle_run(oracle, o, w0, grads, lr)
    w, st = _torch_run(lambda t, ps, lr: t.optim.Adam(
        ps, lr=lr, betas=(conf.get("beta1", 0.9), conf.get("beta2", 0.999)),
        eps=conf.get("eps", 1e-8), weight_decay=conf.get("weight_decay", 0.0)), w0, grads, lr)
    np.testing.assert_allclose(v.val, w, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(v.state(oracle.ST_FIRST_MOMENT), st["exp_avg"].numpy(), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(v.state(oracle.ST_SECOND_MOMENT), st["exp_avg_sq"].numpy(), rtol=RTOL, atol=ATOL)
    assert v.steps == 8 and int(st["step"]) == 8


def test_adam_amsgrad_special_cases(oracle):
    """The reference takes max over the bias-corrected second moment
    (ps/optim/adam.cc:63,72-75), which torch does not. Two cases still reduce to
    torch: one step, and a constant gradient (corrected v is then constant and
    equals torch's max(v)/bc2). The general case is evaluated in float64 below
    from the order of operations in adam.cc:57-75."""
    w0, _ = _inputs(seed=4)
    lr = 1e-2
    g = np.full_like(w0, 0.3)
    o = oracle.optim(oracle.ADAM, amsgrad=True)
    v = _oracle_run(oracle, o, w0, [g] * 5, lr)
    w, _ = _torch_run(lambda t, ps, lr: t.optim.Adam(ps, lr=lr, amsgrad=True), w0, [g] * 5, lr)
    np.testing.assert_allclose(v.val, w, rtol=1e-5, atol=1e-6)
    # shrinking gradients: corrected max stays at the early, larger value
    grads = [np.full_like(w0, s) for s in (1.0, 0.5, 0.1, 0.01)]
    v = _oracle_run(oracle, o, w0, grads, lr)
    w = w0.astype(np.float64)
    m = np.zeros_like(w)
    vv = np.zeros_like(w)
    vmax = np.zeros_like(w)
    for t, gg in enumerate(grads, 1):
        gg = gg.astype(np.float64)
        m = 0.9 * m + (1 - 0.9) * gg
        vv = 0.999 * vv + (1 - 0.999) * gg * gg
        vhat = vv / (1 - 0.999 ** t)
        vmax = np.maximum(vmax, vhat)
        w = w - (lr * (m / (1 - 0.9 ** t))) / (np.sqrt(vmax) + 1e-8)
    np.testing.assert_allclose(v.val, w, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(v.state(oracle.ST_SECOND_MOMENT_MAX), vmax, rtol=1e-5)


def test_adam_amsgrad_closed_forms(oracle):
    """What the mathematics fixes for the branch of ps/optim/adam.cc:66-75, without restating it.

    Impulse: g_1 = s*a, zero afterwards, beta1 = beta2 = 1/2, eps = 1. Then m_t = s*a/2^t and
    v_t = a^2/2^t, the corrected moments are s*a/(2^t - 1) and a^2/(2^t - 1), so the corrected
    second moment peaks at t = 1 with exactly a^2 and the running maximum stays there: every step
    divides by sqrt(a^2) + 1, and

        W_T = W_0 - lr * s*a/(a + 1) * sum_{t=1..T} 1/(2^t - 1).

    The partial sums are 1, 4/3, 31/21, 54/35, ... A maximum taken
    over the uncorrected moment (torch's order), no maximum at all, eps inside the root or a
    missing correction of m each give a different W_2 already.

    Growth: |g_t| doubling makes the corrected second moment grow at every step, so the maximum
    is always the newest value and the result is plain Adam's, which torch pins."""
    a = np.array([1.0, 2.0, 4.0, 0.5, 8.0, 0.25], np.float32)
    sgn = np.array([1, -1, 1, -1, -1, 1], np.float32)
    w0 = np.array([0.5, -1.0, 2.0, 0.0, -0.25, 3.0], np.float32)
    lr = 0.125
    o = oracle.optim(oracle.ADAM, amsgrad=True, beta1=0.5, beta2=0.5, eps=1.0)
    from fractions import Fraction
    exact = [sum(Fraction(1, 2 ** t - 1) for t in range(1, T + 1)) for T in range(1, 6)]
    assert exact[:4] == [Fraction(1), Fraction(4, 3), Fraction(31, 21), Fraction(54, 35)]
    v = oracle.Value(w0)
    zero = np.zeros_like(w0)
    for T in range(1, 6):
        assert v.update(o, (sgn * a) if T == 1 else zero, lr) == 0
        want = w0.astype(np.float64) - lr * (sgn * a / (a + 1.0)).astype(np.float64) * float(exact[T - 1])
        np.testing.assert_allclose(v.val, want, rtol=1e-6, atol=1e-7)
        np.testing.assert_array_equal(v.state(oracle.ST_SECOND_MOMENT_MAX), a * a)
    assert v.steps == 5

    w0, _ = _inputs(seed=6)
    rng = np.random.default_rng(7)
    base = (rng.choice([-1.0, 1.0], size=w0.size) * rng.uniform(0.5, 1.0, size=w0.size)).astype(np.float32)
    grads = [base * np.float32(2.0 ** t) for t in range(6)]
    for conf in ({"beta1": 0.5, "beta2": 0.5}, {}):
        o = oracle.optim(oracle.ADAM, amsgrad=True, **conf)
        v = _oracle_run(oracle, o, w0, grads, 1e-2)
        w, st = _torch_run(lambda t, ps, lr: t.optim.Adam(
            ps, lr=lr, betas=(conf.get("beta1", 0.9), conf.get("beta2", 0.999))), w0, grads, 1e-2)
        np.testing.assert_allclose(v.val, w, rtol=1e-5, atol=1e-6)
        # the maximum is the newest corrected second moment
        bc2 = 1.0 - conf.get("beta2", 0.999) ** 6
        np.testing.assert_allclose(v.state(oracle.ST_SECOND_MOMENT_MAX), st["exp_avg_sq"].numpy() / bc2, rtol=1e-5)


@pytest.mark.parametrize("conf", [
    {}, {"alpha": 0.9}, {"centered": True}, {"momentum": 0.7}, {"momentum": 0.7, "centered": True},
    {"weight_decay": 0.03, "alpha": 0.9, "eps": 1e-6},
])
def test_rmsprop_vs_torch(oracle, conf):
    w0, grads = _inputs(seed=5)
    lr = 1e-2
    o = oracle.optim(oracle.RMSPROP, **conf)
    v = _oracle_run(oracle, o, w0, grads, lr)
    w, st = _torch_run(lambda t, ps, lr: t.optim.RMSprop(
        ps, lr=lr, alpha=conf.get("alpha", 0.99), eps=conf.get("eps", 1e-8),
        weight_decay=conf.get("weight_decay", 0.0), momentum=conf.get("momentum", 0.0),
        centered=conf.get("centered", False)), w0, grads, lr)
    np.testing.assert_allclose(v.val, w, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(v.state(oracle.ST_SQUARE_AVERAGE), st["square_avg"].numpy(),
                               rtol=RTOL, atol=ATOL)
    if conf.get("centered"):
        np.testing.assert_allclose(v.state(oracle.ST_G_AVE), st["grad_avg"].numpy(), rtol=RTOL, atol=ATOL)
    if "momentum" in conf:
        np.testing.assert_allclose(v.state(oracle.ST_MOMENTUM_BUFFER),
                                   st["momentum_buffer"].numpy(), rtol=1e-5, atol=1e-6)


def test_optimizer_defaults_and_lazy_state(oracle):
    """ps/optim/optim.cc:23-101 defaults; state tensors appear on first use only."""
    a = oracle.optim(oracle.ADAGRAD)
    assert a.eps == np.float32(1e-10) and not a.has_weight_decay
    r = oracle.optim(oracle.RMSPROP)
    assert r.alpha == np.float32(0.99) and r.eps == np.float32(1e-8)
    ad = oracle.optim(oracle.ADAM)
    assert (ad.beta1, ad.beta2, ad.eps) == (np.float32(0.9), np.float32(0.999), np.float32(1e-8))
    v = oracle.Value(np.ones(4, np.float32))
    assert v.state(oracle.ST_STATE_SUM) is None and v.steps == 0
    assert v.update(a, np.ones(5, np.float32), 0.1) == 11      # size mismatch
    assert v.state(oracle.ST_STATE_SUM) is None
    assert v.update(a, np.ones(4, np.float32), 0.1) == 0
    assert v.state(oracle.ST_STATE_SUM) is not None


# --------------------------------------------------------------------------- #
# sparse table semantics, initialisers, dedup
# --------------------------------------------------------------------------- #

def test_sparse_table_semantics(oracle):
    """emitter_test.cc:65-110 shape: Constant init insert-on-pull, then SGD push."""
    v0 = 3.25
    t = oracle.SparseTable(100, oracle.init(oracle.INIT_CONSTANT, v0))
    rc, rows = t.pull([0, 1])
    assert rc == 0 and np.array_equal(rows, np.full((2, 100), v0, np.float32))
    assert len(t) == 2
    rng = np.random.default_rng(0)
    g = rng.standard_normal((2, 100)).astype(np.float32)
    lr = np.float32(0.6)
    assert t.push(oracle.optim(oracle.SGD), [0, 1], g, float(lr)) == 0
    rc, after = t.pull([0, 1])
    assert np.array_equal(after, np.float32(v0) - lr * g)
    # pull twice gives identical rows and inserts nothing new
    rc, again = t.pull([1, 0, 1])
    assert np.array_equal(again, after[[1, 0, 1]]) and len(t) == 2
    # unseen id on push -> 12, wrong gradient width -> 11, empty request -> 0
    assert t.push(oracle.optim(oracle.SGD), [0, 99], g, 0.1) == 12
    assert t.push(oracle.optim(oracle.SGD), [0, 1], g[:, :50], 0.1) == 11
    assert t.push(oracle.optim(oracle.SGD), [], np.zeros((0, 100), np.float32), 0.1) == 0
    rc, none = t.pull([])
    assert rc == 0 and none.shape == (0, 100)


def test_initialisers(oracle):
    d = 64
    # Xavier on a 1-D [d] tensor: fan_out = d, fan_in = 1 (t/math.cc:24-50)
    std = oracle.lib().kro_xavier_std(1.5, d)
    assert abs(std - 1.5 * np.sqrt(2.0 / (1 + d))) < 1e-7
    n = 4000
    ids = np.arange(n, dtype=np.uint64) * np.uint64(2654435761)
    def rows(init):
        return np.stack([oracle.init_row(init, int(i), d) for i in ids])
    x = rows(oracle.init(oracle.INIT_NORMAL, 0.5, 0.01, seed=7))
    assert abs(x.mean() - 0.5) < 1e-4 and abs(x.std() - 0.01) < 1e-4
    assert abs(((x - 0.5) / 0.01) ** 4).mean() - 3.0 < 0.1          # kurtosis of a normal
    # rows and elements are decorrelated
    assert abs(np.corrcoef(x[:, 0], x[:, 1])[0, 1]) < 0.06
    assert abs(np.corrcoef(x[0::2, 0], x[1::2, 0])[0, 1]) < 0.08
    u = rows(oracle.init(oracle.INIT_UNIFORM, -2.0, 3.0, seed=7))
    assert u.min() >= -2.0 and u.max() <= 3.0
    assert abs(u.mean() - 0.5) < 0.02 and abs(u.var() - 25.0 / 12.0) < 0.03
    xu = rows(oracle.init(oracle.INIT_XAVIER_UNIFORM, 1.0, seed=1))
    bound = np.sqrt(3.0) * np.sqrt(2.0 / (1 + d))
    assert np.abs(xu).max() <= bound * (1 + 1e-6) and abs(xu.std() - bound / np.sqrt(3)) < 2e-3
    xn = rows(oracle.init(oracle.INIT_XAVIER_NORMAL, 2.0, seed=1))
    assert abs(xn.std() - 2.0 * np.sqrt(2.0 / (1 + d))) < 2e-3
    # a different seed gives different rows, the same seed the same rows
    a = oracle.init_row(oracle.init(oracle.INIT_NORMAL, 0, 1, seed=1), 42, d)
    b = oracle.init_row(oracle.init(oracle.INIT_NORMAL, 0, 1, seed=2), 42, d)
    c = oracle.init_row(oracle.init(oracle.INIT_NORMAL, 0, 1, seed=1), 42, d)
    assert not np.array_equal(a, b) and np.array_equal(a, c)


def test_elementary_functions_of_the_normal_draw(oracle):
    """The normal initialiser's logarithm and sine / cosine are written out (so that the oracle
    and the kernels agree to the bit); here they are held against libm: every power of two, the
    ends of the ranges, and a random sample, to 1e-13 absolute (the draw is rounded to fp32)."""
    import ctypes as C
    import math
    L = oracle.lib()
    rng = np.random.default_rng(12)
    ks = [1, 2, 3, 2**24, 2**24 - 1, 11863283, 11863284] + [2**e for e in range(25)] + [2**e + 1 for e in range(24)]
    ks += [int(x) for x in rng.integers(1, 2**24 + 1, 20000)]
    worst = max(abs(L.kro_log_u24(k) - math.log(k / 2.0**24)) for k in ks)
    assert worst < 1e-13, worst
    assert L.kro_log_u24(2**24) == 0.0
    sn, cs = C.c_double(), C.c_double()
    js = [0, 1, 2**21 - 1, 2**21, 2**21 + 1, 2**22, 3 * 2**21, 2**23, 2**24 - 2**21 - 1, 2**24 - 2**21, 2**24 - 1]
    js += [int(x) for x in rng.integers(0, 2**24, 20000)]
    worst = 0.0
    for j in js:
        L.kro_sincos_u24(j, C.byref(sn), C.byref(cs))
        a = 2.0 * math.pi * j / 2.0**24
        worst = max(worst, abs(sn.value - math.sin(a)), abs(cs.value - math.cos(a)))
        assert abs(sn.value ** 2 + cs.value ** 2 - 1.0) < 1e-13
    assert worst < 1e-13, worst
    L.kro_sincos_u24(0, C.byref(sn), C.byref(cs))
    assert (sn.value, cs.value) == (0.0, 1.0)
    L.kro_sincos_u24(2**22, C.byref(sn), C.byref(cs))
    assert (sn.value, cs.value) == (1.0, 0.0)


def _brute_dedup(ids, grads=None):
    seen = {}
    uids = []
    inv = []
    acc = []
    for p, i in enumerate(ids):
        i = int(i)
        if i not in seen:
            seen[i] = len(uids)
            uids.append(i)
            if grads is not None:
                acc.append(grads[p].copy())
        elif grads is not None:
            acc[seen[i]] = acc[seen[i]] + grads[p]     # fp32 +=, position order
        inv.append(seen[i])
    return uids, inv, acc


@pytest.mark.parametrize("ids", [
    [], [5], [5, 5, 5, 5], [1, 2, 3, 4], [9, 1, 9, 2, 1, 9, 2**64 - 1, 0, 2**64 - 1],
])
def test_dedup_small(oracle, ids):
    ids = np.array(ids, dtype=np.uint64)
    uids, inv = oracle.dedup(ids)
    bu, bi, _ = _brute_dedup(ids)
    assert [int(x) for x in uids] == bu and list(inv) == bi


def test_dedup_sum_random(oracle):
    rng = np.random.default_rng(11)
    ids = rng.zipf(1.3, size=3000).astype(np.uint64)
    g = rng.standard_normal((ids.size, 8)).astype(np.float32)
    uids, out = oracle.dedup_sum(ids, g)
    bu, bi, acc = _brute_dedup(ids, g)
    assert [int(x) for x in uids] == bu
    assert np.array_equal(out, np.stack(acc))          # same order => bit-exact
    u2, inv = oracle.dedup(ids)
    assert np.array_equal(u2, uids) and np.array_equal(uids[inv], ids)
    # first-occurrence positions are increasing in unique order
    first = [int(np.argmax(ids == u)) for u in uids[:50]]
    assert first == sorted(first)


def test_dense_table_and_coo(oracle):
    rng = np.random.default_rng(3)
    n = 1000
    w0 = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    t = oracle.DenseTable(w0)
    assert np.array_equal(t.pull(), w0)                          # emitter_test.cc:36-49
    lr = np.float32(0.4)
    assert t.push(oracle.optim(oracle.SGD), g, float(lr)) == 0
    assert np.array_equal(t.pull(), w0 - lr * g)                 # emitter_test.cc:51-63
    assert t.push(oracle.optim(oracle.SGD), g[:10], 0.1) == 11
    # COO gradient == densified gradient; empty COO leaves Adam's step counter alone
    a = oracle.DenseTable(w0)
    b = oracle.DenseTable(w0)
    idx, val = oracle.to_coo(g, 1.0)
    o = oracle.optim(oracle.ADAM)
    assert a.push_coo(o, idx, val, 0.01) == 0
    assert b.push(o, oracle.coo_to_dense(idx, val, n), 0.01) == 0
    assert np.array_equal(a.pull(), b.pull()) and a.steps == 1
    assert a.push_coo(o, [], [], 0.01) == 0 and a.steps == 1
    # repeated COO indices accumulate (t/math.cc:1043 "Should add the r maybe same")
    d = oracle.coo_to_dense([3, 3, 5], [1.0, 2.0, 4.0], 8)
    assert np.array_equal(d, np.array([0, 0, 0, 3, 0, 4, 0, 0], np.float32))


# --------------------------------------------------------------------------- #
# jagged pooling vs the compiled reference, a library routine and autograd
# --------------------------------------------------------------------------- #

def _jagged_cases():
    for c in json.load(open(os.path.join(GOLDEN, "ref_jagged.json")))["cases"]:
        col = c["col"]
        off = np.array(c["offsets"], np.int64)
        yield (c, col, off, np.array(c["values"], np.float32).reshape(-1, col),
               np.array(c["grads"], np.float32).reshape(-1, col))


def test_jagged_forward_matches_reference_vectors(oracle):
    for c, col, off, v, g in _jagged_cases():
        for mode in ("sum", "mean"):
            want = np.array(c[mode + "_forward"], np.float32).reshape(-1, col)
            got = oracle.jagged_forward(v, off, mode, c["patch_value"])
            assert np.array_equal(got, want), (mode, col)


def test_jagged_backward_matches_reference_vectors(oracle):
    for c, col, off, v, g in _jagged_cases():
        want = np.array(c["mean_backward"], np.float32).reshape(-1, col)
        got = oracle.jagged_backward(off, g, "mean")
        live = want != np.float32(c["sentinel"])      # rows of non-empty bags
        assert live.all()
        assert np.array_equal(got, want)
        # the reference's SumBackward only ever writes the first row of a bag; where it wrote,
        # the oracle agrees, and everywhere else the oracle holds the bag's gradient
        ref = np.array(c["sum_backward"], np.float32).reshape(-1, col)
        got = oracle.jagged_backward(off, g, "sum")
        firsts = off[:-1][off[1:] > off[:-1]]
        wrote = np.zeros(ref.shape[0], bool)
        wrote[firsts] = True
        assert np.array_equal(got[wrote], ref[wrote])
        assert (ref[~wrote] == np.float32(c["sentinel"])).all()
        bag_of = np.repeat(np.arange(off.size - 1), np.diff(off))
        assert np.array_equal(got, g[bag_of])


def test_jagged_matches_torch_segment_reduce_and_autograd(oracle):
    """Independent of the reference build: torch.segment_reduce for the forward, autograd of
    an index_add formulation for the backward (the transpose the reference's SumBackward was
    meant to be)."""
    import torch
    rng = np.random.default_rng(9)
    lengths = rng.integers(0, 9, size=40)
    off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
    # values on a binary grid: every order of summation gives the same fp32 result
    v = (rng.integers(-512, 513, size=(int(off[-1]), 6)) / 256.0).astype(np.float32)
    tv = torch.tensor(v, requires_grad=True)
    for mode in ("sum", "mean"):
        want = torch.segment_reduce(tv, mode, offsets=torch.tensor(off))
        got = oracle.jagged_forward(v, off, mode, 0.5)
        nonempty = lengths > 0
        np.testing.assert_allclose(got[nonempty], want.detach().numpy()[nonempty], rtol=1e-6, atol=0)
        assert (got[~nonempty] == 0.5).all()
        g = (rng.integers(-64, 65, size=(lengths.size, 6)) / 64.0).astype(np.float32)
        bag_of = torch.tensor(np.repeat(np.arange(lengths.size), lengths))
        pooled = torch.zeros(lengths.size, 6).index_add(0, bag_of, tv)
        if mode == "mean":
            pooled = pooled / torch.tensor(np.maximum(lengths, 1), dtype=torch.float32)[:, None]
        (gv,) = torch.autograd.grad(pooled, tv, torch.tensor(g))
        np.testing.assert_allclose(oracle.jagged_backward(off, g, mode), gv.numpy(), rtol=1e-6, atol=0)


def test_jagged_matches_reference_live(oracle):
    L = oracle.ref_jagged_lib()
    if L is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    import ctypes as C
    rng = np.random.default_rng(10)
    lengths = rng.integers(0, 30, size=200)
    off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
    for col in (3, 8, 32):
        v = rng.standard_normal((int(off[-1]), col)).astype(np.float32)
        for mode in ("sum", "mean"):
            want = np.empty((lengths.size, col), np.float32)
            getattr(L, "ref_jagged_%s_forward" % mode)(
                v.ctypes.data_as(C.POINTER(C.c_float)), col, off.ctypes.data_as(C.POINTER(C.c_int64)),
                lengths.size, -1.5, want.ctypes.data_as(C.POINTER(C.c_float)))
            assert np.array_equal(oracle.jagged_forward(v, off, mode, -1.5), want)
