"""Dense table apply and the threshold ("DCT") codec on the GPU against the oracle.

Known answers come from the reference's own tests: dense pull round trip and SGD
(kraken/test/worker/emitter_test.cc:36-63), Abs/TopK/Take/ToCoo/ToDense/LtKeep vectors
(kraken/test/t/math_test.cc:323-382).
"""
import numpy as np
import pytest

from util import OPTIM_CASES, STATE_OF, assert_close, make_optims

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def test_dense_roundtrip_and_sgd(api, oracle):
    rng = np.random.default_rng(0)
    d0 = rng.standard_normal((10, 10)).astype(np.float32)
    g0 = rng.standard_normal((10, 10)).astype(np.float32)
    t = api.DenseTable(d0)
    rc, r0 = t.Pull()
    assert rc == 0 and np.array_equal(r0, d0.ravel())            # emitter_test.cc:36-49
    lr = 0.37
    assert t.Push(api.Optim.create(api.OptimType.kSGD), g0, lr) == 0
    assert np.array_equal(t.Pull()[1], (d0 - np.float32(lr) * g0).ravel())   # :51-63
    assert t.Push(api.Optim.create(api.OptimType.kSGD), g0.ravel()[:7], lr) == 11


@pytest.mark.parametrize("name,type_,conf", OPTIM_CASES, ids=[c[0] for c in OPTIM_CASES])
@pytest.mark.parametrize("n", [1000, 150_000, 4099])
def test_dense_optimizers_match_oracle(api, oracle, name, type_, conf, n):
    rng = np.random.default_rng(n + type_)
    w0 = rng.standard_normal(n).astype(np.float32)
    t = api.DenseTable(w0)
    r = oracle.DenseTable(w0)
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    for step in range(5):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        assert t.Push(o_gpu, g, 0.01) == 0
        assert r.push(o_ref, g, 0.01) == 0
    assert_close(t.Pull()[1], r.pull(), name)
    for st in STATE_OF[type_]:
        want = r.state(st)
        got = t.state(st)
        assert_close(got, want if want is not None else np.zeros(n, np.float32), "%s state %d" % (name, st))
    if type_ == 1:
        assert t.steps == r.steps == 5


def test_dense_coo_push(api, oracle):
    rng = np.random.default_rng(5)
    n = 20_000
    w0 = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    idx, val = oracle.to_coo(g, 1.0)
    for type_, conf in ((1, {}), (0, {}), (3, {"momentum": 0.9}), (2, {"centered": True})):
        t = api.DenseTable(w0)
        r = oracle.DenseTable(w0)
        o_ref, o_gpu = make_optims(oracle, api, type_, conf)
        for _ in range(3):
            assert t.PushCoo(o_gpu, idx, val, 0.01) == 0
            assert r.push_coo(o_ref, idx, val, 0.01) == 0
        assert_close(t.Pull()[1], r.pull(), "coo push type %d" % type_)
        # an empty COO gradient changes nothing, not even Adam's step counter (adam.cc:26-29)
        before = t.Pull()[1]
        assert t.PushCoo(o_gpu, np.zeros(0, np.int64), np.zeros(0, np.float32), 0.01) == 0
        assert np.array_equal(t.Pull()[1], before)
        if type_ == 1:
            assert t.steps == 3
    # repeated indices add up (t/math.cc:1043)
    t = api.DenseTable(np.zeros(8, np.float32))
    assert t.PushCoo(api.Optim.create(api.OptimType.kSGD), [3, 3, 5], [1.0, 2.0, 4.0], 1.0) == 0
    assert np.array_equal(t.Pull()[1], np.float32([0, 0, 0, -3, 0, -4, 0, 0]))


KAT10 = np.array([-1.0, 1.0, 2.0, 3.0, -4.0, -0.1, 0.001, 0.00001, 0.000001, 128], np.float32)


def test_coo_to_dense_known_answer(api, oracle):
    """math_test.cc:356-370: ToCoo(0.01) -> ToDense."""
    idx, val = oracle.to_coo(KAT10, 0.01)
    dense = api.coo_to_dense(idx, val, 10)
    assert np.array_equal(dense, np.float32([-1.0, 1.0, 2.0, 3.0, -4.0, -0.1, 0, 0, 0, 128]))
    assert np.array_equal(api.coo_to_dense([3, 3, 5], [1.0, 2.0, 4.0], 8),
                          np.float32([0, 0, 0, 3, 0, 4, 0, 0]))


def test_codec_small_passthrough(api):
    bag = api.DenseBag(100)
    assert bag.MaybeToCoo(1000, 0.75, np.ones(100, np.float32)) == (None, None)
    assert bag.step == 0


@pytest.mark.parametrize("n", [256, 4096, 65_536, 1_000_003])
@pytest.mark.parametrize("eta", [0.5, 0.75, 0.9])
def test_codec_matches_oracle(api, oracle, n, eta):
    """Three consecutive steps with life_span 2: a re-select, a stale-threshold step, a
    re-select; indices, values, threshold and residual all exact."""
    rng = np.random.default_rng(n)
    bag = api.DenseBag(n)
    ref = oracle.DctState(n)
    for step in range(3):
        g = rng.standard_normal(n).astype(np.float32)
        if step == 1:
            m = g[1::3].size
            g[::3][:m] = g[1::3]                   # ties around the threshold
        idx, val = bag.MaybeToCoo(2, eta, g)
        ridx, rval = ref.compress(g, life_span=2, eta=eta, exact_select=True)
        assert bag.tau == ref.tau
        assert np.array_equal(idx, ridx) and np.array_equal(val, rval)
        assert np.array_equal(bag.residual, ref.residual)
        if step % 2 == 0:
            assert idx.size >= int(n * (1.0 - eta))
    assert bag.step == ref.step == 3
    # decode(coo) + residual == corrected gradient, exactly
    dense = api.coo_to_dense(idx, val, n)
    assert np.array_equal(dense, oracle.coo_to_dense(ridx, rval, n))


def test_codec_reference_chunked_topk_agrees_when_chunks_divide(api, oracle):
    """The reference's TopK splits the tensor into t_num chunks and drops n mod t_num trailing
    elements (t/math.cc:573-586). When t_num divides n its threshold is the true k-th largest,
    which is what the GPU computes."""
    n = 8192
    rng = np.random.default_rng(3)
    g = rng.standard_normal(n).astype(np.float32)
    bag = api.DenseBag(n)
    ref = oracle.DctState(n)
    idx, val = bag.MaybeToCoo(1000, 0.75, g)
    ridx, rval = ref.compress(g, life_span=1000, eta=0.75, hw_threads=4, exact_select=False)
    assert bag.tau == ref.tau and np.array_equal(idx, ridx) and np.array_equal(val, rval)


def test_codec_device_pointers_and_capacity(api, oracle):
    n = 300_000
    rng = np.random.default_rng(8)
    g = rng.standard_normal(n).astype(np.float32)
    bag = api.DenseBag(n)
    small_i = np.empty(10, np.int64)
    small_v = np.empty(10, np.float32)
    with pytest.raises(api.KrakenHipError) as e:
        bag.MaybeToCoo(1000, 0.75, g, small_i, small_v)
    assert e.value.code == api.E_CAPACITY and bag.step == 0     # nothing was committed
    d_g = api.DeviceArray.from_host(g)
    d_idx, d_val, nnz = bag.MaybeToCoo(1000, 0.75, d_g)
    ref = oracle.DctState(n)
    ridx, rval = ref.compress(g, exact_select=True)
    assert nnz == ridx.size
    assert np.array_equal(d_idx.to_host()[:nnz], ridx) and np.array_equal(d_val.to_host()[:nnz], rval)
    assert np.array_equal(bag.residual, ref.residual)


@pytest.mark.parametrize("n", [1 << 22, (1 << 22) + 1, 5_000_003])
def test_coo_to_dense_large_tensors(api, oracle, n):
    """From 2^22 elements on the dense result is written tile by tile when the indices ascend
    strictly (what ToCoo produces); anything else is zeroed and scattered into. Both against the
    oracle: ascending with long gaps and a full last tile, every element present, nothing present,
    shuffled, with repeats (which add up, t/math.cc:1043)."""
    rng = np.random.default_rng(n)

    def check(idx, val):
        idx = np.ascontiguousarray(idx, np.int64)
        val = np.ascontiguousarray(val, np.float32)
        want = np.zeros(n, np.float32)
        np.add.at(want, idx, val)
        if np.unique(idx).size == idx.size:
            assert np.array_equal(want, oracle.coo_to_dense(idx, val, n))
        assert np.array_equal(api.coo_to_dense(idx, val, n), want)
        d = api.coo_to_dense(api.DeviceArray.from_host(idx), api.DeviceArray.from_host(val), n)
        assert np.array_equal(d.to_host(), want)

    quarter = np.sort(rng.choice(n, size=n // 4, replace=False))
    check(quarter, rng.standard_normal(quarter.size))
    few = np.array([0, 5, 4095, 4096, n - 4097, n - 1])          # empty tiles in between, both ends
    check(few, rng.standard_normal(few.size))
    check(np.arange(n), rng.standard_normal(n))                   # every element
    check(np.zeros(0, np.int64), np.zeros(0, np.float32))         # nothing
    check(rng.permutation(quarter), rng.standard_normal(quarter.size))          # not ascending
    twice = np.sort(np.concatenate([quarter[:1000], quarter[:1000], quarter[5000:6000]]))
    check(twice, (rng.integers(-8, 9, size=twice.size) / 8.0))    # repeats add up (exact sums)
    # device indices that start 8 bytes into a 16-byte unit (a view into a larger buffer)
    import ctypes as C
    val = rng.standard_normal(quarter.size).astype(np.float32)
    shifted = api.DeviceArray.from_host(np.concatenate([[0], quarter]).astype(np.int64))
    d_val = api.DeviceArray.from_host(val)
    out = api.DeviceArray(n, np.float32)
    rc = api.lib().krk_coo_to_dense(C.c_void_p(shifted.ptr + 8), C.c_void_p(d_val.ptr), quarter.size,
                                    C.c_void_p(out.ptr), n, api.DEVICE_PTRS)
    assert rc == 0
    want = np.zeros(n, np.float32)
    want[quarter] = val
    assert np.array_equal(out.to_host(), want)


def test_dense_push_coo_large(api, oracle):
    n = (1 << 22) + 77
    rng = np.random.default_rng(4)
    w0 = rng.standard_normal(n).astype(np.float32)
    t, r = api.DenseTable(w0), oracle.DenseTable(w0)
    from util import make_optims
    o_ref, o_gpu = make_optims(oracle, api, 1, {})
    for step in range(3):
        idx = np.sort(rng.choice(n, size=n // 5, replace=False)).astype(np.int64)
        if step == 2:
            idx = rng.permutation(idx)                            # the scatter path
        val = (rng.integers(-64, 65, size=idx.size) / 1024.0).astype(np.float32)
        assert t.PushCoo(o_gpu, idx, val, 0.01) == 0 and r.push_coo(o_ref, idx, val, 0.01) == 0
        assert_close(t.Pull()[1], r.pull(), "step %d" % step)
    # an entry outside [0, n) is skipped, the others are applied
    bad = np.array([0, n], np.int64)
    one = np.ones(2, np.float32)
    assert t.PushCoo(o_gpu, bad, one, 0.01) == 0 and r.push_coo(o_ref, bad[:1], one[:1], 0.01) == 0
    assert_close(t.Pull()[1], r.pull(), "after an out-of-range entry")


_GROUP_CASES = [c for c in OPTIM_CASES if c[0] in ("sgd_mom", "adagrad_wd", "adam", "adam_amsgrad", "rmsprop_all")]


@pytest.mark.parametrize("name,type_,conf", _GROUP_CASES, ids=[c[0] for c in _GROUP_CASES])
def test_dense_group_matches_the_per_table_loop(api, oracle, name, type_, conf):
    """Ps::CombinePullDenseTable (ps/ps_op.cc:177-252) and a step's PushDenseTable calls for every
    dense parameter of a model, as one launch each: against the oracle's loop over the tables.
    Member sizes put some members off the 16-byte grid of the concatenated arrays (the scalar
    path), one member is empty, 40 members take two launches, and a member that was updated on its
    own before joining keeps its own Adam step count."""
    rng = np.random.default_rng(type_ + 40)
    sizes = [64, 1, 150_000, 4099, 0, 7, 1024, 333] + [int(x) for x in rng.integers(1, 3000, size=32)]
    w0 = [rng.standard_normal(n).astype(np.float32) for n in sizes]
    tables = [api.DenseTable(w) for w in w0]
    refs = [oracle.DenseTable(w) for w in w0]
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    g = (rng.standard_normal(sizes[2]) * 1e-3).astype(np.float32)
    assert tables[2].Push(o_gpu, g, 0.01) == 0 and refs[2].push(o_ref, g, 0.01) == 0
    grp = api.DenseGroup(tables)
    assert grp.n == sum(sizes)
    for step in range(3):
        grads = (rng.standard_normal(grp.n) * 1e-3).astype(np.float32)
        assert grp.CombinePush(o_gpu, grads, 0.01) == 0
        at = 0
        for r, n in zip(refs, sizes):
            if n:
                assert r.push(o_ref, grads[at:at + n], 0.01) == 0
            at += n
        if step == 1:    # a member's own call in between is ordered with the group's
            g = (rng.standard_normal(sizes[3]) * 1e-3).astype(np.float32)
            assert tables[3].Push(o_gpu, g, 0.01) == 0 and refs[3].push(o_ref, g, 0.01) == 0
    rc, got = grp.CombinePull()
    assert rc == 0
    want = np.concatenate([r.pull() for r in refs])
    assert_close(got, want, name + " combined pull")
    for t, r, n in zip(tables, refs, sizes):
        if n:
            assert np.array_equal(t.Pull()[1], got[sum(sizes[:tables.index(t)]):][:n])
            for st in STATE_OF[type_]:
                ws = r.state(st)
                assert_close(t.state(st), ws if ws is not None else np.zeros(n, np.float32), "%s state %d" % (name, st))
    if type_ == 1:
        assert [t.steps for t in tables if t.n] == [r.steps for r, n in zip(refs, sizes) if n]
        assert tables[2].steps == 4 and tables[3].steps == 4
    # the wrong total is the reference's code 11; device pointers work the same way
    assert grp.CombinePush(o_gpu, np.zeros(grp.n - 1, np.float32), 0.01) == 11
    d_out = api.DeviceArray(grp.n, np.float32)
    assert grp.CombinePull(out=d_out, async_=True)[0] == 0 and grp.sync() == 0
    assert np.array_equal(d_out.to_host(), got)
    grp.close()
    assert tables[0].Pull()[0] == 0       # members work on their own again
