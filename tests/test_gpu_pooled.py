"""Multi-hot fields: Pull / Push fused with jagged sum / mean pooling, through the C ABI.

The oracle side is the reference's path taken literally: SparseTable::Pull of the ids, the
optional `embeddings *= weights`, then jagged::SumForward / MeanForward
(pytorch/jagged_embedding.py:32-52, pytorch/py/jagged_ops.cc); backwards: Mean/SumBackward,
times the weights, Emitter's dedup + sum, SparseTable::Push. The forward is compared bit for
bit (the GPU adds a bag's rows in the same order); the push like every other push test.
"""
import numpy as np
import pytest

from util import OPTIM_CASES, STATE_OF, assert_close, make_optims, splitmix64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def _bags(rng, bags, max_len, space, empty_every=7, pow2=False):
    lengths = rng.integers(1, max_len + 1, size=bags)
    if pow2:
        lengths = 2 ** rng.integers(0, int(np.log2(max_len)) + 1, size=bags)
    lengths[::empty_every] = 0
    off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
    ids = splitmix64(rng.integers(0, space, size=int(off[-1])).astype(np.uint64))
    return ids, off


def _tables(api, oracle, dim, seed):
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": str(seed)})
    return api.SparseTable(dim, gi), oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=seed))


def _oracle_pooled_pull(oracle, ref, ids, off, mode, patch, weights):
    u, inv = oracle.dedup(ids)
    rc, rows = ref.pull(u)
    assert rc == 0
    emb = rows[inv]
    if weights is not None:
        emb = emb * weights[:, None]          # fp32 times fp32, rounded once
    return oracle.jagged_forward(emb, off, mode, patch)


@pytest.mark.parametrize("dim", [8, 16, 32, 128, 6])
@pytest.mark.parametrize("mode", ["sum", "mean"])
@pytest.mark.parametrize("weighted", [False, True])
def test_pooled_pull_matches_pull_then_pool(api, oracle, dim, mode, weighted):
    rng = np.random.default_rng(dim * 7 + weighted)
    t, ref = _tables(api, oracle, dim, seed=dim)
    seen = splitmix64(np.arange(0, 3000, dtype=np.uint64))
    assert t.Pull(seen)[0] == 0 and ref.pull(seen)[0] == 0
    ids, off = _bags(rng, 900, 20, 5000)       # ids 3000..4999 are unseen: inserted by the pull
    w = rng.standard_normal(ids.size).astype(np.float32) if weighted else None
    rc, got = t.PullPooled(ids, off, mode, patch_value=-0.75, weights=w)
    assert rc == 0
    want = _oracle_pooled_pull(oracle, ref, ids, off, mode, -0.75, w)
    assert np.array_equal(got, want)
    assert len(t) == len(ref)
    # the same call again finds every id resident and returns the same bits
    assert np.array_equal(t.PullPooled(ids, off, mode, patch_value=-0.75, weights=w)[1], got)
    # and the inserted rows are the rows a plain Pull returns
    u = np.unique(ids)
    assert np.array_equal(t.Pull(u)[1], ref.pull(u)[1])


def test_pooled_pull_device_arrays_and_edge_shapes(api, oracle):
    rng = np.random.default_rng(3)
    t, ref = _tables(api, oracle, 16, seed=3)
    ids, off = _bags(rng, 4000, 30, 20000)
    d_ids, d_off = api.DeviceArray.from_host(ids), api.DeviceArray.from_host(off)
    rc, d_out = t.PullPooled(d_ids, d_off, "mean", patch_value=2.5)
    assert rc == 0
    assert np.array_equal(d_out.to_host(), _oracle_pooled_pull(oracle, ref, ids, off, "mean", 2.5, None))
    # one bag holding everything, and a field of empty bags only
    one = np.array([0, ids.size], np.int64)
    rc, got = t.PullPooled(ids, one, "sum")
    assert rc == 0 and np.array_equal(got, _oracle_pooled_pull(oracle, ref, ids, one, "sum", 0.0, None))
    rc, got = t.PullPooled(np.zeros(0, np.uint64), np.zeros(6, np.int64), "sum", patch_value=1.25)
    assert rc == 0 and got.shape == (5, 16) and (got == 1.25).all()
    # the same id many times in one bag and across bags
    rep = np.full(1000, ids[0], np.uint64)
    off2 = np.arange(0, 1001, 100, dtype=np.int64)
    rc, got = t.PullPooled(rep, off2, "sum")
    assert rc == 0 and np.array_equal(got, _oracle_pooled_pull(oracle, ref, rep, off2, "sum", 0.0, None))


@pytest.mark.parametrize("dim", [16, 6])
def test_pooled_pulls_while_a_table_is_being_filled(api, oracle, dim):
    """A pooled pull of 8192 positions or more that follows a pull which inserted rows looks its
    positions up without inserting, queues the missing ones and inserts them in a launch of their
    own (rows numbered once per workgroup). Steps whose id space keeps growing (every step brings
    new ids, repeated inside and across bags), then the same request twice: the pooled rows are
    the oracle's bit for bit, and the rows in the table are the rows a plain pull returns."""
    rng = np.random.default_rng(dim)
    t, ref = _tables(api, oracle, dim, seed=40 + dim)
    ids = off = None
    for step in range(6):
        if step < 4:
            ids, off = _bags(rng, 9000, 12, 30_000 * (step + 1))
        assert ids.size >= 32_768
        rc, got = t.PullPooled(ids, off, "mean" if step % 2 else "sum", patch_value=0.5)
        assert rc == 0
        want = _oracle_pooled_pull(oracle, ref, ids, off, "mean" if step % 2 else "sum", 0.5, None)
        assert np.array_equal(got, want), step
        assert len(t) == len(ref)
    u = np.unique(ids)
    assert np.array_equal(t.Pull(u)[1], ref.pull(u)[1])
    gid = t.export()[0]
    assert np.unique(gid).size == gid.size == len(ref)

def test_pooled_argument_errors(api, oracle):
    t, _ = _tables(api, oracle, 16, seed=1)
    ids = np.arange(10, dtype=np.uint64)
    rc, _ = t.PullPooled(ids, np.array([0, 4, 9], np.int64))            # does not end at n
    assert rc == api.E_ARGUMENT
    rc, _ = t.PullPooled(ids, np.array([1, 4, 10], np.int64))           # does not start at 0
    assert rc == api.E_ARGUMENT
    off = np.array([0, 4, 10], np.int64)
    assert t.PullPooled(ids, off)[0] == 0
    _, o_gpu = make_optims(oracle, api, 0, {})
    assert t.PushPooled(o_gpu, ids, off, np.zeros((2, 8), np.float32), 0.1) == api.GRADIENT_UNCOMPATIBLE
    assert t.PushPooled(o_gpu, ids, np.array([0, 4, 9], np.int64), np.zeros((2, 16), np.float32), 0.1) \
        == api.E_ARGUMENT
    other = np.arange(100, 110, dtype=np.uint64)                        # never pulled
    assert t.PushPooled(o_gpu, other, off, np.zeros((2, 16), np.float32), 0.1) == api.SPARSE_ID_NOT_EXIST
    wide, _ = _tables(api, oracle, 512, seed=2)
    assert wide.PullPooled(ids, off)[0] == api.INTERFACE_UNIMPLEMENTED


@pytest.mark.parametrize("case", range(len(OPTIM_CASES)), ids=[c[0] for c in OPTIM_CASES])
@pytest.mark.parametrize("mode,weighted", [("sum", False), ("mean", False), ("mean", True)])
def test_pooled_push_matches_backward_dedup_push(api, oracle, case, mode, weighted):
    _, type_, conf = OPTIM_CASES[case]
    dim = 16
    rng = np.random.default_rng(100 + case)
    t, ref = _tables(api, oracle, dim, seed=case)
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)
    for step in range(3):
        # binary-grid gradients, power-of-two weights and bag lengths: every addend is exact, so
        # the sums do not depend on their order (inexact ratios are covered by
        # test_pooled_push_equals_push_raw_of_the_expanded_gradient)
        ids, off = _bags(rng, 700, 8, 2500, pow2=True)
        bags = off.size - 1
        g = (rng.integers(-64, 65, size=(bags, dim)) / 512.0).astype(np.float32)
        w = (2.0 ** rng.integers(-2, 3, size=ids.size)).astype(np.float32) if weighted else None
        rc, _ = t.PullPooled(ids, off, mode, weights=w)
        assert rc == 0
        ref.pull(oracle.dedup(ids)[0])
        assert t.PushPooled(o_gpu, ids, off, g, 0.05, mode=mode, weights=w) == 0
        vg = oracle.jagged_backward(off, g, mode)
        if w is not None:
            vg = vg * w[:, None]
        u, gs = oracle.dedup_sum(ids, vg)
        assert ref.push(o_ref, u, gs, 0.05) == 0
    for st in STATE_OF[type_]:
        rid, rval, rstate, rsteps = ref.export(state_type=st)
        gid, gval, gstate, gsteps = t.export(state_type=st)
        a, b = np.argsort(rid), np.argsort(gid)
        assert np.array_equal(rid[a], gid[b])
        assert_close(gval[b], rval[a], "weights")
        if rstate is not None and gstate is not None:
            assert_close(gstate[b], rstate[a], "state %d" % st)
        if type_ == 1:
            assert np.array_equal(gsteps[b], rsteps[a])


def test_pooled_push_equals_push_raw_of_the_expanded_gradient(api, oracle):
    """Size-independent property: the pooled push is PushRaw of the per-position gradient the
    worker would have materialised (inexact mean ratios and arbitrary weights included). Two
    tables number their rows differently, so the additions are grouped differently: SGD keeps
    the comparison well conditioned (the update is linear in the summed gradient), and the
    tolerance is that of two fp32 summation orders, far below one wrong ratio or weight."""
    dim, n_bags = 32, 60000
    rng = np.random.default_rng(8)
    ids, off = _bags(rng, n_bags, 20, 200000)
    g = (rng.standard_normal((n_bags, dim)) * 1e-2).astype(np.float32)
    w = rng.standard_normal(ids.size).astype(np.float32)
    u = np.unique(ids)
    for mode, weights in (("sum", None), ("mean", None), ("sum", w), ("mean", w)):
        a, _ = _tables(api, oracle, dim, seed=5)
        b, _ = _tables(api, oracle, dim, seed=5)
        assert a.Pull(u)[0] == 0 and b.Pull(u)[0] == 0
        before = a.Pull(u)[1]
        _, o_gpu = make_optims(oracle, api, 3, {})
        for _ in range(2):
            assert a.PushPooled(o_gpu, ids, off, g, 0.5, mode=mode, weights=weights) == 0
            vg = oracle.jagged_backward(off, g, mode)
            if weights is not None:
                vg = vg * weights[:, None]
            assert b.PushRaw(o_gpu, ids, vg, 0.5) == 0
        wa, wb = a.Pull(u)[1], b.Pull(u)[1]
        moved = np.abs(wb - before).max()
        assert moved > 1e-3                                   # the pushes did something
        assert np.abs(wa - wb).max() <= 1e-6 * max(1.0, moved * 10), (mode, weights is not None)
