"""The operations Ps performs on a sparse table through SparseTable::mutable_vals():
fetch without insert (ps/ps.cc:914-935), erase after a cluster change (ps/ps.cc:92-109),
and moving whole Values (weights + optimizer state + step counter) from one table into
another (transfer ps/ps.cc:289-321 / 789-792, checkpoint load checkpoint/checkpoint.cc:620-645).
"""
import ctypes as C

import numpy as np
import pytest

from util import OPTIM_CASES, STATE_OF, assert_close, make_optims, splitmix64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from kraken_amd import api as a
    a.lib()
    return a


def _tables(api, oracle, dim, seed):
    gi = api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": str(seed)})
    return api.SparseTable(dim, gi), oracle.SparseTable(dim, oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=seed))


def _same_tables(t, ref, what=""):
    gid, gval, _, _ = t.export()
    rid, rval, _, _ = ref.export()
    a, b = np.argsort(gid), np.argsort(rid)
    assert np.array_equal(gid[a], rid[b]), what
    assert_close(gval[a], rval[b], what)


@pytest.mark.parametrize("dim", [16, 6, 128])
def test_fetch_returns_existing_rows_and_inserts_nothing(api, oracle, dim):
    rng = np.random.default_rng(dim)
    t, ref = _tables(api, oracle, dim, seed=dim)
    ids = splitmix64(np.arange(5000, dtype=np.uint64))
    assert t.Pull(ids)[0] == 0 and ref.pull(ids)[0] == 0
    o_ref, o_gpu = make_optims(oracle, api, 1, {})
    g = (rng.integers(-64, 65, size=(2000, dim)) / 4096.0).astype(np.float32)
    assert t.Push(o_gpu, ids[:2000], g, 1e-3) == 0 and ref.push(o_ref, ids[:2000], g, 1e-3) == 0
    probe = np.concatenate([ids[::3], splitmix64(np.arange(10**6, 10**6 + 700, dtype=np.uint64)),
                            np.array([2**64 - 1], np.uint64)])
    rng.shuffle(probe)
    found, vals, st, steps = t.fetch(probe, state_type=api.StateType.kFirstMoment)
    rfound, rvals = ref.fetch(probe)
    assert np.array_equal(found, rfound)
    assert_close(vals, rvals, "fetched weights")
    assert (vals[~found] == 0).all() and (st[~found] == 0).all() and (steps[~found] == 0).all()
    pushed = np.isin(probe, ids[:2000])
    assert np.array_equal(steps, pushed.astype(np.int64))          # one Adam step on the pushed rows
    assert (np.abs(st[pushed]).sum(axis=1) > 0).all() and (st[~pushed] == 0).all()
    assert len(t) == len(ref) == 5000
    # the all-ones id, once present, is fetched like any other
    assert t.Pull(np.array([2**64 - 1], np.uint64))[0] == 0
    assert t.fetch(np.array([2**64 - 1, 12345], np.uint64))[0].tolist() == [True, False]


def test_erase_matches_the_reference_walk(api, oracle):
    rng = np.random.default_rng(1)
    dim = 16
    t, ref = _tables(api, oracle, dim, seed=1)
    ids = splitmix64(np.arange(20000, dtype=np.uint64))
    ids[77] = np.uint64(2**64 - 1)
    assert t.Pull(ids)[0] == 0 and ref.pull(ids)[0] == 0
    o_ref, o_gpu = make_optims(oracle, api, 0, {})
    for round_ in range(4):
        live = ref.export()[0]
        g = (rng.integers(-64, 65, size=(live.size, dim)) / 4096.0).astype(np.float32)
        assert t.Push(o_gpu, live, g, 0.05) == 0 and ref.push(o_ref, live, g, 0.05) == 0
        # what a node keeps after a cluster change: here, a pseudo-random 70 % of its rows
        goes = live[(oracle_hash(oracle, live) % np.uint64(10)) < np.uint64(3 + round_)]
        drop = np.concatenate([goes, goes[:50], splitmix64(np.arange(10**7, 10**7 + 300, dtype=np.uint64))])
        assert t.erase(drop) == ref.erase(drop) == goes.size
        assert len(t) == len(ref)
        _same_tables(t, ref, "after erase %d" % round_)
        found, _, _, _ = t.fetch(drop)
        assert not found.any()
        assert (t.lookup(ref.export()[0]) >= 0).all()
        assert sorted(t.lookup(ref.export()[0]).tolist()) == list(range(len(ref)))   # rows stay dense
        # erased ids come back as new rows with fresh values and no optimizer history
        back = goes[: goes.size // 2]
        rc, rows = t.Pull(back)
        rc2, want = ref.pull(back)
        assert rc == 0 and rc2 == 0
        assert_close(rows, want, "re-inserted rows", rtol=1e-6)
        _, _, state, steps = t.fetch(back, state_type=api.StateType.kStateSum)
        assert (state == 0).all() and (steps == 0).all()
    # optimizer state of the survivors is intact
    _, _, gs, _ = t.export(state_type=api.StateType.kStateSum)
    _, _, rs, _ = ref.export(state_type=oracle.ST_STATE_SUM)
    assert_close(gs[np.argsort(t.export()[0])], rs[np.argsort(ref.export()[0])], "state_sum")
    assert t.erase(ref.export()[0]) == len(ref)          # everything
    assert len(t) == 0 and t.Pull(ids[:10])[0] == 0 and len(t) == 10


def oracle_hash(oracle, ids):
    return np.array([oracle.lib().kro_hash64(int(k)) for k in ids], dtype=np.uint64)


@pytest.mark.parametrize("name,type_,conf", [c for c in OPTIM_CASES if c[0] in (
    "sgd_mom", "sgd_damp", "adagrad", "adam", "adam_amsgrad", "rmsprop_all")])
def test_values_move_between_tables_with_their_state(api, oracle, name, type_, conf):
    """Transfer / checkpoint load: rows fetched from one table and brought into another carry on
    exactly as if they had never moved (compared with an oracle table that never moved)."""
    rng = np.random.default_rng(3)
    dim = 16
    src, ref = _tables(api, oracle, dim, seed=2)
    dst, _ = _tables(api, oracle, dim, seed=99)            # another initializer: values must travel
    ids = splitmix64(np.arange(3000, dtype=np.uint64))
    assert src.Pull(ids)[0] == 0 and ref.pull(ids)[0] == 0
    o_ref, o_gpu = make_optims(oracle, api, type_, conf)

    def push(table, which):
        g = (np.random.default_rng(which).integers(-64, 65, size=(ids.size, dim)) / 4096.0).astype(np.float32)
        return table.Push(o_gpu, ids, g, 0.01) if table is not ref else table.push(o_ref, ids, g, 0.01)

    for step in range(2):
        assert push(src, step) == 0 and push(ref, step) == 0
    moved = ids[::2]
    found, vals, _, steps = src.fetch(moved)
    assert found.all()
    dst.load(moved, vals)
    for st in STATE_OF[type_]:
        _, _, state, _ = src.fetch(moved, state_type=st)
        assert dst.load_state(moved, state_type=st, state=state) == 0
    assert dst.load_state(moved, steps=steps) == 0
    assert dst.load_state(np.array([424242], np.uint64), steps=np.array([1])) == api.SPARSE_ID_NOT_EXIST
    assert src.erase(moved) == moved.size
    # both halves keep training; together they must equal the table that never moved
    rest = ids[1::2]
    for step in range(2, 4):
        g = (np.random.default_rng(step).integers(-64, 65, size=(ids.size, dim)) / 4096.0).astype(np.float32)
        assert dst.Push(o_gpu, moved, g[::2], 0.01) == 0
        assert src.Push(o_gpu, rest, g[1::2], 0.01) == 0
        assert ref.push(o_ref, ids, g, 0.01) == 0
    rc, want = ref.pull(ids)
    assert_close(dst.Pull(moved)[1], want[::2], name + " moved half")
    assert_close(src.Pull(rest)[1], want[1::2], name + " staying half")


def test_select_routed_follows_the_references_ring(api, oracle):
    """The clean-up (ps/ps.cc:92-109) and the transfer-out walk (ps/ps.cc:289-321) decide by
    Router::Hit(utils::Hash(table_id, sparse_id)). Rings built by the reference's own router
    (tests/golden/ref_router.json); the owner of every row by the oracle, itself pinned on the
    same file."""
    import json
    import os
    cases = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "ref_router.json")))
    dim = 4
    for case in cases:
        ring = [(int(h), int(n)) for h, n in case["ring"]]
        table_id = case["table_id"]
        t, _ = _tables(api, oracle, dim, seed=3)
        # the ids the reference answered for, and many more
        ids = np.concatenate([np.array([int(i) for i, _ in case["ids"]], np.uint64),
                              splitmix64(np.arange(1000, 41000, dtype=np.uint64))])
        ids = ids[np.sort(np.unique(ids, return_index=True)[1])]
        assert t.Pull(ids)[0] == 0
        golden = {int(i): int(o) for i, o in case["ids"]}
        for i, o in zip(ids[:len(golden)].tolist(), oracle.route_owners(ring, table_id, ids[:len(golden)]).tolist()):
            assert golden[i] == o
        ids = t.export()[0]                                   # row order: what a selection follows
        owners = oracle.route_owners(ring, table_id, ids)
        nodes = sorted(set(n for _, n in ring))
        total = 0
        for node in nodes + [max(nodes) + 1]:                 # the last one owns nothing
            mine = t.select_routed(table_id, ring, node, owned=True)
            assert np.array_equal(mine, ids[owners == node])  # row order
            others = t.select_routed(table_id, ring, node, owned=False)
            assert np.array_equal(others, ids[owners != node])
            total += mine.size
        assert total == ids.size
        # another table id routes the same ids differently
        if len(nodes) > 1:
            assert not np.array_equal(oracle.route_owners(ring, table_id + 1, ids), owners)
            assert np.array_equal(t.select_routed(table_id + 1, ring, nodes[0]),
                                  ids[oracle.route_owners(ring, table_id + 1, ids) == nodes[0]])
        # the clean-up itself: drop what belongs to the others, keep the rest
        keep = ids[owners == nodes[0]]
        gone = t.erase(t.select_routed(table_id, ring, nodes[0], owned=False))
        assert gone == ids.size - keep.size and len(t) == keep.size
        assert np.array_equal(np.sort(t.export()[0]), np.sort(keep))
        assert t.select_routed(table_id, ring, nodes[0], owned=False).size == 0
    # an empty ring owns nothing; an empty table selects nothing; an unsorted ring is refused
    t, _ = _tables(api, oracle, dim, seed=4)
    assert t.select_routed(1, [(5, 0)], 0).size == 0
    assert t.Pull(np.arange(10, dtype=np.uint64))[0] == 0
    assert t.select_routed(1, [], 0).size == 0 and t.select_routed(1, [], 0, owned=False).size == 10
    assert t.select_routed(1, [(5, 0)], 0).size == 10          # one virtual node owns the whole ring
    with pytest.raises(api.KrakenHipError):
        t.select_routed(1, [(9, 0), (5, 1)], 0)


def test_route_ids_partitions_a_request_like_the_worker(api, oracle):
    """Emitter::PullSparseTableImpl (worker/emitter.cc:139-149) sends every distinct id to
    router_.Hit(utils::Hash(table_id, sparse_id)) and lists each server's ids in the order it met
    them. Owners against every id the reference's own router answered for
    (tests/golden/ref_router.json) and, for a million more, against the oracle (pinned on the same
    file); the grouping against a plain stable partition."""
    import json
    import os
    cases = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "ref_router.json")))
    for ci, case in enumerate(cases):
        ring = [(int(h), int(n)) for h, n in case["ring"]]
        table_id = int(case["table_id"])
        golden_ids = np.array([int(i) for i, _ in case["ids"]], np.uint64)
        golden_owner = np.array([int(o) for _, o in case["ids"]], np.uint64)
        node_ids, counts, owner, perm = api.route_ids(table_id, ring, golden_ids)
        assert np.array_equal(owner, golden_owner)
        assert node_ids.tolist() == sorted(set(n for _, n in ring))
        n_more = 1_000_000 if ci == 0 else 50_000
        ids = np.concatenate([golden_ids, splitmix64(np.arange(7, 7 + n_more, dtype=np.uint64))])
        want_owner = oracle.route_owners(ring, table_id, ids)
        # host pointers and device pointers give the same answer
        node_ids, counts, owner, perm = api.route_ids(table_id, ring, ids)
        d_nodes, d_counts, d_owner, d_perm = api.route_ids(table_id, ring, api.DeviceArray.from_host(ids))
        assert np.array_equal(owner, want_owner) and np.array_equal(d_owner.to_host()[:ids.size], want_owner)
        rank = np.searchsorted(node_ids, want_owner)
        want_perm = np.argsort(rank, kind="stable")
        assert np.array_equal(perm, want_perm) and np.array_equal(d_perm.to_host()[:ids.size], want_perm)
        assert counts.tolist() == np.bincount(rank, minlength=node_ids.size).tolist() == d_counts.tolist()
        assert counts.sum() == ids.size
    # the library keeps the last ring on the device: a ring of the same hashes whose virtual nodes
    # changed hands, then the first one again, must each be answered for themselves
    ring = [(int(h), int(n)) for h, n in cases[0]["ring"]]
    nodes = sorted(set(n for _, n in ring))
    if len(nodes) > 1:
        moved = [(h, nodes[(nodes.index(n) + 1) % len(nodes)]) for h, n in ring]
        ids = splitmix64(np.arange(99, 99 + 30_000, dtype=np.uint64))
        for r in (ring, moved, moved, ring):
            node_ids, counts, owner, perm = api.route_ids(5, r, ids)
            want_owner = oracle.route_owners(r, 5, ids)
            assert np.array_equal(owner, want_owner)
            assert counts.tolist() == np.bincount(np.searchsorted(node_ids, want_owner),
                                                  minlength=node_ids.size).tolist()
        assert not np.array_equal(oracle.route_owners(ring, 5, ids), oracle.route_owners(moved, 5, ids))
    # errors: an unsorted ring, too little room for the nodes, an empty ring with ids to route
    with pytest.raises(api.KrakenHipError):
        api.route_ids(1, [(9, 0), (5, 1)], np.arange(4, dtype=np.uint64))
    with pytest.raises(api.KrakenHipError):
        api.route_ids(1, [], np.arange(4, dtype=np.uint64))
    node_ids, counts, owner, perm = api.route_ids(1, ring, np.zeros(0, np.uint64))
    assert counts.tolist() == [0] * node_ids.size and perm.size == 0
    m = C.c_int64()
    rh = np.array([h for h, _ in ring], np.uint64)
    rn = np.array([n for _, n in ring], np.uint64)
    one = np.zeros(1, np.uint64)
    rc = api.lib().krk_route_ids(1, api._ptr(rh), api._ptr(rn), len(ring), api._ptr(one), 1, None,
                                 api._ptr(np.zeros(1, np.int64)), api._ptr(one), api._ptr(np.zeros(1, np.int64)), 1,
                                 C.byref(m), 0)
    assert rc == api.E_CAPACITY and m.value == len(set(n for _, n in ring))
