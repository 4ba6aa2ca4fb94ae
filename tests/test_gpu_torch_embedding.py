"""The worker-side embedding modules (kraken/pytorch/embedding.py, jagged_embedding.py) on GPU
tensors: forward values and the rows after backward agree with the oracle fed with the very
gradient torch's autograd produced."""
import numpy as np
import pytest

from util import assert_close, make_optims

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def mods():
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    from kraken_amd import api, torch_embedding
    api.lib()
    return api, torch_embedding


def _init(api, oracle, seed):
    return (api.Initializer.create(api.InitializerType.kNormal, {"stddev": "0.01", "seed": str(seed)}),
            oracle.init(oracle.INIT_NORMAL, 0.0, 0.01, seed=seed))


def test_embedding_forward_backward(mods, oracle):
    api, te = mods
    dim = 16
    gi, oi = _init(api, oracle, 3)
    o_ref, o_gpu = make_optims(oracle, api, 0, {})
    emb = te.Embedding(dim, initializer=gi, optim=o_gpu, lr=0.05)
    head = torch.nn.Linear(dim, 1, bias=False).cuda()
    ref = oracle.SparseTable(dim, oi)
    g = torch.Generator(device="cpu").manual_seed(0)
    for step in range(3):
        idx = torch.randint(0, 500, (64, 7), generator=g).cuda()        # a batch of 7 fields, with repeats
        out = emb(idx)
        ids = idx.cpu().numpy().astype(np.uint64).ravel()
        u, inv = oracle.dedup(ids)
        rc, rows = ref.pull(u)
        assert_close(out.detach().cpu().numpy().reshape(-1, dim), rows[inv], "forward %d" % step, rtol=1e-6)
        out.retain_grad()
        loss = head(out).square().sum()
        loss.backward()
        grad = out.grad.detach().cpu().numpy().reshape(-1, dim)
        assert np.abs(grad).sum() > 0
        u2, gs = oracle.dedup_sum(ids, grad)
        assert ref.push(o_ref, u2, gs, 0.05) == 0
        assert emb.sparse_table.grad is None                            # the rows are not in the Parameter
    torch.cuda.synchronize()
    t = emb.sparse_table.table()
    rid, rval, _, _ = ref.export()
    assert len(t) == len(ref)
    # sums of fp32 gradients in two orders: compared at the tolerance of the values they move
    assert_close(t.Pull(rid)[1], rval, "rows after three steps", rtol=1e-4, atol=1e-6)


def test_embedding_used_twice_before_backward(mods, oracle):
    """The module's pull leaves the row of every index behind for its backward's push. Two
    forwards on one table before either backward: the second pull's notes replace the first's,
    and the first backward (another index tensor) must look its ids up again; both updates land
    on the right rows."""
    api, te = mods
    dim = 16
    gi, oi = _init(api, oracle, 5)
    o_ref, o_gpu = make_optims(oracle, api, 0, {})                      # plain SGD: updates commute
    emb = te.Embedding(dim, initializer=gi, optim=o_gpu, lr=0.1)
    ref = oracle.SparseTable(dim, oi)
    g = torch.Generator(device="cpu").manual_seed(4)
    a = torch.randint(0, 300, (512,), generator=g).cuda()
    b = torch.randint(200, 600, (640,), generator=g).cuda()
    out_a, out_b = emb(a), emb(b)
    wa = torch.linspace(-1.0, 1.0, dim).cuda()
    (out_a * wa).sum().backward()
    (out_b * (2.0 * wa)).sum().backward()
    torch.cuda.synchronize()
    for idx, scale in ((a, 1.0), (b, 2.0)):
        ids = idx.cpu().numpy().astype(np.uint64)
        ref.pull(np.unique(ids))
    for idx, scale in ((a, 1.0), (b, 2.0)):
        ids = idx.cpu().numpy().astype(np.uint64)
        grad = np.tile((scale * wa.cpu().numpy()).astype(np.float32), (ids.size, 1))
        u, gs = oracle.dedup_sum(ids, grad)
        assert ref.push(o_ref, u, gs, 0.1) == 0
    rid, rval, _, _ = ref.export()
    t = emb.sparse_table.table()
    assert len(t) == len(ref)
    assert_close(t.Pull(rid)[1], rval, "rows after two interleaved uses", rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("mode", ["sum", "mean"])
@pytest.mark.parametrize("weighted", [False, True])
def test_jagged_embedding_forward_backward(mods, oracle, mode, weighted):
    api, te = mods
    dim = 8
    gi, oi = _init(api, oracle, 9)
    o_ref, o_gpu = make_optims(oracle, api, 3, {})                      # plain SGD: linear in the summed gradient
    emb = te.JaggedEmbedding(dim, initializer=gi, optim=o_gpu, lr=0.5, mode=mode, patch_value=0.25)
    ref = oracle.SparseTable(dim, oi)
    rng = np.random.default_rng(1)
    for step in range(2):
        lengths = rng.integers(0, 6, size=200)
        off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
        ids = rng.integers(0, 300, size=int(off[-1])).astype(np.uint64)
        w = (2.0 ** rng.integers(-1, 2, size=ids.size)).astype(np.float32) if weighted else None
        out = emb(torch.from_numpy(ids.astype(np.int64)).cuda(), torch.from_numpy(off).cuda(),
                  torch.from_numpy(w).cuda() if weighted else None)
        u, inv = oracle.dedup(ids)
        rows = ref.pull(u)[1][inv]
        if weighted:
            rows = rows * w[:, None]
        want = oracle.jagged_forward(rows, off, mode, 0.25)
        if step == 0 or mode == "sum":
            # the bag is added up in the reference's order: identical bits (after a mean step
            # the rows themselves carry sums of inexact addends and agree to rounding only)
            assert np.array_equal(out.detach().cpu().numpy(), want)
        else:
            assert_close(out.detach().cpu().numpy(), want, "pooled forward", rtol=1e-5, atol=1e-6)
        coef = (rng.integers(-8, 9, size=(lengths.size, dim)) / 16.0).astype(np.float32)
        (out * torch.from_numpy(coef).cuda()).sum().backward()
        vg = oracle.jagged_backward(off, coef, mode)
        if weighted:
            vg = vg * w[:, None]
        u2, gs = oracle.dedup_sum(ids, vg)
        assert ref.push(o_ref, u2, gs, 0.5) == 0
    torch.cuda.synchronize()
    rid, rval, _, _ = ref.export()
    assert_close(emb.sparse_table.table().Pull(rid)[1], rval, "rows after two steps", rtol=1e-5, atol=1e-6)


def test_rejects_host_tensors(mods):
    api, te = mods
    emb = te.Embedding(4)
    with pytest.raises(TypeError):
        emb(torch.zeros(3, dtype=torch.int64))
    with pytest.raises(TypeError):
        emb(torch.zeros(3, dtype=torch.int32).cuda())


def test_combine_embedding_forward_backward(mods, oracle):
    """pytorch/combine_embedding.py: tables of two widths in one request, ids repeated within a
    table and shared between tables, one output left out of the loss."""
    api, te = mods
    dims = [8, 16, 8, 8]
    seeds = [5, 6, 7, 8]
    inits = [_init(api, oracle, s) for s in seeds]
    o_ref, o_gpu = make_optims(oracle, api, 3, {})                      # plain SGD
    emb = te.CombineEmbedding(dims, initializers=[g for g, _ in inits], optim=o_gpu, lr=0.5)
    refs = [oracle.SparseTable(d, oi) for d, (_, oi) in zip(dims, inits)]
    g = torch.Generator(device="cpu").manual_seed(2)
    for step in range(3):
        idx = [torch.randint(0, 200, shape, generator=g).cuda() for shape in ((32, 3), (50,), (7, 2, 2), (64,))]
        outs = emb(idx)
        assert [tuple(o.shape) for o in outs] == [(32, 3, 8), (50, 16), (7, 2, 2, 8), (64, 8)]
        coefs = []
        loss = 0.0
        for k, (o, r, i, d) in enumerate(zip(outs, refs, idx, dims)):
            ids = i.cpu().numpy().astype(np.uint64).ravel()
            u, inv = oracle.dedup(ids)
            assert np.array_equal(o.detach().cpu().numpy().reshape(-1, d), r.pull(u)[1][inv])
            c = (torch.randint(-8, 9, o.shape, generator=g) / 16.0).cuda()
            coefs.append(c)
            if k != 3:                                                   # table 3 gets no gradient
                loss = loss + (o * c).sum()
        loss.backward()
        for k, (r, i, d, c) in enumerate(zip(refs, idx, dims, coefs)):
            ids = i.cpu().numpy().astype(np.uint64).ravel()
            grad = c.cpu().numpy().reshape(-1, d) if k != 3 else np.zeros((ids.size, d), np.float32)
            u, gs = oracle.dedup_sum(ids, grad)
            assert r.push(o_ref, u, gs, 0.5) == 0
    torch.cuda.synchronize()
    for t, r in zip(emb.combine_sparse_table.tables(), refs):
        rid, rval, _, _ = r.export()
        assert len(t) == len(r)
        assert np.array_equal(t.Pull(rid)[1], rval)                     # dyadic gradients, SGD: exact


def test_jagged_tensor(mods, oracle):
    """test/pytorch/jagged_tensor_test.py: values and offsets of from_list_tensors, also for
    pieces of more than one dimension; then the module called with a JaggedTensor."""
    api, te = mods
    g = torch.Generator(device="cpu").manual_seed(0)
    for tail in ((), (2, 3)):
        pieces = [torch.rand((int(n),) + tail, generator=g) for n in torch.randint(1, 11, (5,), generator=g)]
        jt = te.JaggedTensor.from_list_tensors(pieces)
        assert torch.equal(jt.values(), torch.cat(pieces, 0))
        want, at = [0], 0
        for p in pieces:
            at += p.shape[0]
            want.append(at)
        assert jt.offsets().tolist() == want and jt.weights() is None
    with pytest.raises(ValueError):
        te.JaggedTensor(torch.zeros(5), torch.tensor([0, 3, 2, 5]))
    with pytest.raises(ValueError):
        te.JaggedTensor(torch.zeros(5), torch.tensor([0, 6]))
    with pytest.raises(ValueError):
        te.JaggedTensor.from_list_tensors([torch.zeros(2, 3), torch.zeros(2, 4)])
    bags = [torch.randint(0, 50, (int(n),), generator=g) for n in (3, 0, 5, 1)]
    jt = te.JaggedTensor.from_list_tensors(bags).to("cuda")
    gi, oi = _init(api, oracle, 4)
    emb = te.JaggedEmbedding(8, initializer=gi, mode="sum", patch_value=0.5)
    out = emb(jt)
    ref = oracle.SparseTable(8, oi)
    ids = torch.cat(bags).numpy().astype(np.uint64)
    u, inv = oracle.dedup(ids)
    want = oracle.jagged_forward(ref.pull(u)[1][inv], np.array([0, 3, 3, 8, 9], np.int64), "sum", 0.5)
    assert np.array_equal(out.detach().cpu().numpy(), want)


def test_combine_jagged_embedding(mods, oracle):
    """pytorch/combine_jagged_embedding.py: a JaggedTensor per table, each table with its own
    mode and patch value; forward and the rows after backward against the oracle."""
    api, te = mods
    dims, modes, patches = [8, 8, 4], ["sum", "mean", "sum"], [0.0, 0.25, -1.0]
    inits = [_init(api, oracle, 20 + i) for i in range(3)]
    o_ref, o_gpu = make_optims(oracle, api, 3, {})
    emb = te.CombineJaggedEmbedding(dims, initializers=[g for g, _ in inits], modes=modes, patch_values=patches,
                                    optim=o_gpu, lr=0.5)
    refs = [oracle.SparseTable(d, oi) for d, (_, oi) in zip(dims, inits)]
    rng = np.random.default_rng(3)
    for step in range(2):
        batch, inputs = [], []
        for i in range(3):
            lengths = rng.choice([0, 1, 2, 4], size=120)
            off = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int64)
            ids = rng.integers(0, 200, size=int(off[-1])).astype(np.uint64)
            w = (2.0 ** rng.integers(-1, 2, size=ids.size)).astype(np.float32) if i == 2 else None
            batch.append((off, ids, w))
            inputs.append(te.JaggedTensor(torch.from_numpy(ids.astype(np.int64)).cuda(), torch.from_numpy(off).cuda(),
                                          torch.from_numpy(w).cuda() if w is not None else None))
        outs = emb(inputs)
        assert len(outs) == 3
        loss, coefs = 0, []
        for i, (off, ids, w) in enumerate(batch):
            u, inv = oracle.dedup(ids)
            rows = refs[i].pull(u)[1][inv]
            if w is not None:
                rows = rows * w[:, None]
            want = oracle.jagged_forward(rows, off, modes[i], patches[i])
            assert outs[i].shape == (off.size - 1, dims[i])
            assert_close(outs[i].detach().cpu().numpy(), want, "pooled forward of table %d" % i, rtol=1e-5, atol=1e-6)
            coef = (rng.integers(-8, 9, size=(off.size - 1, dims[i])) / 16.0).astype(np.float32)
            coefs.append(coef)
            if i != 1 or step == 0:                 # table 1's output stays out of the second loss
                loss = loss + (outs[i] * torch.from_numpy(coef).cuda()).sum()
        loss.backward()
        for i, (off, ids, w) in enumerate(batch):
            if i == 1 and step == 1:
                continue
            vg = oracle.jagged_backward(off, coefs[i], modes[i])
            if w is not None:
                vg = vg * w[:, None]
            u2, gs = oracle.dedup_sum(ids, vg)
            assert refs[i].push(o_ref, u2, gs, 0.5) == 0
    torch.cuda.synchronize()
    for i in range(3):
        rid, rval, _, _ = refs[i].export()
        assert_close(emb.combine_sparse_table.tables()[i].Pull(rid)[1], rval, "rows of table %d" % i,
                     rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        te.CombineJaggedEmbedding([4], modes=["max"])


def test_modules_take_the_reference_descriptions(mods, oracle):
    """Initializers and optimizers given as the reference's Python classes
    (pytorch/initializer.py, pytorch/optim.py) reach the engine with the same meaning."""
    api, te = mods

    class Described:       # what kraken.pytorch.initializer / optim objects answer
        def __init__(self, type_, conf):
            self.type, self.conf = (lambda: type_), (lambda: conf)
    dim = 4
    emb = te.Embedding(dim, initializer=Described(0, {"value": "0.5"}),        # ConstantInitializer(0.5)
                       optim=Described(0, {"eps": "1e-06"}), lr=0.25)          # Adagrad(eps=1e-6)
    ref = oracle.SparseTable(dim, oracle.init(oracle.INIT_CONSTANT, 0.5, 0.0))
    o_ref, _ = make_optims(oracle, api, 0, {"eps": 1e-6})
    ids = np.array([5, 9, 5, 2], np.uint64)
    out = emb(torch.from_numpy(ids.astype(np.int64)).cuda())
    assert np.array_equal(out.detach().cpu().numpy(), np.full((4, dim), 0.5, np.float32))
    coef = np.arange(16, dtype=np.float32).reshape(4, dim) / 8
    (out * torch.from_numpy(coef).cuda()).sum().backward()
    torch.cuda.synchronize()
    u, inv = oracle.dedup(ids)
    assert np.array_equal(ref.pull(u)[1], np.full((3, dim), 0.5, np.float32))
    u2, gs = oracle.dedup_sum(ids, coef)
    assert ref.push(o_ref, u2, gs, 0.25) == 0
    rid, rval, _, _ = ref.export()
    assert_close(emb.sparse_table.table().Pull(rid)[1], rval, "rows after an Adagrad step", rtol=1e-5, atol=1e-6)


def _ordered_with_torch(api, te, oracle, seed):
    """The pull must see indices that torch's stream produces behind a long kernel, and torch's
    next kernel must see the rows the pull wrote: both only hold when the table's launches are
    enqueued on the very stream torch is using."""
    dim = 16
    gi, oi = _init(api, oracle, seed)
    o_ref, o_gpu = make_optims(oracle, api, 0, {})
    emb = te.Embedding(dim, initializer=gi, optim=o_gpu, lr=0.05)
    ref = oracle.SparseTable(dim, oi)
    g = torch.Generator(device="cpu").manual_seed(seed)
    a = torch.randn(4096, 4096, device="cuda")
    for step in range(3):
        want = torch.randint(0, 5000, (4096,), generator=g)
        staged = want.cuda()
        idx = torch.full((4096,), 10**9 + step, dtype=torch.int64, device="cuda")   # stale ids
        torch.cuda.synchronize()
        b = a
        for _ in range(6):                       # some milliseconds of work ahead of the copy
            b = b @ a
            b = b / b.abs().max()
        idx.copy_(staged)                        # the real ids arrive behind it, on torch's stream
        out = emb(idx)
        total = out.sum(dim=0)                   # torch reads the rows right behind the pull
        out.backward(torch.ones_like(out) * 0.01)
        ids = want.numpy().astype(np.uint64)
        u, inv = oracle.dedup(ids)
        rc, rows = ref.pull(u)
        assert_close(out.detach().cpu().numpy(), rows[inv], "ordered pull %d" % step, rtol=1e-6)
        assert_close(total.detach().cpu().numpy(), rows[inv].astype(np.float64).sum(axis=0).astype(np.float32),
                     "torch op behind the pull %d" % step, rtol=1e-4, atol=1e-6)
        u2, gs = oracle.dedup_sum(ids, np.full((ids.size, dim), 0.01, np.float32))
        assert ref.push(o_ref, u2, gs, 0.05) == 0
    torch.cuda.synchronize()
    rid, rval, _, _ = ref.export()
    t = emb.sparse_table.table()
    assert len(t) == len(ref)                    # no stale id was ever inserted
    assert_close(t.Pull(rid)[1], rval, "rows after ordered steps", rtol=1e-4, atol=1e-6)


def test_embedding_is_ordered_on_torchs_default_stream(mods, oracle):
    api, te = mods
    assert torch.cuda.current_stream().cuda_stream == 0      # the handle a NULL stream stands for
    _ordered_with_torch(api, te, oracle, 21)


def test_embedding_is_ordered_on_a_side_stream(mods, oracle):
    api, te = mods
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        _ordered_with_torch(api, te, oracle, 22)
    side.synchronize()
