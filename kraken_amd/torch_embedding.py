"""The reference's worker-side embedding modules on GPU tensors.

`kraken/pytorch/embedding.py` and `jagged_embedding.py` wrap an autograd Function around
`kraken_native.pull_sparse_table / push_sparse_table`, which reject device tensors
(pytorch/py/pytorch.cc:42,102,116,188) and send the request to a server. Here the table lives on
the same GPU as the tensors: forward is one pull (or one pooled pull) straight into a torch
tensor, backward is one fused dedup + sum + optimizer step on the gradient torch hands over.
Nothing is copied to the host and nothing is synchronised: the table enqueues its kernels on
torch's current stream.

PyTorch is plumbing here (it owns the tensors and the stream); the arithmetic is the table
engine's. Importing this module needs torch; nothing else in the package does.
"""
import ctypes as C

import torch

from . import api
from .configs import as_initializer, as_optim


def _stream_ptr():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ids_ptr(indices):
    """int64 indices are the uint64 ids bit for bit (worker/emitter.cc:126 casts the same way)."""
    if indices.dtype != torch.int64 or not indices.is_cuda:
        raise TypeError("indices must be an int64 CUDA tensor")
    indices = indices.contiguous()
    return indices, C.c_void_p(indices.data_ptr())


class GpuSparseTable(torch.nn.Parameter):
    """pytorch/sparse_table.py: a Parameter that stands for the table so that autograd calls the
    Function's backward. The rows are not in this tensor but in the engine's table.
    `initializer` and `optim` are the engine's (api.Initializer / api.Optim) or the reference's
    descriptions of them (configs.NormalInitializer(...), configs.Adagrad(...))."""

    def __new__(cls, dimension, initializer=None, optim=None, lr=0.01, capacity_hint=0):
        self = super().__new__(cls, torch.empty(0), requires_grad=True)
        self._dimension = int(dimension)
        self._table = api.SparseTable(dimension, as_initializer(initializer) or api.Initializer.create(
            api.InitializerType.kNormal, {}), capacity_hint=capacity_hint)
        self._optim = as_optim(optim) or api.Optim.create(api.OptimType.kSGD)
        self.lr = float(lr)
        return self

    def dimension(self):
        return self._dimension

    def table(self):
        return self._table

    def _on_current_stream(self):
        api._check(api.lib().krk_sparse_set_stream(self._table.h, _stream_ptr()), "krk_sparse_set_stream")
        return self._table.h


class EmbeddingFunction(torch.autograd.Function):
    """pytorch/embedding.py:9-23"""

    @staticmethod
    def forward(ctx, sparse_table, indices):
        ids, p_ids = _ids_ptr(indices)
        dim = sparse_table.dimension()
        out = torch.empty(tuple(indices.shape) + (dim,), dtype=torch.float32, device=indices.device)
        h = sparse_table._on_current_stream()
        # the table notes where it found every id: backward pushes gradients for this very
        # tensor (autograd keeps it alive and unchanged), so its look-up need not be repeated
        api._check(api.lib().krk_sparse_pull(h, p_ids, ids.numel(), C.c_void_p(out.data_ptr()),
                                             api.DEVICE_PTRS | api.ASYNC | api.NOTE_ROWS), "krk_sparse_pull")
        ctx.table = sparse_table
        ctx.save_for_backward(ids)
        return out

    @staticmethod
    def backward(ctx, grad):
        (ids,) = ctx.saved_tensors
        t = ctx.table
        grad = grad.contiguous().to(torch.float32)
        h = t._on_current_stream()
        api._check(api.lib().krk_sparse_push_raw(h, C.byref(t._optim.raw), C.c_void_p(ids.data_ptr()), ids.numel(),
                                                 C.c_void_p(grad.data_ptr()), t.dimension(), t.lr,
                                                 api.DEVICE_PTRS | api.ASYNC | api.IDS_AS_PULLED),
                   "krk_sparse_push_raw")
        return None, None


class Embedding(torch.nn.Module):
    """pytorch/embedding.py:26-43 with the table on the GPU. The optimizer step of the rows is
    part of backward (the reference applies it on the server when the push arrives)."""

    def __init__(self, dimension, initializer=None, optim=None, lr=0.01, capacity_hint=0):
        super().__init__()
        self.sparse_table = GpuSparseTable(dimension, initializer, optim, lr, capacity_hint)

    def forward(self, indices):
        return EmbeddingFunction.apply(self.sparse_table, indices)


class JaggedTensor:
    """pytorch/jagged_tensor.py: tensors that agree in all but their first dimension, kept as one
    `values` tensor and the `offsets` of the pieces (offsets[0] = 0, offsets[-1] = len(values)),
    with optional per-row `weights`. Offsets that live on the GPU are not read back to be checked
    (that would wait for the device); the pooling kernels clamp them to the values' range."""

    def __init__(self, values, offsets, weights=None):
        if not offsets.is_cuda:
            o = offsets.tolist()
            if not o or o[0] != 0 or o[-1] != values.shape[0] or any(b < a for a, b in zip(o, o[1:])):
                raise ValueError("JaggedTensor's offsets is invalid:%s, values shape:%s" % (o, tuple(values.shape)))
        if weights is not None and weights.shape != values.shape:
            raise ValueError("JaggedTensor need values and weights has same shape but got weights shape:%s, "
                             "values shape:%s." % (tuple(weights.shape), tuple(values.shape)))
        self._values, self._offsets, self._weights = values, offsets, weights

    def values(self):
        return self._values

    def offsets(self):
        return self._offsets

    def weights(self):
        return self._weights

    def to(self, device):
        return JaggedTensor(self._values.to(device), self._offsets.to(device),
                            None if self._weights is None else self._weights.to(device))

    @staticmethod
    def from_list_tensors(list_values, list_weights=None):
        """pytorch/jagged_tensor.py:56-84"""
        assert len(list_values) > 0
        tail = list_values[0].shape[1:]
        offsets = [0]
        for v in list_values:
            if v.shape[1:] != tail:
                raise ValueError("JaggedTensor need values has tha same dimension except the first rank.")
            offsets.append(offsets[-1] + v.shape[0])
        weights = None
        if list_weights:
            assert len(list_values) == len(list_weights)
            weights = torch.cat(list_weights, dim=0)
        return JaggedTensor(torch.cat(list_values, dim=0), torch.as_tensor(offsets), weights)


class JaggedEmbeddingFunction(torch.autograd.Function):
    """pytorch/jagged_embedding_funcs.py over pytorch/py/jagged_ops.cc, fused with the table."""

    @staticmethod
    def forward(ctx, sparse_table, indices, offsets, weights, mode, patch_value):
        ids, p_ids = _ids_ptr(indices)
        if offsets.dtype != torch.int64 or not offsets.is_cuda:
            raise TypeError("offsets must be an int64 CUDA tensor")
        offsets = offsets.contiguous()
        w = weights.contiguous().to(torch.float32) if weights is not None else None
        bags = offsets.numel() - 1
        out = torch.empty((bags, sparse_table.dimension()), dtype=torch.float32, device=indices.device)
        h = sparse_table._on_current_stream()
        api._check(api.lib().krk_sparse_pull_pooled(
            h, p_ids, ids.numel(), C.c_void_p(offsets.data_ptr()), bags,
            C.c_void_p(w.data_ptr()) if w is not None else None, mode, patch_value, C.c_void_p(out.data_ptr()),
            api.DEVICE_PTRS | api.ASYNC), "krk_sparse_pull_pooled")
        ctx.table, ctx.mode, ctx.weights = sparse_table, mode, w
        ctx.save_for_backward(ids, offsets)
        return out

    @staticmethod
    def backward(ctx, grad):
        ids, offsets = ctx.saved_tensors
        t, w = ctx.table, ctx.weights
        grad = grad.contiguous().to(torch.float32)
        h = t._on_current_stream()
        api._check(api.lib().krk_sparse_push_pooled(
            h, C.byref(t._optim.raw), C.c_void_p(ids.data_ptr()), ids.numel(), C.c_void_p(offsets.data_ptr()),
            offsets.numel() - 1, C.c_void_p(w.data_ptr()) if w is not None else None, ctx.mode,
            C.c_void_p(grad.data_ptr()), t.dimension(), t.lr, api.DEVICE_PTRS | api.ASYNC), "krk_sparse_push_pooled")
        return None, None, None, None, None, None


class JaggedEmbedding(torch.nn.Module):
    """pytorch/jagged_embedding.py:10-52: values / offsets / optional weights of a jagged batch,
    pooled per bag with sum or mean; an empty bag yields patch_value."""

    def __init__(self, dimension, initializer=None, optim=None, lr=0.01, mode="sum", patch_value=0.0,
                 capacity_hint=0):
        super().__init__()
        if mode not in ("sum", "mean"):
            raise ValueError("JaggedEmbedding's mode only support sum/mean.")
        self.sparse_table = GpuSparseTable(dimension, initializer, optim, lr, capacity_hint)
        self._mode = 0 if mode == "sum" else 1
        self._patch_value = float(patch_value)

    def forward(self, values, offsets=None, weights=None):
        """forward(JaggedTensor), as the reference's module is called, or forward(values, offsets,
        weights) with the three tensors themselves."""
        if isinstance(values, JaggedTensor):
            values, offsets, weights = values.values(), values.offsets(), values.weights()
        return JaggedEmbeddingFunction.apply(self.sparse_table, values, offsets, weights, self._mode,
                                             self._patch_value)


class GpuCombineSparseTable(torch.nn.Parameter):
    """pytorch/combine_sparse_table.py: the tables of one combined request. Tables of equal
    dimension form one group of the engine (one launch serves a group); the reference allows
    mixed dimensions, which gives one group per distinct dimension here."""

    def __new__(cls, dimensions, initializers=None, optim=None, lr=0.01, capacity_hint=0):
        self = super().__new__(cls, torch.empty(0), requires_grad=True)
        if initializers is not None and len(initializers) != len(dimensions):
            raise ValueError("dimensions and initializers must have the same length")
        self._dimensions = [int(d) for d in dimensions]
        self._tables = [
            api.SparseTable(d, as_initializer(initializers[i] if initializers else None) or api.Initializer.create(
                api.InitializerType.kNormal, {}), capacity_hint=capacity_hint)
            for i, d in enumerate(self._dimensions)]
        self._members = {}                        # dimension -> positions of its tables in the request
        for i, d in enumerate(self._dimensions):
            self._members.setdefault(d, []).append(i)
        self._groups = {d: api.TableGroup([self._tables[i] for i in idx]) for d, idx in self._members.items()}
        self._optim = as_optim(optim) or api.Optim.create(api.OptimType.kSGD)
        self.lr = float(lr)
        return self

    def dimensions(self):
        return self._dimensions

    def tables(self):
        return self._tables

    def _on_current_stream(self, dim):
        g = self._groups[dim]
        api._check(api.lib().krk_group_set_stream(g.h, _stream_ptr()), "krk_group_set_stream")
        return g.h


def _group_offsets(counts):
    off = (C.c_int64 * (len(counts) + 1))()
    for i, c in enumerate(counts):
        off[i + 1] = off[i] + c
    return off


class CombineEmbeddingFunction(torch.autograd.Function):
    """pytorch/combine_embedding.py:10-31 over Emitter::CombinePullSparseTable /
    CombinePushSparseTable (worker/emitter.cc:185-283, 552-632): ids may repeat, within a table
    and across tables."""

    @staticmethod
    def forward(ctx, table, *indices):
        if len(indices) != len(table.dimensions()):
            raise ValueError("one index tensor per table")
        outs = [None] * len(indices)
        saved = []
        for dim, members in table._members.items():
            parts = [_ids_ptr(indices[i])[0].reshape(-1) for i in members]
            ids = torch.cat(parts) if len(parts) > 1 else parts[0]
            off = _group_offsets([p.numel() for p in parts])
            out = torch.empty((ids.numel(), dim), dtype=torch.float32, device=ids.device)
            h = table._on_current_stream(dim)
            api._check(api.lib().krk_group_pull(h, C.c_void_p(ids.data_ptr()), off, C.c_void_p(out.data_ptr()),
                                                api.DEVICE_PTRS | api.ASYNC | api.NOTE_ROWS), "krk_group_pull")
            for k, i in enumerate(members):
                outs[i] = out[off[k]:off[k + 1]].view(tuple(indices[i].shape) + (dim,))
            saved.append(ids)
        ctx.table = table
        ctx.counts = [x.numel() for x in indices]
        ctx.save_for_backward(*saved)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads):
        t = ctx.table
        for ids, (dim, members) in zip(ctx.saved_tensors, t._members.items()):
            counts = [ctx.counts[i] for i in members]
            # an output the loss never used has no gradient: its rows get zeros
            parts = [grads[i].reshape(-1, dim).to(torch.float32) if grads[i] is not None
                     else torch.zeros((c, dim), dtype=torch.float32, device=ids.device)
                     for i, c in zip(members, counts)]
            g = (torch.cat(parts) if len(parts) > 1 else parts[0]).contiguous()
            off = _group_offsets(counts)
            h = t._on_current_stream(dim)
            api._check(api.lib().krk_group_push_raw(h, C.byref(t._optim.raw), C.c_void_p(ids.data_ptr()), off,
                                                    C.c_void_p(g.data_ptr()), dim, t.lr,
                                                    api.DEVICE_PTRS | api.ASYNC | api.IDS_AS_PULLED),
                       "krk_group_push_raw")
        return (None,) * (1 + len(grads))


class CombineEmbedding(torch.nn.Module):
    """pytorch/combine_embedding.py:34-55: one call pulls every table's rows, one backward pushes
    every table's gradients."""

    def __init__(self, dimensions, initializers=None, optim=None, lr=0.01, capacity_hint=0):
        super().__init__()
        self.combine_sparse_table = GpuCombineSparseTable(dimensions, initializers, optim, lr, capacity_hint)

    def forward(self, indices):
        if len(indices) != len(self.combine_sparse_table.dimensions()):
            raise ValueError("one index tensor per table")
        return list(CombineEmbeddingFunction.apply(self.combine_sparse_table, *indices))


class CombineJaggedEmbeddingFunction(torch.autograd.Function):
    """The pooling of pytorch/combine_jagged_embedding.py:47-80 fused with the tables: per table
    one pooled pull forward and one pooled push backward, so the [n, dim] rows that the
    reference pulls, scales and then pools (JaggedEmbeddingSum/MeanFunction over
    pytorch/py/jagged_ops.cc) never exist in memory."""

    @staticmethod
    def forward(ctx, table, modes, patch_values, n_tables, *tensors):
        values = tensors[:n_tables]
        offsets = tensors[n_tables:2 * n_tables]
        weights = tensors[2 * n_tables:]
        outs, saved, ws = [], [], []
        for dim in table._members:                  # members run on their group's stream
            table._on_current_stream(dim)
        for i, t in enumerate(table.tables()):
            ids, p_ids = _ids_ptr(values[i])
            off = offsets[i]
            if off.dtype != torch.int64 or not off.is_cuda:
                raise TypeError("offsets must be an int64 CUDA tensor")
            off = off.contiguous()
            w = weights[i].contiguous().to(torch.float32) if weights[i] is not None else None
            bags = off.numel() - 1
            out = torch.empty((bags, table.dimensions()[i]), dtype=torch.float32, device=ids.device)
            api._check(api.lib().krk_sparse_pull_pooled(
                t.h, p_ids, ids.numel(), C.c_void_p(off.data_ptr()), bags,
                C.c_void_p(w.data_ptr()) if w is not None else None, modes[i], patch_values[i],
                C.c_void_p(out.data_ptr()), api.DEVICE_PTRS | api.ASYNC), "krk_sparse_pull_pooled")
            outs.append(out)
            saved += [ids, off]
            ws.append(w)
        ctx.table, ctx.modes, ctx.weights = table, modes, ws
        ctx.save_for_backward(*saved)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads):
        table = ctx.table
        for dim in table._members:
            table._on_current_stream(dim)
        for i, t in enumerate(table.tables()):
            if grads[i] is None:                    # an output the loss never used: nothing to push
                continue
            ids, off = ctx.saved_tensors[2 * i], ctx.saved_tensors[2 * i + 1]
            w = ctx.weights[i]
            g = grads[i].contiguous().to(torch.float32)
            api._check(api.lib().krk_sparse_push_pooled(
                t.h, C.byref(table._optim.raw), C.c_void_p(ids.data_ptr()), ids.numel(), C.c_void_p(off.data_ptr()),
                off.numel() - 1, C.c_void_p(w.data_ptr()) if w is not None else None, ctx.modes[i],
                C.c_void_p(g.data_ptr()), table.dimensions()[i], table.lr, api.DEVICE_PTRS | api.ASYNC),
                "krk_sparse_push_pooled")
        return (None,) * (4 + 3 * len(table.tables()))


class CombineJaggedEmbedding(torch.nn.Module):
    """pytorch/combine_jagged_embedding.py:11-80: one JaggedTensor per table, pooled per table
    with its own mode and patch value. Per-row weights scale the rows before the pooling, as
    the reference's `embeddings *= weights.unsqueeze(-1)` means to (its `if weights:` raises for
    a tensor of more than one element, so there only a batch without weights gets through)."""

    def __init__(self, dimensions, initializers=None, modes=None, patch_values=None, optim=None, lr=0.01,
                 capacity_hint=0):
        super().__init__()
        if modes:
            assert len(dimensions) == len(modes)
            for mode in modes:
                if mode not in ("sum", "mean"):
                    raise ValueError("CombineJaggedEmbedding's mode only support sum/mean.")
        if patch_values:
            assert len(dimensions) == len(patch_values)
        self.combine_sparse_table = GpuCombineSparseTable(dimensions, initializers, optim, lr, capacity_hint)
        self._modes = [0 if m == "sum" else 1 for m in (modes or ["sum"] * len(dimensions))]
        self._patch_values = [float(p) for p in (patch_values or [0.0] * len(dimensions))]

    def forward(self, inputs):
        assert len(self._modes) == len(inputs)
        n = len(inputs)
        tensors = ([x.values() for x in inputs] + [x.offsets() for x in inputs] + [x.weights() for x in inputs])
        return list(CombineJaggedEmbeddingFunction.apply(self.combine_sparse_table, self._modes,
                                                         self._patch_values, n, *tensors))
