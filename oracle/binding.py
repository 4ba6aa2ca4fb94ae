"""ctypes view of the CPU oracle (oracle/kraken_oracle.c).

TEST INFRASTRUCTURE, NOT PRODUCT CODE: only tests, the smoke check and the
benchmark's cpu_baseline leg may import this module. The shipped package never
does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkraken_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libkraken_ref_containers.so")

ADAGRAD, ADAM, RMSPROP, SGD = 0, 1, 2, 3
INIT_CONSTANT, INIT_UNIFORM, INIT_NORMAL, INIT_XAVIER_UNIFORM, INIT_XAVIER_NORMAL = range(5)
(ST_STEPS, ST_MOMENTUM_BUFFER, ST_STATE_SUM, ST_FIRST_MOMENT, ST_SECOND_MOMENT,
 ST_SECOND_MOMENT_MAX, ST_SQUARE_AVERAGE, ST_G_AVE) = range(8)


class Optim(C.Structure):
    _fields_ = [
        ("type", C.c_int32), ("has_weight_decay", C.c_int32), ("weight_decay", C.c_float),
        ("has_momentum", C.c_int32), ("momentum", C.c_float), ("has_dampening", C.c_int32),
        ("dampening", C.c_float), ("nesterov", C.c_int32), ("beta1", C.c_float),
        ("beta2", C.c_float), ("eps", C.c_float), ("amsgrad", C.c_int32),
        ("alpha", C.c_float), ("centered", C.c_int32),
    ]


class Init(C.Structure):
    _fields_ = [("type", C.c_int32), ("a", C.c_float), ("b", C.c_float), ("seed", C.c_uint64)]


def build(force=False):
    """Compile the oracle with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "libkraken_oracle.so"] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u64(a):
    return np.ascontiguousarray(a, dtype=np.uint64)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def lib():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(_LIB_PATH)
    u64, i64, i32, f32 = C.c_uint64, C.c_int64, C.c_int32, C.c_float
    pf, pu, pi, vp = C.POINTER(f32), C.POINTER(u64), C.POINTER(i64), C.c_void_p
    sig = {
        "kro_hash64": (u64, [u64]),
        "kro_hash64_pair": (u64, [u64, u64]),
        "kro_ring_hit": (u64, [pu, pu, i64, u64]),
        "kro_route_owner": (u64, [pu, pu, i64, u64, u64]),
        "kro_hit_slot": (u64, [u64]),
        "kro_splitmix64": (u64, [u64]),
        "kro_optim_defaults": (None, [i32, C.POINTER(Optim)]),
        "kro_value_create": (vp, [pf, i64]),
        "kro_value_destroy": (None, [vp]),
        "kro_value_val": (pf, [vp]),
        "kro_value_state": (pf, [vp, i32]),
        "kro_value_steps": (i64, [vp]),
        "kro_optim_update": (i32, [C.POINTER(Optim), pf, i64, f32, vp]),
        "kro_init_row": (None, [C.POINTER(Init), u64, i64, pf]),
        "kro_xavier_std": (f32, [f32, i64]),
        "kro_log_u24": (C.c_double, [C.c_uint32]),
        "kro_sincos_u24": (None, [C.c_uint32, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
        "kro_sparse_create": (vp, [i64, C.POINTER(Init)]),
        "kro_sparse_destroy": (None, [vp]),
        "kro_sparse_size": (i64, [vp]),
        "kro_sparse_pull": (i32, [vp, pu, i64, pf]),
        "kro_sparse_push": (i32, [vp, C.POINTER(Optim), pu, i64, pf, i64, f32]),
        "kro_sparse_pull_mt": (i32, [vp, pu, i64, pf]),
        "kro_sparse_push_mt": (i32, [vp, C.POINTER(Optim), pu, i64, pf, i64, f32]),
        "kro_sparse_load": (None, [vp, pu, i64, pf]),
        "kro_sparse_export": (i64, [vp, pu, pf, i32, pf, pi]),
        "kro_sparse_contains": (i32, [vp, u64]),
        "kro_sparse_erase": (i64, [vp, pu, i64]),
        "kro_sparse_fetch": (i64, [vp, pu, i64, C.POINTER(C.c_uint8), pf]),
        "kro_dense_create": (vp, [pf, i64]),
        "kro_dense_destroy": (None, [vp]),
        "kro_dense_pull": (i32, [vp, pf]),
        "kro_dense_push": (i32, [vp, C.POINTER(Optim), pf, i64, f32]),
        "kro_dense_push_coo": (i32, [vp, C.POINTER(Optim), pi, pf, i64, f32]),
        "kro_dense_value": (vp, [vp]),
        "kro_dedup": (i64, [pu, i64, pu, pi]),
        "kro_dedup_sum": (i64, [pu, i64, pf, i64, pu, pf]),
        "kro_jagged_sum_forward": (None, [pf, i64, pi, i64, f32, pf]),
        "kro_jagged_mean_forward": (None, [pf, i64, pi, i64, f32, pf]),
        "kro_jagged_sum_backward": (None, [pi, i64, pf, i64, pf]),
        "kro_jagged_mean_backward": (None, [pi, i64, pf, i64, pf]),
        "kro_abs": (None, [pf, pf, i64]),
        "kro_topk_chunked": (None, [pf, i64, pf, i64, i64]),
        "kro_topk": (None, [pf, i64, pf, i64, i64]),
        "kro_kth_largest_abs": (f32, [pf, i64, i64]),
        "kro_to_coo": (i64, [pf, i64, f32, pi, pf]),
        "kro_lt_keep": (None, [pf, f32, pf, i64]),
        "kro_coo_to_dense": (None, [pi, pf, i64, pf, i64]),
        "kro_take": (None, [pf, pi, pf, i64]),
        "kro_dct_create": (vp, [i64]),
        "kro_dct_destroy": (None, [vp]),
        "kro_dct_compress": (i64, [vp, pf, u64, f32, i64, i32, pi, pf]),
        "kro_dct_tau": (f32, [vp]),
        "kro_dct_residual": (pf, [vp]),
        "kro_dct_step": (u64, [vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def ref_lib():
    """The reference's own containers compiled in place, or None when absent."""
    if not os.path.exists(_REF_PATH):
        return None
    L = C.CDLL(_REF_PATH)
    u64, i64 = C.c_uint64, C.c_int64
    L.ref_hash64.restype = u64
    L.ref_hash64.argtypes = [u64]
    L.ref_hash64_pair.restype = u64
    L.ref_hash64_pair.argtypes = [u64, u64]
    L.ref_map_create.restype = C.c_void_p
    L.ref_map_destroy.argtypes = [C.c_void_p]
    L.ref_map_hit_slot.restype = u64
    L.ref_map_hit_slot.argtypes = [C.c_void_p, u64]
    L.ref_map_insert.restype = i64
    L.ref_map_insert.argtypes = [C.c_void_p, C.POINTER(u64), i64, C.POINTER(C.c_float), i64]
    L.ref_map_find.argtypes = [C.c_void_p, C.POINTER(u64), i64, C.POINTER(C.c_uint8),
                               C.POINTER(C.c_float), i64]
    L.ref_map_keys.restype = i64
    L.ref_map_keys.argtypes = [C.c_void_p, C.POINTER(u64)]
    return L


_REF_JAGGED_PATH = os.path.join(_HERE, "_ref", "libkraken_ref_jagged.so")


def ref_jagged_lib():
    """The reference's own jagged pooling loops (pytorch/py/jagged_ops.cc) compiled in place,
    or None when absent."""
    if not os.path.exists(_REF_JAGGED_PATH):
        return None
    L = C.CDLL(_REF_JAGGED_PATH)
    i64, f32 = C.c_int64, C.c_float
    pf, pi = C.POINTER(f32), C.POINTER(i64)
    for name in ("ref_jagged_sum_forward", "ref_jagged_mean_forward"):
        getattr(L, name).restype = None
        getattr(L, name).argtypes = [pf, i64, pi, i64, f32, pf]
    for name in ("ref_jagged_sum_backward", "ref_jagged_mean_backward"):
        getattr(L, name).restype = None
        getattr(L, name).argtypes = [pi, i64, pf, i64, pf]
    return L


# --------------------------------------------------------------------------- #
# Pythonic wrappers
# --------------------------------------------------------------------------- #

def optim(type_, **conf):
    """Mirror of Optim::Create (ps/optim/optim.cc:18-105): a key that is present
    sets its has_* flag, exactly like the conf-map parser does."""
    o = Optim()
    lib().kro_optim_defaults(type_, C.byref(o))
    for k, v in conf.items():
        if k in ("weight_decay", "momentum", "dampening"):
            setattr(o, k, float(v))
            setattr(o, "has_" + k, 1)
        elif k in ("nesterov", "amsgrad", "centered"):
            setattr(o, k, 1 if v else 0)
        elif k in ("beta1", "beta2", "eps", "alpha"):
            setattr(o, k, float(v))
        else:
            raise KeyError(k)
    return o


def route_owners(ring, table_id, ids):
    """common/router.cc:262-277 over utils::Hash(table_id, id): the owner of every id.
    ring = [(hash_v, node_id), ...] in ascending hash order."""
    rh = np.ascontiguousarray([h for h, _ in ring], dtype=np.uint64)
    rn = np.ascontiguousarray([n for _, n in ring], dtype=np.uint64)
    L = lib()
    return np.array([L.kro_route_owner(_p(rh, C.c_uint64), _p(rn, C.c_uint64), len(ring), int(table_id), int(i))
                     for i in np.asarray(ids, dtype=np.uint64)], dtype=np.uint64)


def init(type_, a=0.0, b=0.0, seed=0):
    return Init(type_, a, b, seed)


class Value:
    def __init__(self, val):
        val = _f32(val)
        self.n = val.size
        self.h = lib().kro_value_create(_p(val, C.c_float), self.n)

    def __del__(self):
        if getattr(self, "h", None):
            lib().kro_value_destroy(self.h)
            self.h = None

    @property
    def val(self):
        return np.ctypeslib.as_array(lib().kro_value_val(self.h), shape=(self.n,)).copy()

    def state(self, st):
        p = lib().kro_value_state(self.h, st)
        if not p:
            return None
        return np.ctypeslib.as_array(p, shape=(self.n,)).copy()

    @property
    def steps(self):
        return lib().kro_value_steps(self.h)

    def update(self, o, grad, lr):
        grad = _f32(grad)
        return lib().kro_optim_update(C.byref(o), _p(grad, C.c_float), grad.size, lr, self.h)


class SparseTable:
    def __init__(self, dim, init_):
        self.dim = dim
        self._init = init_
        self.h = lib().kro_sparse_create(dim, C.byref(init_))

    def __del__(self):
        if getattr(self, "h", None):
            lib().kro_sparse_destroy(self.h)
            self.h = None

    def __len__(self):
        return lib().kro_sparse_size(self.h)

    def pull(self, ids, mt=False):
        ids = _u64(ids)
        out = np.empty((ids.size, self.dim), np.float32)
        fn = lib().kro_sparse_pull_mt if mt else lib().kro_sparse_pull
        rc = fn(self.h, _p(ids, C.c_uint64), ids.size, _p(out, C.c_float))
        return rc, out

    def push(self, o, ids, grads, lr, mt=False):
        ids = _u64(ids)
        grads = _f32(grads)
        gd = grads.shape[-1] if grads.ndim > 1 else (grads.size // max(ids.size, 1))
        fn = lib().kro_sparse_push_mt if mt else lib().kro_sparse_push
        return fn(self.h, C.byref(o), _p(ids, C.c_uint64), ids.size, _p(grads, C.c_float), gd, lr)

    def load(self, ids, vals):
        ids = _u64(ids)
        vals = _f32(vals)
        lib().kro_sparse_load(self.h, _p(ids, C.c_uint64), ids.size, _p(vals, C.c_float))

    def contains(self, id_):
        return bool(lib().kro_sparse_contains(self.h, int(id_)))

    def erase(self, ids):
        ids = _u64(ids)
        return lib().kro_sparse_erase(self.h, _p(ids, C.c_uint64), ids.size)

    def fetch(self, ids):
        """-> found[n] bool, vals[n, dim] (rows of absent ids are zero)"""
        ids = _u64(ids)
        found = np.zeros(ids.size, np.uint8)
        vals = np.zeros((ids.size, self.dim), np.float32)
        lib().kro_sparse_fetch(self.h, _p(ids, C.c_uint64), ids.size, _p(found, C.c_uint8), _p(vals, C.c_float))
        return found.astype(bool), vals

    def export(self, state_type=None):
        n = len(self)
        ids = np.empty(n, np.uint64)
        vals = np.empty((n, self.dim), np.float32)
        steps = np.empty(n, np.int64)
        st = np.empty((n, self.dim), np.float32) if state_type is not None else None
        lib().kro_sparse_export(self.h, _p(ids, C.c_uint64), _p(vals, C.c_float),
                                state_type if state_type is not None else 0,
                                _p(st, C.c_float) if st is not None else None,
                                _p(steps, C.c_int64))
        return ids, vals, st, steps


class DenseTable:
    def __init__(self, val):
        val = _f32(val).ravel()
        self.n = val.size
        self.h = lib().kro_dense_create(_p(val, C.c_float), self.n)

    def __del__(self):
        if getattr(self, "h", None):
            lib().kro_dense_destroy(self.h)
            self.h = None

    def pull(self):
        out = np.empty(self.n, np.float32)
        lib().kro_dense_pull(self.h, _p(out, C.c_float))
        return out

    def push(self, o, grad, lr):
        grad = _f32(grad).ravel()
        return lib().kro_dense_push(self.h, C.byref(o), _p(grad, C.c_float), grad.size, lr)

    def push_coo(self, o, idx, val, lr):
        idx = _i64(idx)
        val = _f32(val)
        return lib().kro_dense_push_coo(self.h, C.byref(o), _p(idx, C.c_int64),
                                        _p(val, C.c_float), idx.size, lr)

    def state(self, st):
        v = lib().kro_dense_value(self.h)
        p = lib().kro_value_state(v, st)
        if not p:
            return None
        return np.ctypeslib.as_array(p, shape=(self.n,)).copy()

    @property
    def steps(self):
        return lib().kro_value_steps(lib().kro_dense_value(self.h))


def dedup(ids):
    ids = _u64(ids)
    uids = np.empty(ids.size, np.uint64)
    inv = np.empty(ids.size, np.int64)
    u = lib().kro_dedup(_p(ids, C.c_uint64), ids.size, _p(uids, C.c_uint64), _p(inv, C.c_int64))
    return uids[:u].copy(), inv


def dedup_sum(ids, grads):
    ids = _u64(ids)
    grads = _f32(grads)
    dim = grads.shape[-1]
    uids = np.empty(ids.size, np.uint64)
    out = np.empty((ids.size, dim), np.float32)
    u = lib().kro_dedup_sum(_p(ids, C.c_uint64), ids.size, _p(grads, C.c_float), dim,
                            _p(uids, C.c_uint64), _p(out, C.c_float))
    return uids[:u].copy(), out[:u].copy()


def jagged_forward(values, offsets, mode="sum", patch_value=0.0):
    """pytorch/py/jagged_ops.cc SumForward / MeanForward on [rows, col] values."""
    values = _f32(values)
    offsets = np.ascontiguousarray(offsets, np.int64)
    col = values.shape[-1]
    k = offsets.size - 1
    out = np.empty((k, col), np.float32)
    fn = lib().kro_jagged_sum_forward if mode == "sum" else lib().kro_jagged_mean_forward
    fn(_p(values, C.c_float), col, _p(offsets, C.c_int64), k, patch_value, _p(out, C.c_float))
    return out


def jagged_backward(offsets, grads, mode="sum"):
    """Gradient of jagged_forward with respect to the values: [offsets[-1], col]."""
    grads = _f32(grads)
    offsets = np.ascontiguousarray(offsets, np.int64)
    col = grads.shape[-1]
    k = offsets.size - 1
    out = np.zeros((int(offsets[-1]), col), np.float32)
    fn = lib().kro_jagged_sum_backward if mode == "sum" else lib().kro_jagged_mean_backward
    fn(_p(offsets, C.c_int64), k, _p(grads, C.c_float), col, _p(out, C.c_float))
    return out


def init_row(init_, id_, dim):
    out = np.empty(dim, np.float32)
    lib().kro_init_row(C.byref(init_), int(id_), dim, _p(out, C.c_float))
    return out


def topk(x, k, hw_threads=8, t_num=None):
    x = _f32(x)
    y = np.empty(k, np.float32)
    if t_num is None:
        lib().kro_topk(_p(x, C.c_float), x.size, _p(y, C.c_float), k, hw_threads)
    else:
        lib().kro_topk_chunked(_p(x, C.c_float), x.size, _p(y, C.c_float), k, t_num)
    return y


def kth_largest_abs(x, k):
    x = _f32(x)
    return lib().kro_kth_largest_abs(_p(x, C.c_float), x.size, k)


def to_coo(x, th):
    x = _f32(x).ravel()
    idx = np.empty(x.size, np.int64)
    val = np.empty(x.size, np.float32)
    nnz = lib().kro_to_coo(_p(x, C.c_float), x.size, th, _p(idx, C.c_int64), _p(val, C.c_float))
    return idx[:nnz].copy(), val[:nnz].copy()


def lt_keep(x, th):
    x = _f32(x).ravel()
    y = np.empty_like(x)
    lib().kro_lt_keep(_p(x, C.c_float), th, _p(y, C.c_float), x.size)
    return y


def coo_to_dense(idx, val, n):
    idx = _i64(idx)
    val = _f32(val)
    out = np.empty(n, np.float32)
    lib().kro_coo_to_dense(_p(idx, C.c_int64), _p(val, C.c_float), idx.size, _p(out, C.c_float), n)
    return out


def take(x, idx):
    x = _f32(x)
    idx = _i64(idx)
    y = np.empty(idx.size, np.float32)
    lib().kro_take(_p(x, C.c_float), _p(idx, C.c_int64), _p(y, C.c_float), idx.size)
    return y


def absf(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().kro_abs(_p(x, C.c_float), _p(y, C.c_float), x.size)
    return y


class DctState:
    """worker/dct_emitter.cc DenseBag."""

    def __init__(self, n):
        self.n = n
        self.h = lib().kro_dct_create(n)

    def __del__(self):
        if getattr(self, "h", None):
            lib().kro_dct_destroy(self.h)
            self.h = None

    def compress(self, grad, life_span=1000, eta=0.75, hw_threads=8, exact_select=True):
        grad = _f32(grad).ravel()
        idx = np.empty(self.n, np.int64)
        val = np.empty(self.n, np.float32)
        nnz = lib().kro_dct_compress(self.h, _p(grad, C.c_float), life_span, eta, hw_threads,
                                     1 if exact_select else 0, _p(idx, C.c_int64),
                                     _p(val, C.c_float))
        if nnz < 0:
            return None, None
        return idx[:nnz].copy(), val[:nnz].copy()

    @property
    def tau(self):
        return lib().kro_dct_tau(self.h)

    @property
    def residual(self):
        return np.ctypeslib.as_array(lib().kro_dct_residual(self.h), shape=(self.n,)).copy()

    @property
    def step(self):
        return lib().kro_dct_step(self.h)
