"""ctypes binding of libkraken_hip.so (include/kraken_hip.h) with the reference's names.

`SparseTable`, `DenseTable`, `Optim.create`, `Initializer.create` and `DenseBag` follow
kraken/ps/{sparse_table,dense_table}.h, ps/optim/optim.h, ps/initializer/initializer.h and
worker/dct_emitter.h: same arguments, same integer error codes. There is no CPU path: when the
library or a GPU is missing every call raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkraken_hip.so")

DEVICE_PTRS = 0x1
ASYNC = 0x2
NOTE_ROWS = 0x4          # on a pull: keep the row of every position for a push_raw of the same ids
IDS_AS_PULLED = 0x8      # on a push_raw: ids is the unchanged buffer of that pull

SUCCESS = 0
UNSUPPORTED_OPTIM = 6
INTERFACE_UNIMPLEMENTED = 10
GRADIENT_UNCOMPATIBLE = 11
SPARSE_ID_NOT_EXIST = 12
UNSUPPORTED_INITIALIZER = 13
E_DEVICE, E_ARGUMENT, E_CAPACITY, E_IO = -2, -3, -4, -5


class OptimType:          # common/info.h:46-51
    kAdagrad, kAdam, kRMSprop, kSGD = 0, 1, 2, 3


class InitializerType:    # common/info.h:54-60
    kConstant, kUniform, kNormal, kXavierUniform, kXavierNormal = range(5)


class StateType:          # common/info.h:63-72
    (kSteps, kMomentumBuffer, kStateSum, kFirstMoment, kSecondMoment, kSecondMomentMax,
     kSquareAverage, kGAve) = range(8)


class krk_optim(C.Structure):
    _fields_ = [
        ("type", C.c_int32), ("has_weight_decay", C.c_int32), ("weight_decay", C.c_float),
        ("has_momentum", C.c_int32), ("momentum", C.c_float), ("has_dampening", C.c_int32),
        ("dampening", C.c_float), ("nesterov", C.c_int32), ("beta1", C.c_float),
        ("beta2", C.c_float), ("eps", C.c_float), ("amsgrad", C.c_int32),
        ("alpha", C.c_float), ("centered", C.c_int32), ("initial_accumulator", C.c_float),
    ]


class krk_init(C.Structure):
    _fields_ = [("type", C.c_int32), ("a", C.c_float), ("b", C.c_float), ("seed", C.c_uint64)]


EXPORTS = {
    # name: (restype, argtypes)
    "krk_optim_defaults": (C.c_int32, [C.c_int32, C.POINTER(krk_optim)]),
    "krk_optim_set": (C.c_int32, [C.POINTER(krk_optim), C.c_char_p, C.c_char_p]),
    "krk_init_defaults": (C.c_int32, [C.c_int32, C.POINTER(krk_init)]),
    "krk_init_set": (C.c_int32, [C.POINTER(krk_init), C.c_char_p, C.c_char_p]),
    "krk_runtime_init": (C.c_int32, [C.c_int32]),
    "krk_last_error_string": (C.c_char_p, []),
    "krk_error_message": (C.c_char_p, [C.c_int32]),
    "krk_malloc": (C.c_int32, [C.POINTER(C.c_void_p), C.c_size_t]),
    "krk_free": (C.c_int32, [C.c_void_p]),
    "krk_memcpy_h2d": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "krk_memcpy_d2h": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "krk_memset": (C.c_int32, [C.c_void_p, C.c_int, C.c_size_t]),
    "krk_device_synchronize": (C.c_int32, []),
    "krk_mem_info": (C.c_int32, [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "krk_wire_rows_bytes": (C.c_int64, [C.c_int64, C.c_int64]),
    "krk_sparse_pull_wire": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "krk_sparse_push_wire": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_int64, C.c_void_p,
                                         C.c_int64, C.c_float]),
    "krk_host_malloc": (C.c_int32, [C.POINTER(C.c_void_p), C.c_size_t]),
    "krk_host_free": (C.c_int32, [C.c_void_p]),
    "krk_stream_copy": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "krk_sparse_create": (C.c_int32, [C.c_int64, C.POINTER(krk_init), C.c_int64, C.POINTER(C.c_void_p)]),
    "krk_sparse_destroy": (C.c_int32, [C.c_void_p]),
    "krk_sparse_dim": (C.c_int32, [C.c_void_p, C.POINTER(C.c_int64)]),
    "krk_sparse_size": (C.c_int32, [C.c_void_p, C.POINTER(C.c_int64)]),
    "krk_sparse_reserve": (C.c_int32, [C.c_void_p, C.c_int64]),
    "krk_sparse_sync": (C.c_int32, [C.c_void_p]),
    "krk_sparse_set_stream": (C.c_int32, [C.c_void_p, C.c_void_p]),
    "krk_sparse_pull": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_uint32]),
    "krk_sparse_push": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_int64, C.c_void_p,
                                    C.c_int64, C.c_float, C.c_uint32]),
    "krk_sparse_push_raw": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_int64,
                                        C.c_void_p, C.c_int64, C.c_float, C.c_uint32]),
    "krk_sparse_pull_pooled": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64,
                                           C.c_void_p, C.c_int32, C.c_float, C.c_void_p, C.c_uint32]),
    "krk_sparse_push_pooled": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_int64,
                                           C.c_void_p, C.c_int64, C.c_void_p, C.c_int32, C.c_void_p,
                                           C.c_int64, C.c_float, C.c_uint32]),
    "krk_sparse_lookup": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_uint32]),
    "krk_sparse_import": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_uint32]),
    "krk_sparse_export": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p,
                                      C.c_void_p, C.c_int64, C.POINTER(C.c_int64), C.c_uint32]),
    "krk_sparse_fetch": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int32,
                                     C.c_void_p, C.c_void_p, C.c_uint32]),
    "krk_sparse_import_state": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p,
                                            C.c_void_p, C.c_uint32]),
    "krk_sparse_states": (C.c_int32, [C.c_void_p, C.POINTER(C.c_uint32)]),
    "krk_dense_states": (C.c_int32, [C.c_void_p, C.POINTER(C.c_uint32)]),
    "krk_dense_import_state": (C.c_int32, [C.c_void_p, C.c_int32, C.c_void_p, C.c_int64, C.c_uint32]),
    "krk_sparse_save_file": (C.c_int32, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_char_p]),
    "krk_sparse_load_file": (C.c_int32, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_char_p, C.c_void_p, C.c_void_p,
                                         C.POINTER(C.c_int64)]),
    "krk_dense_size": (C.c_int32, [C.c_void_p, C.POINTER(C.c_int64)]),
    "krk_dense_save_file": (C.c_int32, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_char_p, C.POINTER(C.c_int64),
                                        C.c_int32]),
    "krk_dense_load_file": (C.c_int32, [C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64), C.c_char_p,
                                        C.c_size_t, C.POINTER(C.c_int64), C.POINTER(C.c_int32)]),
    "krk_sparse_erase": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.POINTER(C.c_int64), C.c_uint32]),
    "krk_sparse_select_routed": (C.c_int32, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p, C.c_int64,
                                             C.c_uint64, C.c_int32, C.c_void_p, C.c_int64,
                                             C.POINTER(C.c_int64), C.c_uint32]),
    "krk_hbm_probe": (C.c_int32, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t]),
    "krk_hbm_probe_lines": (C.c_int32, [C.c_int32, C.c_void_p, C.c_size_t, C.c_int64, C.c_uint64]),
    "krk_route_ids": (C.c_int32, [C.c_uint64, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64,
                                  C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                  C.POINTER(C.c_int64), C.c_uint32]),
    "krk_dedup": (C.c_int32, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.POINTER(C.c_int64),
                              C.c_uint32]),
    "krk_dedup_noalloc": (C.c_int32, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "krk_dedup_sum": (C.c_int32, [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                                  C.c_void_p, C.POINTER(C.c_int64), C.c_uint32]),
    "krk_expand_rows": (C.c_int32, [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p,
                                    C.c_uint32]),
    "krk_dense_create": (C.c_int32, [C.c_void_p, C.c_int64, C.c_uint32, C.POINTER(C.c_void_p)]),
    "krk_dense_destroy": (C.c_int32, [C.c_void_p]),
    "krk_dense_sync": (C.c_int32, [C.c_void_p]),
    "krk_dense_pull": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "krk_dense_push": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_int64, C.c_float,
                                   C.c_uint32]),
    "krk_dense_push_coo": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_void_p,
                                       C.c_int64, C.c_float, C.c_uint32]),
    "krk_dense_state": (C.c_int32, [C.c_void_p, C.c_int32, C.c_void_p, C.c_uint32]),
    "krk_dense_steps": (C.c_int32, [C.c_void_p, C.POINTER(C.c_int64)]),
    "krk_dense_group_create": (C.c_int32, [C.POINTER(C.c_void_p), C.c_int32, C.POINTER(C.c_void_p)]),
    "krk_dense_group_destroy": (C.c_int32, [C.c_void_p]),
    "krk_dense_group_sync": (C.c_int32, [C.c_void_p]),
    "krk_dense_group_size": (C.c_int32, [C.c_void_p, C.POINTER(C.c_int64)]),
    "krk_dense_group_pull": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "krk_dense_group_push": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_float, C.c_uint32]),
    "krk_dct_create": (C.c_int32, [C.c_int64, C.POINTER(C.c_void_p)]),
    "krk_dct_destroy": (C.c_int32, [C.c_void_p]),
    "krk_dct_compress": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_float, C.c_void_p,
                                     C.c_void_p, C.c_int64, C.POINTER(C.c_int64), C.c_uint32]),
    "krk_dct_tau": (C.c_int32, [C.c_void_p, C.POINTER(C.c_float)]),
    "krk_dct_step": (C.c_int32, [C.c_void_p, C.POINTER(C.c_uint64)]),
    "krk_dct_residual": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "krk_coo_to_dense": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64,
                                     C.c_uint32]),
    "krk_event_create": (C.c_int32, [C.POINTER(C.c_void_p)]),
    "krk_event_destroy": (C.c_int32, [C.c_void_p]),
    "krk_event_record": (C.c_int32, [C.c_void_p, C.c_void_p]),
    "krk_event_wait": (C.c_int32, [C.c_void_p, C.c_void_p]),
    "krk_group_create": (C.c_int32, [C.POINTER(C.c_void_p), C.c_int32, C.POINTER(C.c_void_p)]),
    "krk_group_destroy": (C.c_int32, [C.c_void_p]),
    "krk_group_sync": (C.c_int32, [C.c_void_p]),
    "krk_group_pull": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32]),
    "krk_group_push": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.c_int64, C.c_float, C.c_uint32]),
    "krk_group_push_raw": (C.c_int32, [C.c_void_p, C.POINTER(krk_optim), C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_int64, C.c_float, C.c_uint32]),
    "krk_group_set_stream": (C.c_int32, [C.c_void_p, C.c_void_p]),
    "krk_event_elapsed_ms": (C.c_int32, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "krk_dct2_forward": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_uint32]),
    "krk_dct2_inverse": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_uint32]),
}

_lib = None


class KrakenHipError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        msg = lib().krk_last_error_string().decode() if _lib is not None else ""
        super().__init__("%s failed with code %d (%s) %s" % (
            what, code, lib().krk_error_message(code).decode(), msg))


def lib():
    """Loads the shared library; raises when it has not been built (no fallback exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is missing: build it with `python -m kraken_amd.build`; "
                           "there is no CPU implementation to fall back to" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    for name, (res, args) in EXPORTS.items():
        if not hasattr(L, name):
            continue
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def _check(rc, what):
    if rc != SUCCESS:
        raise KrakenHipError(rc, what)


def _ptr(a):
    if a is None:
        return None
    if isinstance(a, DeviceArray):
        return C.c_void_p(a.ptr)
    return a.ctypes.data_as(C.c_void_p)


class DeviceArray:
    """A typed device buffer owned by the harness (krk_malloc); not part of the table engine."""

    def __init__(self, shape, dtype):
        self.shape = tuple(shape) if isinstance(shape, (tuple, list)) else (int(shape),)
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        p = C.c_void_p()
        _check(lib().krk_malloc(C.byref(p), max(self.nbytes, 16)), "krk_malloc")
        self.ptr = p.value

    @classmethod
    def from_host(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        _check(lib().krk_memcpy_h2d(C.c_void_p(d.ptr), a.ctypes.data_as(C.c_void_p), a.nbytes), "h2d")
        return d

    def to_host(self):
        out = np.empty(self.shape, self.dtype)
        _check(lib().krk_memcpy_d2h(out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr), self.nbytes),
               "d2h")
        return out

    def free(self):
        if self.ptr:
            lib().krk_free(C.c_void_p(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def pinned_empty(shape, dtype):
    """A numpy array in page-locked host memory (krk_host_malloc); it is freed with the array."""
    shape = tuple(shape) if isinstance(shape, (tuple, list)) else (int(shape),)
    dtype = np.dtype(dtype)
    nbytes = int(np.prod(shape)) * dtype.itemsize
    p = C.c_void_p()
    _check(lib().krk_host_malloc(C.byref(p), max(nbytes, 16)), "krk_host_malloc")

    class _Owner:
        def __init__(self, ptr):
            self.ptr = ptr
            self.__array_interface__ = {"data": (ptr, False), "shape": (max(nbytes, 1),), "typestr": "|u1",
                                        "version": 3}

        def __del__(self):
            try:
                lib().krk_host_free(C.c_void_p(self.ptr))
            except Exception:
                pass

    raw = np.asarray(_Owner(p.value))
    return raw[:nbytes].view(dtype).reshape(shape)


def pinned_copy(a):
    a = np.ascontiguousarray(a)
    out = pinned_empty(a.shape, a.dtype)
    out[...] = a
    return out


def synchronize():
    _check(lib().krk_device_synchronize(), "krk_device_synchronize")


class Optim:
    """ps/optim/optim.h: built from (OptimType, string conf) like Optim::Create."""

    def __init__(self, raw):
        self.raw = raw

    @staticmethod
    def create(optim_type, conf=None):
        o = krk_optim()
        rc = lib().krk_optim_defaults(int(optim_type), C.byref(o))
        if rc != SUCCESS:
            return None          # Optim::Create returns an empty pointer for an unknown type
        for k, v in (conf or {}).items():
            if isinstance(v, bool):
                v = "true" if v else "false"
            lib().krk_optim_set(C.byref(o), str(k).encode(), str(v).encode())
        return Optim(o)

    @property
    def optim_type(self):
        return self.raw.type


class Initializer:
    """ps/initializer/initializer.h: built from (InitializerType, string conf)."""

    def __init__(self, raw):
        self.raw = raw

    @staticmethod
    def create(init_type, conf=None):
        i = krk_init()
        rc = lib().krk_init_defaults(int(init_type), C.byref(i))
        if rc != SUCCESS:
            return None
        for k, v in (conf or {}).items():
            lib().krk_init_set(C.byref(i), str(k).encode(), str(v).encode())
        return Initializer(i)

    @property
    def type(self):
        return self.raw.type


def _flags(*arrays, extra=0):
    dev = [isinstance(a, DeviceArray) for a in arrays if a is not None]
    if dev and all(dev):
        return DEVICE_PTRS | extra
    if any(dev):
        raise ValueError("mix of host and device arrays in one call")
    return extra


class SparseTable:
    """ps/sparse_table.h. Pull/Push return the reference's int32 error code."""

    def __init__(self, dimension, initializer, capacity_hint=0):
        self.dimension = int(dimension)
        h = C.c_void_p()
        _check(lib().krk_sparse_create(self.dimension, C.byref(initializer.raw), capacity_hint,
                                       C.byref(h)), "krk_sparse_create")
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            lib().krk_sparse_destroy(self.h)
            self.h = None

    __del__ = close

    def __len__(self):
        n = C.c_int64()
        _check(lib().krk_sparse_size(self.h, C.byref(n)), "krk_sparse_size")
        return n.value

    def reserve(self, rows):
        _check(lib().krk_sparse_reserve(self.h, rows), "krk_sparse_reserve")

    def sync(self):
        return lib().krk_sparse_sync(self.h)

    def Pull(self, sparse_ids, out=None, async_=False, note_rows=False):
        """-> (code, vals[n, dimension]). note_rows (device ids): see KRK_NOTE_ROWS."""
        if isinstance(sparse_ids, DeviceArray):
            n = sparse_ids.size
            if out is None:
                out = DeviceArray((n, self.dimension), np.float32)
        else:
            sparse_ids = np.ascontiguousarray(sparse_ids, dtype=np.uint64)
            n = sparse_ids.size
            if out is None:
                out = np.empty((n, self.dimension), np.float32)
        rc = lib().krk_sparse_pull(self.h, _ptr(sparse_ids), n, _ptr(out),
                                   _flags(sparse_ids, out, extra=(ASYNC if async_ else 0) |
                                          (NOTE_ROWS if note_rows else 0)))
        return rc, out

    def Push(self, optim, sparse_ids, grads, lr, async_=False, raw=False, as_pulled=False):
        if isinstance(sparse_ids, DeviceArray):
            n = sparse_ids.size
            gd = grads.shape[-1]
        else:
            sparse_ids = np.ascontiguousarray(sparse_ids, dtype=np.uint64)
            grads = np.ascontiguousarray(grads, dtype=np.float32)
            n = sparse_ids.size
            gd = grads.shape[-1] if grads.ndim > 1 else (grads.size // max(n, 1))
        fn = lib().krk_sparse_push_raw if raw else lib().krk_sparse_push
        return fn(self.h, C.byref(optim.raw), _ptr(sparse_ids), n, _ptr(grads), gd, lr,
                  _flags(sparse_ids, grads, extra=(ASYNC if async_ else 0) |
                         (IDS_AS_PULLED if as_pulled else 0)))

    def PushRaw(self, optim, ids, grads, lr, async_=False, as_pulled=False):
        """Emitter::PushSparseTable's dedup + sum fused with Push: ids may repeat. as_pulled:
        ids is the unchanged device buffer of the last Pull(note_rows=True) (KRK_IDS_AS_PULLED)."""
        return self.Push(optim, ids, grads, lr, async_=async_, raw=True, as_pulled=as_pulled)

    _POOL = {"sum": 0, "mean": 1}

    def PullPooled(self, ids, offsets, mode="sum", patch_value=0.0, weights=None, out=None, async_=False):
        """JaggedEmbedding.forward (pytorch/jagged_embedding.py:32-52) in one launch: Pull of the
        bags' ids fused with jagged sum / mean. -> (code, [bags, dim]). Host arrays or
        DeviceArrays (all of one kind)."""
        dev = isinstance(ids, DeviceArray)
        if not dev:
            ids = np.ascontiguousarray(ids, dtype=np.uint64)
            offsets = np.ascontiguousarray(offsets, dtype=np.int64)
            if weights is not None:
                weights = np.ascontiguousarray(weights, dtype=np.float32)
        bags = offsets.size - 1
        if out is None:
            out = DeviceArray((bags, self.dimension), np.float32) if dev else \
                np.empty((bags, self.dimension), np.float32)
        rc = lib().krk_sparse_pull_pooled(self.h, _ptr(ids), ids.size, _ptr(offsets), bags, _ptr(weights),
                                          self._POOL[mode], patch_value, _ptr(out),
                                          _flags(ids, out, extra=ASYNC if async_ else 0))
        return rc, out

    def PushPooled(self, optim, ids, offsets, bag_grads, lr, mode="sum", weights=None, async_=False):
        """The backward of PullPooled fused with PushRaw: bag_grads is [bags, dim]."""
        dev = isinstance(ids, DeviceArray)
        if not dev:
            ids = np.ascontiguousarray(ids, dtype=np.uint64)
            offsets = np.ascontiguousarray(offsets, dtype=np.int64)
            bag_grads = np.ascontiguousarray(bag_grads, dtype=np.float32)
            if weights is not None:
                weights = np.ascontiguousarray(weights, dtype=np.float32)
        bags = offsets.size - 1
        gd = bag_grads.shape[-1] if len(bag_grads.shape) > 1 else bag_grads.size // max(bags, 1)
        return lib().krk_sparse_push_pooled(self.h, C.byref(optim.raw), _ptr(ids), ids.size, _ptr(offsets),
                                            bags, _ptr(weights), self._POOL[mode], _ptr(bag_grads), gd, lr,
                                            _flags(ids, bag_grads, extra=ASYNC if async_ else 0))

    def PullWire(self, sparse_ids, reply=None):
        """Pull whose reply is the body of the reference's PullSparseTableResponse: -> (code, bytes)"""
        sparse_ids = np.ascontiguousarray(sparse_ids, dtype=np.uint64)
        nbytes = lib().krk_wire_rows_bytes(sparse_ids.size, self.dimension)
        if reply is None:
            reply = np.empty(nbytes // 8 + 1, np.uint64).view(np.uint8)[:nbytes]
        rc = lib().krk_sparse_pull_wire(self.h, _ptr(sparse_ids), sparse_ids.size, _ptr(reply))
        return rc, reply

    def PushWire(self, optim, sparse_ids, grads_wire, lr):
        """Push whose gradients are the `grads` member of the reference's PushSparseTableRequest."""
        sparse_ids = np.ascontiguousarray(sparse_ids, dtype=np.uint64)
        return lib().krk_sparse_push_wire(self.h, C.byref(optim.raw), _ptr(sparse_ids), sparse_ids.size,
                                          _ptr(grads_wire), grads_wire.size, lr)

    def lookup(self, ids):
        if isinstance(ids, DeviceArray):
            rows = DeviceArray(ids.size, np.int32)
            n = ids.size
        else:
            ids = np.ascontiguousarray(ids, dtype=np.uint64)
            rows = np.empty(ids.size, np.int32)
            n = ids.size
        _check(lib().krk_sparse_lookup(self.h, _ptr(ids), n, _ptr(rows), _flags(ids, rows)),
               "krk_sparse_lookup")
        return rows

    def load(self, ids, vals):
        if not isinstance(ids, DeviceArray):
            ids = np.ascontiguousarray(ids, dtype=np.uint64)
            vals = np.ascontiguousarray(vals, dtype=np.float32)
        _check(lib().krk_sparse_import(self.h, _ptr(ids), ids.size, _ptr(vals), _flags(ids, vals)),
               "krk_sparse_import")

    def fetch(self, ids, state_type=None):
        """Ps::TryFetchSparseValues (ps/ps.cc:914-935): nothing is inserted.
        -> found[n] bool, vals[n, dim], state[n, dim] or None, steps[n]"""
        ids = np.ascontiguousarray(ids, dtype=np.uint64)
        n = ids.size
        found = np.zeros(n, np.uint8)
        vals = np.empty((n, self.dimension), np.float32)
        steps = np.empty(n, np.int64)
        st = np.empty((n, self.dimension), np.float32) if state_type is not None else None
        _check(lib().krk_sparse_fetch(self.h, _ptr(ids), n, _ptr(found), _ptr(vals),
                                      state_type if state_type is not None else 1, _ptr(st), _ptr(steps), 0),
               "krk_sparse_fetch")
        return found.astype(bool), vals, st, steps

    def load_state(self, ids, state_type=None, state=None, steps=None):
        """Optimizer state / step counters of rows brought in with load(); returns the code."""
        ids = np.ascontiguousarray(ids, dtype=np.uint64)
        if state is not None:
            state = np.ascontiguousarray(state, dtype=np.float32)
        if steps is not None:
            steps = np.ascontiguousarray(steps, dtype=np.int64)
        return lib().krk_sparse_import_state(self.h, _ptr(ids), ids.size,
                                             state_type if state_type is not None else 1,
                                             _ptr(state), _ptr(steps), 0)

    def save(self, path, table_id, name):
        """Checkpoint::SaveSparseTable (checkpoint/checkpoint.cc:465-509); returns the code."""
        return lib().krk_sparse_save_file(self.h, os.fsencode(path), table_id, name.encode())

    def load_file(self, path, table_id, name, keep=None):
        """Checkpoint::LoadSparseTable (checkpoint/checkpoint.cc:586-649). keep(id) -> bool plays
        the routing test of line 640. -> (code, rows taken)"""
        KEEP = C.CFUNCTYPE(C.c_int32, C.c_uint64, C.c_void_p)
        cb = KEEP(lambda id_, ctx: 1 if keep(id_) else 0) if keep is not None else None
        taken = C.c_int64()
        rc = lib().krk_sparse_load_file(self.h, os.fsencode(path), table_id, name.encode(),
                                        C.cast(cb, C.c_void_p) if cb is not None else None, None,
                                        C.byref(taken))
        return rc, taken.value

    def erase(self, ids):
        """The clean-up of ps/ps.cc:92-109 for the listed ids; returns how many rows went."""
        ids = np.ascontiguousarray(ids, dtype=np.uint64)
        gone = C.c_int64()
        _check(lib().krk_sparse_erase(self.h, _ptr(ids), ids.size, C.byref(gone), 0), "krk_sparse_erase")
        return gone.value

    def select_routed(self, table_id, ring, node_id, owned=True):
        """The ids of the rows that the reference's router (common/router.cc:262-277 over
        utils::Hash(table_id, id)) gives to node_id (owned) or to other nodes (not owned), in
        row order (export's). ring = [(hash_v, node_id), ...] in ascending hash order."""
        rh = np.ascontiguousarray([h for h, _ in ring], dtype=np.uint64)
        rn = np.ascontiguousarray([n for _, n in ring], dtype=np.uint64)
        count = C.c_int64()
        rc = lib().krk_sparse_select_routed(self.h, int(table_id), _ptr(rh), _ptr(rn), len(ring), int(node_id),
                                            1 if owned else 0, None, 0, C.byref(count), 0)
        if rc == SUCCESS:
            return np.empty(0, np.uint64)
        if rc != E_CAPACITY:
            _check(rc, "krk_sparse_select_routed")
        ids = np.empty(count.value, np.uint64)
        _check(lib().krk_sparse_select_routed(self.h, int(table_id), _ptr(rh), _ptr(rn), len(ring), int(node_id),
                                              1 if owned else 0, _ptr(ids), ids.size, C.byref(count), 0),
               "krk_sparse_select_routed")
        return ids[:count.value]

    def export(self, state_type=None):
        """-> ids[rows], vals[rows, dim], state[rows, dim] or None, steps[rows] (insertion order)"""
        n = len(self)
        ids = np.empty(n, np.uint64)
        vals = np.empty((n, self.dimension), np.float32)
        steps = np.empty(n, np.int64)
        st = np.empty((n, self.dimension), np.float32) if state_type is not None else None
        rows = C.c_int64()
        _check(lib().krk_sparse_export(self.h, _ptr(ids), _ptr(vals),
                                       state_type if state_type is not None else 1, _ptr(st),
                                       _ptr(steps), n, C.byref(rows), 0), "krk_sparse_export")
        assert rows.value == n
        return ids, vals, st, steps


class TableGroup:
    """The sparse tables of one combined request (Ps::CombinePullSparseTable /
    CombinePushSparseTable, ps/ps_op.cc:370-387, 456-469): one launch serves all of them."""

    def __init__(self, tables):
        self.tables = list(tables)
        self.dimension = self.tables[0].dimension
        arr = (C.c_void_p * len(self.tables))(*[t.h for t in self.tables])
        h = C.c_void_p()
        _check(lib().krk_group_create(arr, len(self.tables), C.byref(h)), "krk_group_create")
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            lib().krk_group_destroy(self.h)
            self.h = None

    __del__ = close

    def sync(self):
        return lib().krk_group_sync(self.h)

    @staticmethod
    def _offsets(counts):
        off = np.zeros(len(counts) + 1, np.int64)
        np.cumsum(counts, out=off[1:])
        return off

    def CombinePull(self, ids, offsets, out=None, async_=False, note_rows=False):
        """ids: concatenated per-table ids; offsets: int64[n_tables + 1] -> (code, vals).
        note_rows (device ids): see KRK_NOTE_ROWS."""
        offsets = np.ascontiguousarray(offsets, dtype=np.int64)
        total = int(offsets[-1])
        if isinstance(ids, DeviceArray):
            if out is None:
                out = DeviceArray((total, self.dimension), np.float32)
        else:
            ids = np.ascontiguousarray(ids, dtype=np.uint64)
            if out is None:
                out = np.empty((total, self.dimension), np.float32)
        rc = lib().krk_group_pull(self.h, _ptr(ids), _ptr(offsets), _ptr(out),
                                  _flags(ids, out, extra=(ASYNC if async_ else 0) |
                                         (NOTE_ROWS if note_rows else 0)))
        return rc, out

    def CombinePush(self, optim, ids, offsets, grads, lr, async_=False, raw=False, as_pulled=False):
        offsets = np.ascontiguousarray(offsets, dtype=np.int64)
        if not isinstance(ids, DeviceArray):
            ids = np.ascontiguousarray(ids, dtype=np.uint64)
            grads = np.ascontiguousarray(grads, dtype=np.float32)
        gd = grads.shape[-1]
        fn = lib().krk_group_push_raw if raw else lib().krk_group_push
        return fn(self.h, C.byref(optim.raw), _ptr(ids), _ptr(offsets), _ptr(grads),
                  gd, lr, _flags(ids, grads, extra=(ASYNC if async_ else 0) |
                                 (IDS_AS_PULLED if as_pulled else 0)))

    def CombinePushRaw(self, optim, ids, offsets, grads, lr, async_=False, as_pulled=False):
        """Emitter::CombinePushSparseTable's dedup + sum fused with CombinePush: ids may repeat.
        as_pulled: ids is the unchanged device buffer of the last CombinePull(note_rows=True)."""
        return self.CombinePush(optim, ids, offsets, grads, lr, async_=async_, raw=True, as_pulled=as_pulled)


class DenseTable:
    """ps/dense_table.h"""

    def __init__(self, val):
        if isinstance(val, DeviceArray):
            self.n = val.size
            flags = DEVICE_PTRS
        else:
            val = np.ascontiguousarray(val, dtype=np.float32).ravel()
            self.n = val.size
            flags = 0
        h = C.c_void_p()
        _check(lib().krk_dense_create(_ptr(val), self.n, flags, C.byref(h)), "krk_dense_create")
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            lib().krk_dense_destroy(self.h)
            self.h = None

    __del__ = close

    def sync(self):
        return lib().krk_dense_sync(self.h)

    def save(self, path, table_id, name, shape=None):
        """Checkpoint::SaveDenseTable (checkpoint/checkpoint.cc:444-463); returns the code."""
        shape = np.ascontiguousarray(shape if shape is not None else [], dtype=np.int64)
        return lib().krk_dense_save_file(self.h, os.fsencode(path), table_id, name.encode(),
                                         shape.ctypes.data_as(C.POINTER(C.c_int64)), shape.size)

    @classmethod
    def from_file(cls, path):
        """Checkpoint::LoadDenseTable (checkpoint/checkpoint.cc:535-557)
        -> (code, table or None, table id, name, shape)"""
        h, tid, rank = C.c_void_p(), C.c_uint64(), C.c_int32(16)
        name = C.create_string_buffer(1024)
        shape = (C.c_int64 * 16)()
        rc = lib().krk_dense_load_file(os.fsencode(path), C.byref(h), C.byref(tid), name, 1024, shape,
                                       C.byref(rank))
        if rc != 0:
            return rc, None, None, None, None
        t = cls.__new__(cls)
        t.h = h
        n = C.c_int64()
        _check(lib().krk_dense_size(h, C.byref(n)), "krk_dense_size")
        t.n = n.value
        return 0, t, tid.value, name.value.decode(), list(shape[:rank.value])

    def Pull(self, out=None):
        if out is None:
            out = np.empty(self.n, np.float32)
        rc = lib().krk_dense_pull(self.h, _ptr(out), _flags(out))
        return rc, out

    def Push(self, optim, grad, lr, async_=False):
        if not isinstance(grad, DeviceArray):
            grad = np.ascontiguousarray(grad, dtype=np.float32).ravel()
        return lib().krk_dense_push(self.h, C.byref(optim.raw), _ptr(grad), grad.size, lr,
                                    _flags(grad, extra=ASYNC if async_ else 0))

    def PushCoo(self, optim, indices, values, lr):
        if not isinstance(indices, DeviceArray):
            indices = np.ascontiguousarray(indices, dtype=np.int64)
            values = np.ascontiguousarray(values, dtype=np.float32)
        return lib().krk_dense_push_coo(self.h, C.byref(optim.raw), _ptr(indices), _ptr(values),
                                        indices.size, lr, _flags(indices, values))

    def state(self, state_type):
        out = np.empty(self.n, np.float32)
        _check(lib().krk_dense_state(self.h, state_type, _ptr(out), 0), "krk_dense_state")
        return out

    @property
    def steps(self):
        s = C.c_int64()
        _check(lib().krk_dense_steps(self.h, C.byref(s)), "krk_dense_steps")
        return s.value


class DenseGroup:
    """The dense tables of one combined request (Ps::CombinePullDenseTable, ps/ps_op.cc:177-252):
    one launch serves all of them; values and gradients are the members' arrays one after the
    other."""

    def __init__(self, tables):
        self.tables = list(tables)
        arr = (C.c_void_p * len(self.tables))(*[t.h for t in self.tables])
        h = C.c_void_p()
        _check(lib().krk_dense_group_create(arr, len(self.tables), C.byref(h)), "krk_dense_group_create")
        self.h = h
        n = C.c_int64()
        _check(lib().krk_dense_group_size(h, C.byref(n)), "krk_dense_group_size")
        self.n = n.value

    def close(self):
        if getattr(self, "h", None):
            lib().krk_dense_group_destroy(self.h)
            self.h = None

    __del__ = close

    def sync(self):
        return lib().krk_dense_group_sync(self.h)

    def CombinePull(self, out=None, async_=False):
        """-> (code, the members' values concatenated)"""
        if out is None:
            out = np.empty(self.n, np.float32)
        rc = lib().krk_dense_group_pull(self.h, _ptr(out), _flags(out, extra=ASYNC if async_ else 0))
        return rc, out

    def CombinePush(self, optim, grads, lr, async_=False):
        if not isinstance(grads, DeviceArray):
            grads = np.ascontiguousarray(grads, dtype=np.float32).ravel()
        return lib().krk_dense_group_push(self.h, C.byref(optim.raw), _ptr(grads), grads.size, lr,
                                          _flags(grads, extra=ASYNC if async_ else 0))


def dedup(ids):
    """Emitter::PullSparseTableImpl's dedup -> (uids, inv)"""
    if isinstance(ids, DeviceArray):
        n = ids.size
        uids = DeviceArray(n, np.uint64)
        inv = DeviceArray(n, np.int64)
    else:
        ids = np.ascontiguousarray(ids, dtype=np.uint64)
        n = ids.size
        uids = np.empty(n, np.uint64)
        inv = np.empty(n, np.int64)
    u = C.c_int64()
    _check(lib().krk_dedup(_ptr(ids), n, _ptr(uids), _ptr(inv), C.byref(u), _flags(ids, uids, inv)),
           "krk_dedup")
    if isinstance(ids, DeviceArray):
        return uids, inv, u.value
    return uids[:u.value].copy(), inv


def route_ids(table_id, ring, ids):
    """The worker's routing of a request's (unique) ids (worker/emitter.cc:139-149).
    ring = [(hash_v, node_id), ...] in ascending hash order.
    -> (node_ids[m], counts[m], owner[n], perm[n]); device ids give device owner / perm."""
    rh = np.ascontiguousarray([h for h, _ in ring], dtype=np.uint64)
    rn = np.ascontiguousarray([n for _, n in ring], dtype=np.uint64)
    dev = isinstance(ids, DeviceArray)
    if not dev:
        ids = np.ascontiguousarray(ids, dtype=np.uint64)
    n = ids.size
    owner = DeviceArray(max(n, 1), np.uint64) if dev else np.empty(n, np.uint64)
    perm = DeviceArray(max(n, 1), np.int64) if dev else np.empty(n, np.int64)
    cap = max(len(set(int(x) for x in rn)), 1)
    node_ids = np.empty(cap, np.uint64)
    counts = np.empty(cap, np.int64)
    m = C.c_int64()
    _check(lib().krk_route_ids(int(table_id), _ptr(rh), _ptr(rn), len(ring), _ptr(ids), n, _ptr(owner),
                               _ptr(perm), _ptr(node_ids), _ptr(counts), cap, C.byref(m),
                               DEVICE_PTRS if dev else 0), "krk_route_ids")
    return node_ids[:m.value], counts[:m.value], owner, perm


DEDUP_NOALLOC_MAX = 1 << 18


def dedup_noalloc(ids, uids, inv, n_unique, n=None, stream=None):
    """krk_dedup for callers that cannot allocate: every argument is a DeviceArray the caller
    owns (n_unique: one int64), the launches go to `stream` (None = the null stream) and nothing
    is waited for. Returns the call's code."""
    n = ids.size if n is None else n
    return lib().krk_dedup_noalloc(_ptr(ids), n, _ptr(uids), _ptr(inv), _ptr(n_unique),
                                   C.c_void_p(stream) if stream else None)


def dedup_sum(ids, grads):
    """Emitter::PushSparseTable's dedup + sum (worker/emitter.cc:510-531)
    -> (uids, inv, sums[U, dim]); device inputs give device outputs plus U."""
    dev = isinstance(ids, DeviceArray)
    if not dev:
        ids = np.ascontiguousarray(ids, dtype=np.uint64)
        grads = np.ascontiguousarray(grads, dtype=np.float32)
    n = ids.size
    dim = grads.shape[-1]
    mk = (lambda shape, dt: DeviceArray(shape, dt)) if dev else (lambda shape, dt: np.empty(shape, dt))
    uids, inv, sums = mk(max(n, 1), np.uint64), mk(max(n, 1), np.int64), mk((max(n, 1), dim), np.float32)
    u = C.c_int64()
    _check(lib().krk_dedup_sum(_ptr(ids), n, _ptr(grads), dim, _ptr(uids), _ptr(inv), _ptr(sums), C.byref(u),
                               _flags(ids, grads, uids)), "krk_dedup_sum")
    if dev:
        return uids, inv, sums, u.value
    return uids[:u.value].copy(), inv[:n], sums[:u.value].copy()


def expand_rows(rows, inv):
    """The re-expansion of worker/emitter.cc:162-182: out[p] = rows[inv[p]]; returns (code, out)."""
    dev = isinstance(rows, DeviceArray)
    if not dev:
        rows = np.ascontiguousarray(rows, dtype=np.float32)
        inv = np.ascontiguousarray(inv, dtype=np.int64)
    n, dim = inv.size, rows.shape[-1]
    out = DeviceArray((n, dim), np.float32) if dev else np.empty((n, dim), np.float32)
    rc = lib().krk_expand_rows(_ptr(rows), rows.shape[0], _ptr(inv), n, dim, _ptr(out), _flags(rows, inv, out))
    return rc, out


class DenseBag:
    """worker/dct_emitter.h DCTEmitter::DenseBag: error-feedback threshold codec state."""

    def __init__(self, n):
        self.n = int(n)
        h = C.c_void_p()
        _check(lib().krk_dct_create(self.n, C.byref(h)), "krk_dct_create")
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            lib().krk_dct_destroy(self.h)
            self.h = None

    __del__ = close

    def MaybeToCoo(self, life_span, eta, grad, idx=None, val=None):
        """-> (indices, values) or (None, None) when the gradient is to be sent dense."""
        dev = isinstance(grad, DeviceArray)
        if not dev:
            grad = np.ascontiguousarray(grad, dtype=np.float32).ravel()
        if idx is None:
            idx = DeviceArray(self.n, np.int64) if dev else np.empty(self.n, np.int64)
            val = DeviceArray(self.n, np.float32) if dev else np.empty(self.n, np.float32)
        nnz = C.c_int64()
        _check(lib().krk_dct_compress(self.h, _ptr(grad), life_span, eta, _ptr(idx), _ptr(val),
                                      idx.size, C.byref(nnz), _flags(grad, idx, val)),
               "krk_dct_compress")
        if nnz.value < 0:
            return None, None
        if dev:
            return idx, val, nnz.value
        return idx[:nnz.value].copy(), val[:nnz.value].copy()

    @property
    def tau(self):
        t = C.c_float()
        _check(lib().krk_dct_tau(self.h, C.byref(t)), "krk_dct_tau")
        return t.value

    @property
    def step(self):
        s = C.c_uint64()
        _check(lib().krk_dct_step(self.h, C.byref(s)), "krk_dct_step")
        return s.value

    @property
    def residual(self):
        out = np.empty(self.n, np.float32)
        _check(lib().krk_dct_residual(self.h, _ptr(out), 0), "krk_dct_residual")
        return out


def coo_to_dense(indices, values, n):
    """CooTensorImpl::ToDense for a 1-D shape."""
    if isinstance(indices, DeviceArray):
        out = DeviceArray(n, np.float32)
        nnz = indices.size
    else:
        indices = np.ascontiguousarray(indices, dtype=np.int64)
        values = np.ascontiguousarray(values, dtype=np.float32)
        out = np.empty(n, np.float32)
        nnz = indices.size
    _check(lib().krk_coo_to_dense(_ptr(indices), _ptr(values), nnz, _ptr(out), n,
                                  _flags(indices, values, out)), "krk_coo_to_dense")
    return out


class Event:
    def __init__(self):
        h = C.c_void_p()
        _check(lib().krk_event_create(C.byref(h)), "krk_event_create")
        self.h = h

    def record(self, obj):
        # obj None: the null stream, where the calls that own no object (dedup, dct2) run
        _check(lib().krk_event_record(self.h, obj.h if obj is not None else None), "krk_event_record")

    def wait(self, obj):
        # what is enqueued on obj's stream from now on starts after this (already recorded) event
        _check(lib().krk_event_wait(self.h, obj.h if obj is not None else None), "krk_event_wait")

    def elapsed_ms(self, stop):
        ms = C.c_float()
        _check(lib().krk_event_elapsed_ms(self.h, stop.h, C.byref(ms)), "krk_event_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            if getattr(self, "h", None):
                lib().krk_event_destroy(self.h)
                self.h = None
        except Exception:
            pass
