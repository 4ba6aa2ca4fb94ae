"""Blockwise orthonormal DCT-II on the GPU (no reference counterpart; see include/kraken_hip.h)."""
import numpy as np

from . import api

BLOCK = 256


def forward(x, keep=BLOCK, out=None):
    """x: n floats (n % 256 == 0) -> coefficients [n / 256, keep]"""
    if isinstance(x, api.DeviceArray):
        n = x.size
        if out is None:
            out = api.DeviceArray((n // BLOCK, keep), np.float32)
    else:
        x = np.ascontiguousarray(x, dtype=np.float32).ravel()
        n = x.size
        if out is None:
            out = np.empty((n // BLOCK, keep), np.float32)
    api._check(api.lib().krk_dct2_forward(api._ptr(x), api._ptr(out), n, keep, api._flags(x, out)),
               "krk_dct2_forward")
    return out


def inverse(coeff, n, keep=BLOCK, out=None):
    """coefficients [n / 256, keep] -> n floats"""
    if isinstance(coeff, api.DeviceArray):
        if out is None:
            out = api.DeviceArray(n, np.float32)
    else:
        coeff = np.ascontiguousarray(coeff, dtype=np.float32)
        if out is None:
            out = np.empty(n, np.float32)
    api._check(api.lib().krk_dct2_inverse(api._ptr(coeff), api._ptr(out), n, keep, api._flags(coeff, out)),
               "krk_dct2_inverse")
    return out
