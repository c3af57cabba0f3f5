"""Helpers for the GPU parity tests: numpy storage arrays in, C-ABI calls, numpy out."""
import ctypes

import numpy as np

import oracle
from recpulse_amd import capi

F32, F64, F16, BF16 = capi.F32, capi.F64, capi.F16, capi.BF16
ALL = [F32, F64, F16, BF16]
NAMES = {F32: "f32", F64: "f64", F16: "f16", BF16: "bf16"}


def tol(dtype, k):
    """Normwise relative error bounds of the parity target."""
    return {F32: 1e-5 * np.sqrt(k), F64: 1e-12, F16: 2e-2, BF16: 2e-2}[dtype]


def rand_storage(rng, shape, dtype, dist="normal"):
    x = rng.normal(0, 1, shape) if dist == "normal" else rng.uniform(-1, 1, shape)
    return oracle.to_storage(x, dtype)


def elem_strides(arr):
    return [s // arr.itemsize for s in arr.strides]


def device_gemm(a_view, b_view, dtype, bias=None, c_init=None, accumulate=False):
    """C = A @ B (+bias)(+C) for numpy VIEWS of storage arrays (2-D or 3-D with a leading batch).

    The views' own strides are passed to the entry point; only their base
    buffers are uploaded, so transposed / sliced views are exercised without copies.
    """
    a_base = a_view.base if a_view.base is not None else a_view
    b_base = b_view.base if b_view.base is not None else b_view
    while a_base.base is not None:
        a_base = a_base.base
    while b_base.base is not None:
        b_base = b_base.base
    es = a_view.itemsize

    def off(view, base):
        return view.__array_interface__["data"][0] - base.__array_interface__["data"][0]

    if a_view.ndim == 2:
        batch, (m, k), n = 1, a_view.shape, b_view.shape[1]
        a_st = (0,) + tuple(elem_strides(a_view)); b_st = (0,) + tuple(elem_strides(b_view))
    else:
        batch, m, k = a_view.shape; n = b_view.shape[2]
        a_st = tuple(elem_strides(a_view)); b_st = tuple(elem_strides(b_view))
    da = capi.DeviceBuffer.from_numpy(np.ascontiguousarray(a_base).reshape(-1) if a_base.flags.c_contiguous else a_base)
    db = capi.DeviceBuffer.from_numpy(np.ascontiguousarray(b_base).reshape(-1) if b_base.flags.c_contiguous else b_base)
    c_shape = (m, n) if a_view.ndim == 2 else (batch, m, n)
    c0 = np.zeros(c_shape, dtype=capi.NP_STORAGE[dtype]) if c_init is None else np.ascontiguousarray(c_init)
    dc = capi.DeviceBuffer.from_numpy(c0)
    dbias = capi.DeviceBuffer.from_numpy(bias) if bias is not None else None
    capi.gemm(dc.ptr, da.at(off(a_view, a_base)), db.at(off(b_view, b_base)), dbias.ptr if dbias else None,
              batch, m, k, n, a_st, b_st, (m * n, n, 1), accumulate, dtype)
    capi.synchronize()
    out = dc.to_numpy(capi.NP_STORAGE[dtype], c_shape)
    for d in (da, db, dc, dbias):
        if d is not None:
            d.free()
    return out


def oracle_gemm(a_view, b_view, dtype, bias=None, c_init=None, accumulate=False):
    """The same product through the CPU oracle (densify, 2-D matmul per batch, op chain epilogue)."""
    if a_view.ndim == 2:
        a_view = a_view[None]; b_view = b_view[None]
        c_init = None if c_init is None else c_init[None]
        squeeze = True
    else:
        squeeze = False
    outs = []
    for z in range(a_view.shape[0]):
        y = oracle.matmul(np.ascontiguousarray(a_view[z]), np.ascontiguousarray(b_view[z]), dtype)
        if bias is not None:
            y = oracle.bias_add(y, bias, dtype)
        if accumulate:
            y = oracle.add(np.ascontiguousarray(c_init[z]), y, dtype)
        outs.append(y)
    out = np.stack(outs)
    return out[0] if squeeze else out


def f64_gemm(a_view, b_view, dtype, bias=None, c_init=None, accumulate=False):
    y = np.matmul(oracle.to_f64(a_view, dtype), oracle.to_f64(b_view, dtype))
    if bias is not None:
        y = y + oracle.to_f64(bias, dtype)
    if accumulate:
        y = y + oracle.to_f64(c_init, dtype)
    return y


class Dev:
    """Tiny wrapper: a device copy of a numpy storage array."""

    def __init__(self, arr, dtype):
        self.shape = tuple(arr.shape); self.dtype = dtype
        self.buf = capi.DeviceBuffer.from_numpy(np.ascontiguousarray(arr))

    @classmethod
    def empty(cls, shape, dtype):
        self = cls.__new__(cls)
        self.shape = tuple(shape); self.dtype = dtype
        self.buf = capi.DeviceBuffer(int(np.prod(shape)) * capi.DTYPE_SIZE[dtype])
        return self

    @property
    def ptr(self):
        return self.buf.ptr

    @property
    def size(self):
        return int(np.prod(self.shape))

    def numpy(self):
        capi.synchronize()
        return self.buf.to_numpy(capi.NP_STORAGE[self.dtype], self.shape)


def scalar_arg(value, dtype):
    return ctypes.byref(ctypes.c_double(value)) if dtype == F64 else ctypes.byref(ctypes.c_float(value))
