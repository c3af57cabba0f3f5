"""ctypes binding of librp_hip.so — the C ABI declared in include/rp_hip.h.

Nothing here computes: it loads the shared library, declares argument types and
offers a small device-buffer helper so that Python callers (tests, bench, the
host-side tensor layer) can hand raw device pointers to the entry points.
The library is required; a missing build raises instead of falling back.
"""
import ctypes
import os

import numpy as np

F32, F64, F16, BF16 = 0, 1, 2, 3          # reference core/tensor.h:7-13
DTYPE_SIZE = {F32: 4, F64: 8, F16: 2, BF16: 2}
NP_STORAGE = {F32: np.float32, F64: np.float64, F16: np.uint16, BF16: np.uint16}

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librp_hip.so")

_vp, _i, _ll, _sz, _d = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_size_t, ctypes.c_double
_ip = ctypes.POINTER(ctypes.c_int)

# name -> (restype, argtypes); one entry per function declared in include/rp_hip.h
SIGNATURES = {
    "rp_hip_device_count": (_i, [_ip]),
    "rp_hip_set_device": (_i, [_i]),
    "rp_hip_get_device": (_i, [_ip]),
    "rp_hip_malloc": (_i, [ctypes.POINTER(_vp), _sz]),
    "rp_hip_free": (_i, [_vp]),
    "rp_hip_empty_cache": (_i, []),
    "rp_hip_memory_stats": (_i, [ctypes.POINTER(_ll)] * 4),
    "rp_hip_memset": (_i, [_vp, _i, _sz]),
    "rp_hip_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "rp_hip_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "rp_hip_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "rp_hip_synchronize": (_i, []),
    "rp_hip_last_error": (ctypes.c_char_p, []),
    "rp_hip_set_stream": (_i, [_vp]),
    "rp_hip_get_stream": (_vp, []),
    "rp_hip_stream_create": (_i, [ctypes.POINTER(_vp)]),
    "rp_hip_stream_destroy": (_i, [_vp]),
    "rp_hip_stream_synchronize": (_i, []),
    "rp_hip_graph_capture_begin": (_i, []),
    "rp_hip_graph_capture_end": (_i, [ctypes.POINTER(_vp)]),
    "rp_hip_graph_launch": (_i, [_vp]),
    "rp_hip_graph_destroy": (_i, [_vp]),
    "rp_hip_event_create": (_i, [ctypes.POINTER(_vp)]),
    "rp_hip_event_record": (_i, [_vp]),
    "rp_hip_event_synchronize": (_i, [_vp]),
    "rp_hip_event_elapsed_ms": (_i, [ctypes.POINTER(ctypes.c_float), _vp, _vp]),
    "rp_hip_event_destroy": (_i, [_vp]),
    "matmul_kernel_device": (_i, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "rp_hip_gemm_strided_batched": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i] + [_ll] * 9 + [_i, _i]),
    "rp_hip_gemm_strided_batched_noalloc": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i] + [_ll] * 9 + [_i, _i]),
    "rp_hip_gemm_kernel_name": (ctypes.c_char_p, [_i, _i, _i, _i] + [_ll] * 6 + [_i]),
    "rp_hip_last_gemm_kernel": (ctypes.c_char_p, []),
    "add_kernel_device": (_i, [_vp, _vp, _vp, _sz, _i]),
    "add_strided_kernel_device": (_i, [_vp, _vp, _vp, _i, _ip, _ip, _ip, _sz, _i]),
    "mul_scalar_kernel_device": (_i, [_vp, _vp, _vp, _sz, _i]),
    "relu_kernel_device": (_i, [_vp, _vp, _sz, _i]),
    "backwards_relu_device": (_i, [_vp, _vp, _vp, _sz, _i]),
    "softmax_kernel_device": (_i, [_vp, _vp, _sz, _sz, _sz, _i]),
    "log_softmax_kernel_device": (_i, [_vp, _vp, _sz, _sz, _sz, _i]),
    "backwards_softmax_device": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _i]),
    "rp_hip_scaled_softmax": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _i]),
    "rp_hip_backwards_scaled_softmax": (_i, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _i]),
    "rp_hip_mul_scalar_deferred": (_i, [_vp, _vp, _vp, _sz, _i]),
    "rp_hip_take_deferred": (_i, [_vp, ctypes.POINTER(_vp), ctypes.POINTER(_d)]),
    "backwards_log_softmax_device": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _i]),
    "contiguous_copy_kernel_device": (_i, [_vp, _vp, _i, _ip, _ip, _sz, _i]),
    "sum_all_kernel_device": (_i, [_vp, _vp, _sz, _i]),
    "mean_all_kernel_device": (_i, [_vp, _vp, _sz, _i]),
    "sum_dim_kernel_device": (_i, [_vp, _vp, _sz, _sz, _sz, _i]),
    "rp_hip_fill": (_i, [_vp, _d, _sz, _i]),
    "rp_hip_convert": (_i, [_vp, _i, _vp, _i, _sz]),
    "rp_hip_reduce_rows": (_i, [_vp, _vp, _i, _i, _i, _i]),
    "rp_hip_linear_backward": (_i, [_vp] * 6 + [_i] * 3 + [_ll] * 8 + [_i] * 4),
    "rp_hip_cross_entropy_mean": (_i, [_vp, _vp, _vp, _vp, _i, _i, _d, _i]),
    "rp_hip_cross_entropy_backward": (_i, [_vp, _vp, _vp, _i, _i, _vp, _i]),
    "rp_hip_cross_entropy_forward": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "rp_hip_cross_entropy_grad": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _i]),
    "rp_hip_fill_scaled": (_i, [_vp, _vp, _d, _sz, _i]),
    "im2col_kernel_device": (_i, [_vp, _vp] + [_i] * 14),
    "col2im_kernel_device": (_i, [_vp, _vp] + [_i] * 14),
    "rp_hip_im2col_batched": (_i, [_vp, _vp] + [_i] * 15),
    "rp_hip_col2im_batched": (_i, [_vp, _vp] + [_i] * 16),
    "rp_hip_channel_bias_add": (_i, [_vp, _vp, _i, _i, _i, _i]),
    "rp_hip_conv2d_same_supported": (_i, [_i] * 6),
    "rp_hip_conv2d_same_forward": (_i, [_vp] * 4 + [_i] * 8),
    "rp_hip_conv2d_same_backward_input": (_i, [_vp] * 3 + [_i] * 8),
    "rp_hip_conv2d_same_backward": (_i, [_vp] * 5 + [_i] * 8),
    "rp_hip_channel_sums": (_i, [_vp, _vp, _i, _i, _i, _i, _i]),
    "rp_hip_lstm_cell_forward": (_i, [_vp] * 6 + [_ll, _i, _i, _i]),
    "rp_hip_lstm_cell_backward": (_i, [_vp] * 6 + [_ll, _i, _i, _i]),
    "rp_hip_gru_cell_forward": (_i, [_vp] * 5 + [_ll, _i, _i, _i]),
    "rp_hip_gru_cell_backward": (_i, [_vp] * 7 + [_ll, _i, _i, _i]),
    "rp_hip_scatter_strided": (_i, [_vp, _vp, _i, _ip, ctypes.POINTER(ctypes.c_longlong), _sz, _i]),
    "rp_hip_attention_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i] + [_ll] * 8 + [_d, _i]),
    "rp_hip_attention_backward": (_i, [_vp] * 9 + [_i] * 4 + [_ll] * 10 + [_d, _i]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m recpulse_amd.build` "
                               "(there is no CPU fallback)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


class RpHipError(RuntimeError):
    pass


def check(rc, what):
    if rc != 0:
        msg = lib().rp_hip_last_error()
        raise RpHipError(f"{what} failed: {msg.decode() if msg else 'unknown error'}")


def device_count():
    n = ctypes.c_int(0)
    check(lib().rp_hip_device_count(ctypes.byref(n)), "rp_hip_device_count")
    return n.value


def synchronize():
    check(lib().rp_hip_synchronize(), "rp_hip_synchronize")


class DeviceBuffer:
    """A raw device allocation from the library's pool."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = _vp()
        check(lib().rp_hip_malloc(ctypes.byref(p), max(self.nbytes, 1)), "rp_hip_malloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        check(lib().rp_hip_memcpy_h2d(buf.ptr, arr.ctypes.data_as(_vp), arr.nbytes), "rp_hip_memcpy_h2d")
        return buf

    def to_numpy(self, np_dtype, shape):
        out = np.empty(shape, dtype=np_dtype)
        assert out.nbytes <= self.nbytes
        check(lib().rp_hip_memcpy_d2h(out.ctypes.data_as(_vp), self.ptr, out.nbytes), "rp_hip_memcpy_d2h")
        return out

    def at(self, byte_offset):
        return self.ptr + int(byte_offset)

    def free(self):
        if self.ptr:
            lib().rp_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def gemm(c_ptr, a_ptr, b_ptr, bias_ptr, batch, m, k, n, a_st, b_st, c_st, accumulate, dtype):
    """rp_hip_gemm_strided_batched; *_st = (batch, row, col) strides in elements."""
    check(lib().rp_hip_gemm_strided_batched(c_ptr, a_ptr, b_ptr, bias_ptr, batch, m, k, n,
                                            *[int(s) for s in a_st], *[int(s) for s in b_st], *[int(s) for s in c_st],
                                            int(bool(accumulate)), dtype), "rp_hip_gemm_strided_batched")


def last_gemm_kernel():
    """Kernel that the calling thread's most recent GEMM call dispatched (reflects bias, accumulation and pointers)."""
    return lib().rp_hip_last_gemm_kernel().decode()


def gemm_kernel_name(batch, m, k, n, a_rc, b_rc, c_rc, dtype):
    return lib().rp_hip_gemm_kernel_name(batch, m, k, n, *[int(s) for s in a_rc], *[int(s) for s in b_rc],
                                         *[int(s) for s in c_rc], dtype).decode()


class Stream:
    """A created stream; `with stream:` makes it the calling thread's current stream."""

    def __init__(self):
        p = _vp()
        check(lib().rp_hip_stream_create(ctypes.byref(p)), "rp_hip_stream_create")
        self.ptr = p.value
        self._prev = None

    def __enter__(self):
        self._prev = lib().rp_hip_get_stream()
        lib().rp_hip_set_stream(self.ptr)
        return self

    def __exit__(self, *exc):
        lib().rp_hip_set_stream(self._prev)
        return False

    def __del__(self):
        try:
            if self.ptr:
                lib().rp_hip_stream_destroy(self.ptr)
                self.ptr = None
        except Exception:
            pass


class Graph:
    """Capture of the calls made inside `with Graph.capture() as g:` on the current (created) stream."""

    def __init__(self):
        self.ptr = None

    @classmethod
    def capture(cls):
        return _GraphCapture(cls())

    def launch(self):
        check(lib().rp_hip_graph_launch(self.ptr), "rp_hip_graph_launch")

    def __del__(self):
        try:
            if self.ptr:
                lib().rp_hip_graph_destroy(self.ptr)
                self.ptr = None
        except Exception:
            pass


class _GraphCapture:
    def __init__(self, graph):
        self.graph = graph

    def __enter__(self):
        check(lib().rp_hip_graph_capture_begin(), "rp_hip_graph_capture_begin")
        return self.graph

    def __exit__(self, exc_type, exc, tb):
        p = _vp()
        rc = lib().rp_hip_graph_capture_end(ctypes.byref(p))
        if exc_type is None:
            check(rc, "rp_hip_graph_capture_end")
            self.graph.ptr = p.value
        return False


class Event:
    def __init__(self):
        p = _vp()
        check(lib().rp_hip_event_create(ctypes.byref(p)), "rp_hip_event_create")
        self.ptr = p.value

    def record(self):
        check(lib().rp_hip_event_record(self.ptr), "rp_hip_event_record")

    def synchronize(self):
        check(lib().rp_hip_event_synchronize(self.ptr), "rp_hip_event_synchronize")

    def elapsed_ms(self, stop):
        ms = ctypes.c_float(0)
        check(lib().rp_hip_event_elapsed_ms(ctypes.byref(ms), self.ptr, stop.ptr), "rp_hip_event_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                lib().rp_hip_event_destroy(self.ptr)
                self.ptr = None
        except Exception:
            pass
