"""ctypes front-end of the CPU oracle — TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Loads ``oracle/librp_oracle.so`` (this repository's restatement of the RecPulse
reference's CPU arithmetic, ``rp_oracle.c``) and, when it has been built,
``oracle/_ref/libref_host.so`` (the reference's own host kernels compiled
unchanged).  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package; the shipped
library never does.

16-bit tensors travel as ``numpy.uint16`` bit patterns: numpy has no bfloat16,
and the reference's narrowing (round half away from zero, reference
core/half_precision.h:50-97) differs from numpy's float16 casts on ties.
"""
import ctypes
import os
import subprocess

import numpy as np

F32, F64, F16, BF16 = 0, 1, 2, 3          # reference core/tensor.h:7-13
DTYPE_NAMES = {F32: "float32", F64: "float64", F16: "float16", BF16: "bfloat16"}
NP_STORAGE = {F32: np.float32, F64: np.float64, F16: np.uint16, BF16: np.uint16}

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librp_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_host.so")


def build():
    """Compile the oracle (and oracle/_ref when the reference tree is mounted)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "all"])


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()
_vp, _i, _ll, _sz, _d = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_size_t, ctypes.c_double
_ip = ctypes.POINTER(ctypes.c_int)
_llp = ctypes.POINTER(ctypes.c_longlong)


def _sig(name, res, *args):
    fn = getattr(_lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


_matmul = _sig("orc_matmul", _i, _vp, _vp, _vp, _i, _i, _i, _i)
_gemm = _sig("orc_gemm_strided_batched", _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i,
             _ll, _ll, _ll, _ll, _ll, _ll, _ll, _ll, _ll, _i, _i)
_add = _sig("orc_add", _i, _vp, _vp, _vp, _sz, _i)
_add_strided = _sig("orc_add_strided", _i, _vp, _vp, _vp, _i, _ip, _ip, _ip, _sz, _i)
_mul_scalar = _sig("orc_mul_scalar", _i, _vp, _vp, _d, _sz, _i)
_relu = _sig("orc_relu", _i, _vp, _vp, _sz, _i)
_bw_relu = _sig("orc_backwards_relu", _i, _vp, _vp, _vp, _sz, _i)
_softmax = _sig("orc_softmax", _i, _vp, _vp, _sz, _sz, _sz, _i)
_log_softmax = _sig("orc_log_softmax", _i, _vp, _vp, _sz, _sz, _sz, _i)
_bw_softmax = _sig("orc_backwards_softmax", _i, _vp, _vp, _vp, _sz, _sz, _sz, _i)
_sum_all = _sig("orc_sum_all", _i, _vp, _vp, _sz, _i)
_reduce_rows = _sig("orc_reduce_rows", _i, _vp, _vp, _i, _i, _i)
_contig = _sig("orc_contiguous_copy", _i, _vp, _vp, _i, _ip, _llp, _i)
_ce = _sig("orc_cross_entropy_mean", _i, _vp, _vp, _vp, _ip, _i, _i, _d, _i)
_ce_any = _sig("orc_cross_entropy", _i, _vp, _vp, _vp, _ip, _i, _i, _i, _i, _vp, _i)
_bw_log_softmax = _sig("orc_backwards_log_softmax", _i, _vp, _vp, _vp, _sz, _sz, _sz, _i)
_sigmoid = _sig("orc_sigmoid", _i, _vp, _vp, _sz, _i)
_tanh = _sig("orc_tanh", _i, _vp, _vp, _sz, _i)
_im2col = _sig("orc_im2col", _i, _vp, _vp, *([_i] * 14))
_col2im = _sig("orc_col2im", _i, _vp, _vp, *([_i] * 14))
_widen = _sig("orc_widen", None, _vp, _vp, _sz, _i)
_narrow = _sig("orc_narrow", None, _vp, _vp, _sz, _i)


def _ptr(a):
    return a.ctypes.data_as(_vp)


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed")


# ---------------------------------------------------------------------------
# dtype helpers
# ---------------------------------------------------------------------------
def widen(bits, dtype):
    """uint16 bit patterns (fp16 or bf16) -> float32, exact."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    _widen(_ptr(bits), _ptr(out), bits.size, dtype)
    return out


def narrow(x, dtype):
    """float32 -> uint16 bit patterns with the reference's rounding."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    _narrow(_ptr(x), _ptr(out), x.size, dtype)
    return out


def to_storage(x64, dtype):
    """float64 array -> the storage array of `dtype` (cast once, reference rounding for 16-bit)."""
    if dtype == F64:
        return np.ascontiguousarray(x64, dtype=np.float64)
    x32 = np.ascontiguousarray(x64, dtype=np.float32)
    if dtype == F32:
        return x32
    return narrow(x32, dtype)


def to_f64(x, dtype):
    """storage array of `dtype` -> float64 values, exact."""
    if dtype in (F16, BF16):
        return widen(x, dtype).astype(np.float64)
    return np.asarray(x, dtype=np.float64)


# ---------------------------------------------------------------------------
# the restated ops (all take and return storage arrays of `dtype`)
# ---------------------------------------------------------------------------
def matmul(a, b, dtype):
    a = np.ascontiguousarray(a); b = np.ascontiguousarray(b)
    m, k = a.shape; k2, n = b.shape
    assert k == k2
    c = np.empty((m, n), dtype=NP_STORAGE[dtype])
    _check(_matmul(_ptr(c), _ptr(a), _ptr(b), m, k, n, dtype), "matmul")
    return c


def gemm_strided_batched(c_buf, a_buf, b_buf, bias, batch, m, k, n, a_st, b_st, c_st, accumulate, dtype):
    """In-place on the flat storage buffer `c_buf`; *_st = (batch, row, col) strides in elements."""
    _check(_gemm(_ptr(c_buf), _ptr(a_buf), _ptr(b_buf), _ptr(bias) if bias is not None else None,
                 batch, m, k, n, *a_st, *b_st, *c_st, int(bool(accumulate)), dtype), "gemm_strided_batched")
    return c_buf


def add(x1, x2, dtype):
    x1 = np.ascontiguousarray(x1); x2 = np.ascontiguousarray(x2)
    out = np.empty_like(x1)
    _check(_add(_ptr(out), _ptr(x1), _ptr(x2), x1.size, dtype), "add")
    return out


def add_strided(x1, x2, out_shape, s1, s2, dtype):
    out = np.empty(out_shape, dtype=NP_STORAGE[dtype])
    nd = len(out_shape)
    arr = lambda v: (ctypes.c_int * nd)(*[int(t) for t in v])
    _check(_add_strided(_ptr(out), _ptr(x1), _ptr(x2), nd, arr(out_shape), arr(s1), arr(s2), out.size, dtype),
           "add_strided")
    return out


def bias_add(y, bias, dtype):
    """[m, n] + [n] the way Linear does it (reference recpulse/module.py:110-114)."""
    m, n = y.shape
    return add_strided(np.ascontiguousarray(y), np.ascontiguousarray(bias), (m, n), (n, 1), (0, 1), dtype)


def mul_scalar(x, scalar, dtype):
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    _check(_mul_scalar(_ptr(out), _ptr(x), float(scalar), x.size, dtype), "mul_scalar")
    return out


def relu(x, dtype):
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    _check(_relu(_ptr(out), _ptr(x), x.size, dtype), "relu")
    return out


def backwards_relu(grad_c, x, dtype):
    grad_c = np.ascontiguousarray(grad_c); x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    _check(_bw_relu(_ptr(grad_c), _ptr(x), _ptr(out), x.size, dtype), "backwards_relu")
    return out


def _split(shape, dim):
    dim = dim % len(shape)
    outer = int(np.prod(shape[:dim], dtype=np.int64)) if dim > 0 else 1
    inner = int(np.prod(shape[dim + 1:], dtype=np.int64)) if dim + 1 < len(shape) else 1
    return outer, int(shape[dim]), inner


def softmax(x, dtype, dim=-1, log=False):
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    o, d, i = _split(x.shape, dim)
    _check((_log_softmax if log else _softmax)(_ptr(out), _ptr(x), o, d, i, dtype), "softmax")
    return out


def backwards_softmax(grad_c, y, dtype, dim=-1):
    grad_c = np.ascontiguousarray(grad_c); y = np.ascontiguousarray(y)
    out = np.empty_like(y)
    o, d, i = _split(y.shape, dim)
    _check(_bw_softmax(_ptr(grad_c), _ptr(y), _ptr(out), o, d, i, dtype), "backwards_softmax")
    return out


def sum_all(x, dtype):
    x = np.ascontiguousarray(x)
    out = np.empty((1,), dtype=NP_STORAGE[dtype])
    _check(_sum_all(_ptr(out), _ptr(x), x.size, dtype), "sum_all")
    return out


def reduce_rows(grad, dtype):
    """Bias gradient of Linear: [rows, cols] -> [cols] (reference ops/ops.c:6970-7101)."""
    grad = np.ascontiguousarray(grad)
    rows, cols = grad.shape
    out = np.empty((cols,), dtype=NP_STORAGE[dtype])
    _check(_reduce_rows(_ptr(out), _ptr(grad), rows, cols, dtype), "reduce_rows")
    return out


def contiguous_copy(buf, shape, strides, dtype, offset=0):
    """Gather the view (shape, strides in elements, offset in elements) of flat `buf`."""
    nd = len(shape)
    out = np.empty(shape, dtype=NP_STORAGE[dtype])
    base = buf.reshape(-1)[offset:]
    _check(_contig(_ptr(out), _ptr(base), nd, (ctypes.c_int * nd)(*[int(s) for s in shape]),
                   (ctypes.c_longlong * nd)(*[int(s) for s in strides]), dtype), "contiguous_copy")
    return out


def cross_entropy_mean(logits, targets, dtype, upstream=1.0):
    """Returns (loss scalar, dlogits) for mean cross-entropy on logits; f32/f64 only."""
    logits = np.ascontiguousarray(logits)
    b, c = logits.shape
    t = np.ascontiguousarray(targets, dtype=np.int32)
    loss = np.empty((1,), dtype=NP_STORAGE[dtype])
    grad = np.empty_like(logits)
    _check(_ce(_ptr(loss), _ptr(grad), _ptr(logits), t.ctypes.data_as(_ip), b, c, float(upstream), dtype),
           "cross_entropy_mean")
    return loss, grad


REDUCTIONS = {"none": 0, "mean": 1, "sum": 2}          # reference ops/ops.h:109-111


def cross_entropy(x, targets, dtype, reduction="mean", from_logits=True, upstream=None):
    """reference ops/ops.c:5545-5643 with every reduction, on logits or on probabilities (from_logits=False).
    Returns (loss, dx): loss has shape [batch] for 'none' and [1] otherwise; dx is None unless `upstream` (the
    gradient of the loss: [batch] for 'none', one element otherwise) is given.  f32 / f64 only."""
    x = np.ascontiguousarray(x)
    b, c = x.shape
    t = np.ascontiguousarray(targets, dtype=np.int32)
    red = REDUCTIONS[reduction]
    loss = np.empty((b if red == 0 else 1,), dtype=NP_STORAGE[dtype])
    grad, up = None, None
    if upstream is not None:
        grad = np.empty_like(x)
        up = np.ascontiguousarray(np.broadcast_to(np.asarray(upstream, dtype=NP_STORAGE[dtype]).reshape(-1), (b if red == 0 else 1,)))
    _check(_ce_any(_ptr(loss), _ptr(grad) if grad is not None else None, _ptr(x), t.ctypes.data_as(_ip), b, c, red, int(bool(from_logits)),
                   _ptr(up) if up is not None else None, dtype), "cross_entropy")
    return loss, grad


def backwards_log_softmax(grad_c, y, dtype, dim=-1):
    """reference ops/grad_host.c:1428-1500: y is the log-softmax output."""
    grad_c = np.ascontiguousarray(grad_c); y = np.ascontiguousarray(y)
    out = np.empty_like(y)
    o, d, i = _split(y.shape, dim)
    _check(_bw_log_softmax(_ptr(grad_c), _ptr(y), _ptr(out), o, d, i, dtype), "backwards_log_softmax")
    return out


# ---------------------------------------------------------------------------
# compositions used by the parity tests (pure chaining of the ops above, in the
# order the reference's autograd runs them)
# ---------------------------------------------------------------------------
def linear_forward(x, w, bias, dtype):
    """reference recpulse/module.py:110-114."""
    y = matmul(x, w, dtype)
    return bias_add(y, bias, dtype) if bias is not None else y


def matmul_backward(a, b, dc, dtype):
    """reference ops/ops.c:6759-6814: dA = dC @ B^T, dB = A^T @ dC on densified transposes."""
    da = matmul(dc, np.ascontiguousarray(b.T), dtype)
    db = matmul(np.ascontiguousarray(a.T), dc, dtype)
    return da, db


def mlp_step(x, weights, biases, targets, dtype=F32):
    """Config-2 style MLP (Linear+ReLU ... Linear, mean cross-entropy) forward and backward.

    Returns dict(loss, logits, dW=[...], db=[...], dX).  Order of operations follows
    the reference autograd: Linear = matmul then broadcasting add; backward of add
    hands dY to the matmul and reduces it over rows for the bias.
    """
    acts, pre = [x], []
    h = x
    nl = len(weights)
    for li in range(nl):
        z = linear_forward(h, weights[li], biases[li], dtype)
        pre.append(z)
        h = relu(z, dtype) if li + 1 < nl else z
        acts.append(h)
    loss, g = cross_entropy_mean(h, targets, dtype)
    dws, dbs = [None] * nl, [None] * nl
    for li in reversed(range(nl)):
        if li + 1 < nl:
            g = backwards_relu(g, pre[li], dtype)
        dbs[li] = reduce_rows(g, dtype) if biases[li] is not None else None
        da, dw = matmul_backward(acts[li], weights[li], g, dtype)
        dws[li] = dw
        g = da
    return {"loss": loss, "logits": h, "dW": dws, "db": dbs, "dX": g}


def attention(q, k, v, dtype, scale=0.125, d_out=None):
    """Config-4 attention for ONE (batch, head) slice: S=q@k^T, P=softmax(S*scale), O=P@v.

    With d_out (dO) also returns dQ, dK, dV following the reference autograd chain
    matmul -> mul_scalar -> softmax -> matmul.
    """
    kt = np.ascontiguousarray(k.T)
    s = matmul(q, kt, dtype)
    ss = mul_scalar(s, scale, dtype)
    p = softmax(ss, dtype)
    o = matmul(p, v, dtype)
    if d_out is None:
        return {"S": s, "P": p, "O": o}
    dp, dv = matmul_backward(p, v, d_out, dtype)
    dss = backwards_softmax(dp, p, dtype)
    ds = mul_scalar(dss, scale, dtype)
    dq, dkt = matmul_backward(q, kt, ds, dtype)
    dk = np.ascontiguousarray(dkt.T)       # permute backward = inverse permutation (reference ops/ops.c:7977-8014)
    return {"S": s, "P": p, "O": o, "dQ": dq, "dK": dk, "dV": dv}


def conv_out_size(size, k, stride, pad, dilation):
    """reference ops/ops.c:4740-4741."""
    return (size + 2 * pad - dilation * (k - 1) - 1) // stride + 1


def im2col(im, kernel, stride, pad, dilation, dtype):
    """im [C, H, W] -> col [C*kH*kW, oH*oW] (reference functional/functional.c:855-883)."""
    im = np.ascontiguousarray(im)
    C, H, W = im.shape
    (kH, kW), (sh, sw), (ph, pw), (dh, dw) = kernel, stride, pad, dilation
    oH, oW = conv_out_size(H, kH, sh, ph, dh), conv_out_size(W, kW, sw, pw, dw)
    col = np.empty((C * kH * kW, oH * oW), dtype=NP_STORAGE[dtype])
    _check(_im2col(_ptr(col), _ptr(im), C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW, dtype), "im2col")
    return col


def col2im(im, col, kernel, stride, pad, dilation, dtype):
    """Adds col [C*kH*kW, oH*oW] into a copy of im [C, H, W] (reference functional/functional.c:885-913)."""
    im = np.array(im, copy=True, order="C")
    col = np.ascontiguousarray(col)
    C, H, W = im.shape
    (kH, kW), (sh, sw), (ph, pw), (dh, dw) = kernel, stride, pad, dilation
    oH, oW = conv_out_size(H, kH, sh, ph, dh), conv_out_size(W, kW, sw, pw, dw)
    assert col.shape == (C * kH * kW, oH * oW)
    _check(_col2im(_ptr(im), _ptr(col), C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW, dtype), "col2im")
    return im


def conv2d_forward(x, w, bias, stride, pad, dilation, dtype):
    """reference ops/ops.c:4723-4836: per sample im2col + matmul, then y[n, c] += bias[c] with one rounding."""
    N, C, H, W = x.shape
    Co, _, kH, kW = w.shape
    oH, oW = conv_out_size(H, kH, stride[0], pad[0], dilation[0]), conv_out_size(W, kW, stride[1], pad[1], dilation[1])
    w2 = np.ascontiguousarray(w).reshape(Co, C * kH * kW)
    y = np.empty((N, Co, oH * oW), dtype=NP_STORAGE[dtype])
    for n in range(N):
        y[n] = matmul(w2, im2col(x[n], (kH, kW), stride, pad, dilation, dtype), dtype)
    if bias is not None:
        b = np.ascontiguousarray(np.broadcast_to(np.asarray(bias)[None, :, None], y.shape))
        y = add(y, b, dtype)
    return y.reshape(N, Co, oH, oW)


def conv2d_backward(x, w, dy, stride, pad, dilation, dtype, with_bias=True):
    """reference ops/ops.c:4473-4720.  Returns (dx, dw, db), each the first gradient written into a zeroed buffer:
    dx[n] = 0 + col2im(W^T dy[n]); dw = ((0 + dy[0] col[0]^T) + dy[1] col[1]^T) + ... with a rounding per add;
    db = the float32 (float64 for float64) sum over n, c-major, hw, added to zero."""
    N, C, H, W = x.shape
    Co, _, kH, kW = w.shape
    oH, oW = dy.shape[2], dy.shape[3]
    w2 = np.ascontiguousarray(w).reshape(Co, C * kH * kW)
    wt = np.ascontiguousarray(w2.T)
    dy2 = np.ascontiguousarray(dy).reshape(N, Co, oH * oW)
    zero_im = np.zeros((C, H, W), dtype=NP_STORAGE[dtype])
    dx = np.zeros(x.shape, dtype=NP_STORAGE[dtype])
    dw = np.zeros(w2.shape, dtype=NP_STORAGE[dtype])
    for n in range(N):
        dcol = matmul(wt, dy2[n], dtype)
        dx[n] = add(dx[n], col2im(zero_im, dcol, (kH, kW), stride, pad, dilation, dtype), dtype)
        col_t = np.ascontiguousarray(im2col(x[n], (kH, kW), stride, pad, dilation, dtype).T)
        dw = add(dw, matmul(dy2[n], col_t, dtype), dtype)
    db = None
    if with_bias:
        if dtype == F64:
            acc = np.zeros(Co, dtype=np.float64)
            g = dy2
        else:
            acc = np.zeros(Co, dtype=np.float32)
            g = dy2 if dtype == F32 else widen(dy2, dtype)
        for n in range(N):
            for c in range(Co):
                for v in g[n, c]:
                    acc[c] += v
        db = acc if dtype in (F32, F64) else narrow(acc, dtype)       # zeros + sum, one rounding for 16-bit
    return dx, dw.reshape(w.shape), db


# ---------------------------------------------------------------------------
# LSTM / GRU cells: the reference's op chain (recpulse/module.py:281-300, 334-351), one rounding per op
# ---------------------------------------------------------------------------
def sigmoid(x, dtype):
    x = np.ascontiguousarray(x); out = np.empty_like(x)
    _check(_sigmoid(_ptr(out), _ptr(x), x.size, dtype), "sigmoid")
    return out


def tanh(x, dtype):
    x = np.ascontiguousarray(x); out = np.empty_like(x)
    _check(_tanh(_ptr(out), _ptr(x), x.size, dtype), "tanh")
    return out


def _ew(fn, dtype, *xs):
    """One element-wise reference op: operands widened to float32 (float64 for float64), one IEEE operation chain
    `fn` in that type, one narrowing (reference functional/functional.c:10-56 for the 16-bit pivot)."""
    ct = np.float64 if dtype == F64 else np.float32
    ws = [to_f64(x, dtype).astype(ct) if dtype in (F16, BF16) else np.asarray(x, dtype=ct) for x in xs]
    y = fn(*ws).astype(ct)
    return narrow(y, dtype) if dtype in (F16, BF16) else y


def mul(a, b, dtype):
    return _ew(lambda x, y: x * y, dtype, a, b)


def sub(a, b, dtype):
    return _ew(lambda x, y: x - y, dtype, a, b)


def _row_add(y, bias, dtype):
    return add(y, np.ascontiguousarray(np.broadcast_to(bias, y.shape)), dtype)


def lstm_cell_forward(x, h, c, w_ih, w_hh, b_ih, b_hh, dtype):
    """recpulse/module.py:281-300.  Returns (h_next, c_next, saved) with saved = the activated gates."""
    H = h.shape[1]
    gates = add(matmul(x, w_ih, dtype), matmul(h, w_hh, dtype), dtype)
    if b_ih is not None:
        gates = _row_add(_row_add(gates, b_ih, dtype), b_hh, dtype)
    i_g, f_g, g_g, o_g = (np.ascontiguousarray(gates[:, q * H:(q + 1) * H]) for q in range(4))
    i_g, f_g, g_g, o_g = sigmoid(i_g, dtype), sigmoid(f_g, dtype), tanh(g_g, dtype), sigmoid(o_g, dtype)
    c_next = add(mul(f_g, c, dtype), mul(i_g, g_g, dtype), dtype)
    tc = tanh(c_next, dtype)
    return mul(o_g, tc, dtype), c_next, (i_g, f_g, g_g, o_g, tc)


def lstm_cell_backward(x, h, c, w_ih, w_hh, saved, dh, dc, dtype):
    """The chain of backward functions the reference's autograd runs for lstm_cell_forward (mul, tanh, add, sigmoid,
    chunk, add, matmul: ops/grad_host.c:365-400, 622-660; ops/ops.c:6759-6814).  Returns dx, dh_prev, dc_prev, dw_ih,
    dw_hh, db (= db_ih = db_hh)."""
    i_g, f_g, g_g, o_g, tc = saved
    one = np.ones_like(to_f64(tc, dtype))
    d_o = mul(dh, tc, dtype)
    d_tc = mul(dh, o_g, dtype)
    dcn = add(dc, _ew(lambda g, t: g * (1 - t * t), dtype, d_tc, tc), dtype)
    d_f, d_cprev, d_i, d_g = mul(dcn, c, dtype), mul(dcn, f_g, dtype), mul(dcn, g_g, dtype), mul(dcn, i_g, dtype)
    sig_b = lambda g, y: g * y * (1 - y)
    dgates = np.concatenate([_ew(sig_b, dtype, d_i, i_g), _ew(sig_b, dtype, d_f, f_g),
                             _ew(lambda g, y: g * (1 - y * y), dtype, d_g, g_g), _ew(sig_b, dtype, d_o, o_g)], axis=1)
    del one
    dx = matmul(dgates, np.ascontiguousarray(w_ih.T), dtype)
    dh_prev = matmul(dgates, np.ascontiguousarray(w_hh.T), dtype)
    dw_ih = matmul(np.ascontiguousarray(x.T), dgates, dtype)
    dw_hh = matmul(np.ascontiguousarray(h.T), dgates, dtype)
    return dx, dh_prev, d_cprev, dw_ih, dw_hh, reduce_rows(dgates, dtype)


def gru_cell_forward(x, h, w_ih, w_hh, b_ih, b_hh, dtype):
    """recpulse/module.py:334-351.  Returns (h_next, saved)."""
    H = h.shape[1]
    gi, gh = matmul(x, w_ih, dtype), matmul(h, w_hh, dtype)
    if b_ih is not None:
        gi, gh = _row_add(gi, b_ih, dtype), _row_add(gh, b_hh, dtype)
    i_r, i_z, i_n = (np.ascontiguousarray(gi[:, q * H:(q + 1) * H]) for q in range(3))
    h_r, h_z, h_n = (np.ascontiguousarray(gh[:, q * H:(q + 1) * H]) for q in range(3))
    r = sigmoid(add(i_r, h_r, dtype), dtype)
    z = sigmoid(add(i_z, h_z, dtype), dtype)
    n = tanh(add(i_n, mul(r, h_n, dtype), dtype), dtype)
    omz = _ew(lambda v: 1 - v, dtype, z)
    return add(mul(omz, n, dtype), mul(z, h, dtype), dtype), (r, z, n, h_n, omz)


def gru_cell_backward(x, h, w_ih, w_hh, saved, dh, dtype):
    """Backward chain of gru_cell_forward.  Returns dx, dh_prev, dw_ih, dw_hh, db_ih, db_hh."""
    r, z, n, h_n, omz = saved
    d_n = mul(dh, omz, dtype)
    d_z = sub(mul(dh, h, dtype), mul(dh, n, dtype), dtype)
    d_pre_n = _ew(lambda g, y: g * (1 - y * y), dtype, d_n, n)
    d_r = mul(d_pre_n, h_n, dtype)
    sig_b = lambda g, y: g * y * (1 - y)
    d_pre_r, d_pre_z = _ew(sig_b, dtype, d_r, r), _ew(sig_b, dtype, d_z, z)
    dgi = np.concatenate([d_pre_r, d_pre_z, d_pre_n], axis=1)
    dgh = np.concatenate([d_pre_r, d_pre_z, mul(d_pre_n, r, dtype)], axis=1)
    dx = matmul(dgi, np.ascontiguousarray(w_ih.T), dtype)
    dh_prev = add(mul(dh, z, dtype), matmul(dgh, np.ascontiguousarray(w_hh.T), dtype), dtype)
    dw_ih = matmul(np.ascontiguousarray(x.T), dgi, dtype)
    dw_hh = matmul(np.ascontiguousarray(h.T), dgh, dtype)
    return dx, dh_prev, dw_ih, dw_hh, reduce_rows(dgi, dtype), reduce_rows(dgh, dtype)


def matmul_f64(a, b, dtype):
    """The float64 oracle: exact inputs of `dtype`, float64 numpy product."""
    return to_f64(a, dtype) @ to_f64(b, dtype)


def rel_err(x, ref):
    """Normwise relative error ||x - ref||_F / ||ref||_F in float64."""
    x = np.asarray(x, dtype=np.float64); ref = np.asarray(ref, dtype=np.float64)
    den = np.linalg.norm(ref.ravel())
    num = np.linalg.norm((x - ref).ravel())
    return num / den if den > 0 else num


# ---------------------------------------------------------------------------
# the reference's own host kernels (oracle/_ref), when built
# ---------------------------------------------------------------------------
def load_reference():
    """ctypes handle of oracle/_ref/libref_host.so, or None when it was not built."""
    if not os.path.exists(_REF_PATH):
        return None
    ref = ctypes.CDLL(_REF_PATH)
    for name, ct in (("matmul_kernel_host_f32", ctypes.c_float), ("matmul_kernel_host_f64", ctypes.c_double)):
        fn = getattr(ref, name)
        fn.restype = _i
        fn.argtypes = [_vp, _vp, _vp, _i, _i, _i]
    for name, ct in (("sigmoid_kernel_host_f32", None), ("sigmoid_kernel_host_f64", None), ("tanh_kernel_host_f32", None), ("tanh_kernel_host_f64", None)):
        if hasattr(ref, name):
            fn = getattr(ref, name)
            fn.restype = _i
            fn.argtypes = [_vp, _vp, _sz]
    for name in ("im2col_kernel_host_f32", "im2col_kernel_host_f64", "col2im_kernel_host_f32", "col2im_kernel_host_f64"):
        if hasattr(ref, name):
            fn = getattr(ref, name)
            fn.restype = _i
            fn.argtypes = [_vp, _vp] + [_i] * 13
    return ref


def reference_matmul(ref, a, b, dtype):
    """C = A @ B through the reference's matmul_kernel_host_f32/f64 (f32/f64 only)."""
    a = np.ascontiguousarray(a); b = np.ascontiguousarray(b)
    m, k = a.shape; n = b.shape[1]
    c = np.empty((m, n), dtype=NP_STORAGE[dtype])
    fn = ref.matmul_kernel_host_f32 if dtype == F32 else ref.matmul_kernel_host_f64
    _check(fn(_ptr(c), _ptr(a), _ptr(b), m, k, n), "reference matmul")
    return c
