"""conv2d on the GPU: the lowering kernels through the C ABI, and op_conv2d / Conv2d through the drop-in module.

Lowering (im2col, col2im, the channel bias add) is index and copy work plus single rounding adds, so it is held to
bit equality with the CPU oracle; the whole convolution is held to the GEMM's tolerances against the oracle's
per-sample chain and against torch.nn.functional.conv2d in float64.  Shapes: the reference's own parity matrix
(tests/stress/stress_torch_parity.py:199-210) and test values (tests/autograd/test_conv2d.py), plus cases that take
the vector store path, several chunks of the batch, and the 1x1 shortcut.
"""
import json
import os

import numpy as np
import pytest

import oracle
import recpulse_cuda as rp
from recpulse.module import Conv2d
from recpulse_amd import capi
from devhelp import ALL, BF16, F16, F32, F64, NAMES, Dev, rand_storage, tol

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))
REF_CASES = [tuple(tuple(v) if isinstance(v, list) else v for v in c) for c in GOLD["conv2d_parity_shapes"]["cases"]]
# (x shape, w shape, stride, pad, dilation, bias): out_H*out_W a multiple of 8 (vector stores), a 1x1 kernel with
# stride, a pointwise kernel (no lowering at all), a wider layer
MORE_CASES = [((3, 4, 16, 16), (6, 4, 3, 3), (1, 1), (1, 1), (1, 1), True),
              ((2, 5, 9, 9), (3, 5, 1, 1), (2, 2), (0, 0), (1, 1), True),
              ((4, 16, 8, 8), (24, 16, 1, 1), (1, 1), (0, 0), (1, 1), True),
              ((2, 32, 14, 14), (64, 32, 3, 3), (1, 1), (1, 1), (1, 1), False),
              # 3 x 3 / stride 1 / padding 1 with whole vectors per row: first, interior and last vectors of a row, and a one-row image
              ((2, 3, 5, 24), (4, 3, 3, 3), (1, 1), (1, 1), (1, 1), True),
              ((1, 2, 1, 8), (2, 2, 3, 3), (1, 1), (1, 1), (1, 1), False),
              # 64 channels in and out: the 16-bit types read the taps from zero-bordered planes, forward and input gradient
              ((2, 64, 8, 8), (64, 64, 3, 3), (1, 1), (1, 1), (1, 1), True)]
CASES = REF_CASES + MORE_CASES
DT_NAME = {F32: "float32", F64: "float64", F16: "float16", BF16: "bfloat16"}


def _geom(xs, ws, s, p, d):
    oH, oW = oracle.conv_out_size(xs[2], ws[2], s[0], p[0], d[0]), oracle.conv_out_size(xs[3], ws[3], s[1], p[1], d[1])
    return (xs[1], xs[2], xs[3], ws[2], ws[3], s[0], s[1], p[0], p[1], d[0], d[1], oH, oW)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[1][2:])))
def test_lowering_is_bit_exact(dt, case):
    xs, ws, s, p, d, _ = case
    N, C, H, W = xs
    geom = _geom(xs, ws, s, p, d)
    oH, oW = geom[-2:]
    rows, cols = C * ws[2] * ws[3], oH * oW
    rng = np.random.default_rng(80)
    x = rand_storage(rng, xs, dt)
    L = capi.lib()
    dx, dcol = Dev(x, dt), Dev.empty((N, rows, cols), dt)
    capi.check(L.rp_hip_im2col_batched(dcol.ptr, dx.ptr, N, *geom, dt), "rp_hip_im2col_batched")
    want = np.stack([oracle.im2col(x[n], ws[2:], s, p, d, dt) for n in range(N)])
    assert np.array_equal(dcol.numpy(), want)
    # the adjoint, overwriting and adding
    c2 = rand_storage(rng, (N, rows, cols), dt)
    base = rand_storage(rng, xs, dt)
    dc2, dim = Dev(c2, dt), Dev(base, dt)
    capi.check(L.rp_hip_col2im_batched(dim.ptr, dc2.ptr, N, *geom, 1, dt), "rp_hip_col2im_batched")
    want = np.stack([oracle.col2im(base[n], c2[n], ws[2:], s, p, d, dt) for n in range(N)])
    assert np.array_equal(dim.numpy(), want)
    capi.check(L.rp_hip_col2im_batched(dim.ptr, dc2.ptr, N, *geom, 0, dt), "rp_hip_col2im_batched")
    want = np.stack([oracle.col2im(np.zeros_like(base[n]), c2[n], ws[2:], s, p, d, dt) for n in range(N)])
    assert np.array_equal(dim.numpy(), want)
    # the reference's single-sample entry points on sample 0
    d1, dim1 = Dev.empty((rows, cols), dt), Dev(base[0], dt)
    capi.check(L.im2col_kernel_device(d1.ptr, dx.ptr, *geom, dt), "im2col_kernel_device")
    assert np.array_equal(d1.numpy(), oracle.im2col(x[0], ws[2:], s, p, d, dt))
    capi.check(L.col2im_kernel_device(dim1.ptr, dc2.ptr, *geom, dt), "col2im_kernel_device")
    assert np.array_equal(dim1.numpy(), oracle.col2im(base[0], c2[0], ws[2:], s, p, d, dt))


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_channel_bias_add_and_channel_sums(dt):
    rng = np.random.default_rng(81)
    N, C, HW = 5, 7, 99
    y, b = rand_storage(rng, (N, C, HW), dt), rand_storage(rng, (C,), dt)
    L = capi.lib()
    dy, db = Dev(y, dt), Dev(b, dt)
    capi.check(L.rp_hip_channel_bias_add(dy.ptr, db.ptr, N, C, HW, dt), "rp_hip_channel_bias_add")
    want = oracle.add(y, np.ascontiguousarray(np.broadcast_to(b[None, :, None], y.shape)), dt)
    assert np.array_equal(dy.numpy(), want)
    # sums: a tree of float32 (float64) partial sums here, one running sum in the reference
    ds = Dev(b, dt)
    capi.check(L.rp_hip_channel_sums(ds.ptr, Dev(y, dt).ptr, N, C, HW, 0, dt), "rp_hip_channel_sums")
    exact = oracle.to_f64(y, dt).sum(axis=(0, 2))
    assert oracle.rel_err(oracle.to_f64(ds.numpy(), dt), exact) <= {F32: 1e-6, F64: 1e-14, F16: 2e-3, BF16: 1e-2}[dt]
    got0 = ds.numpy()
    capi.check(L.rp_hip_channel_sums(ds.ptr, Dev(y, dt).ptr, N, C, HW, 1, dt), "rp_hip_channel_sums")
    assert np.array_equal(ds.numpy(), oracle.add(got0, got0, dt))


def test_lowering_rejects_inconsistent_geometry():
    d = capi.DeviceBuffer(1 << 16)
    L = capi.lib()
    # out_H that the geometry does not imply, zero stride, negative padding
    assert L.rp_hip_im2col_batched(d.ptr, d.ptr, 1, 1, 4, 4, 3, 3, 1, 1, 0, 0, 1, 1, 3, 2, F32) == -1
    assert b"geometry" in L.rp_hip_last_error()
    assert L.rp_hip_im2col_batched(d.ptr, d.ptr, 1, 1, 4, 4, 3, 3, 0, 1, 0, 0, 1, 1, 2, 2, F32) == -1
    assert L.rp_hip_col2im_batched(d.ptr, d.ptr, 1, 1, 4, 4, 3, 3, 1, 1, -1, 0, 1, 1, 2, 2, 0, F32) == -1
    assert L.rp_hip_im2col_batched(None, d.ptr, 1, 1, 4, 4, 3, 3, 1, 1, 0, 0, 1, 1, 2, 2, F32) == -1


SAME_CASES = [  # (batch, C_in, H, W, C_out, kH, kW): whole tiles, ragged columns, several slabs per tap, 5 x 5, one row
    (3, 64, 8, 8, 64, 3, 3), (2, 128, 14, 14, 64, 3, 3), (2, 64, 7, 20, 192, 3, 3), (1, 64, 9, 12, 32, 5, 5),
    (2, 64, 1, 16, 64, 3, 1), (1, 64, 56, 56, 64, 3, 3), (5, 64, 10, 10, 24, 3, 3)]


def _one_rounding(dt, k):
    """Distance from float64 of a sum kept in the accumulate type and rounded once to dt."""
    return {BF16: 2.0 ** -8, F16: 2.0 ** -11}.get(dt, tol(dt, k))


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("case", SAME_CASES, ids=lambda c: "x".join(map(str, c)))
def test_same_convolution_without_lowered_matrix(dt, case):
    """rp_hip_conv2d_same_forward / _backward_input against the oracle's per-sample chain and against float64."""
    import torch
    N, Ci, H, W, Co, kH, kW = case
    L = capi.lib()
    assert L.rp_hip_conv2d_same_supported(Ci, H, W, kH, kW, dt) == 1
    rng = np.random.default_rng(83)
    x, w = rand_storage(rng, (N, Ci, H, W), dt), oracle.to_storage(rng.standard_normal((Co, Ci, kH, kW)) * 0.2, dt)
    b = rand_storage(rng, (Co,), dt)
    s, p, d = (1, 1), (kH // 2, kW // 2), (1, 1)
    dx_, dw_, db_, dy_ = Dev(x, dt), Dev(w, dt), Dev(b, dt), Dev.empty((N, Co, H, W), dt)
    capi.check(L.rp_hip_conv2d_same_forward(dy_.ptr, dx_.ptr, dw_.ptr, db_.ptr, N, Ci, H, W, Co, kH, kW, dt), "same forward")
    y_ref = oracle.conv2d_forward(x, w, b, s, p, d, dt)
    xt, wt = torch.tensor(oracle.to_f64(x, dt)), torch.tensor(oracle.to_f64(w, dt))
    y_exact = torch.nn.functional.conv2d(xt, wt, torch.tensor(oracle.to_f64(b, dt)), padding=p).numpy()
    got = oracle.to_f64(dy_.numpy(), dt)
    assert oracle.rel_err(got, oracle.to_f64(y_ref, dt)) <= tol(dt, Ci * kH * kW)
    assert oracle.rel_err(got, y_exact) <= tol(dt, Ci * kH * kW)
    # without a bias the result is the sum in the accumulate type rounded once: no further from float64 than one rounding of dt
    capi.check(L.rp_hip_conv2d_same_forward(dy_.ptr, dx_.ptr, dw_.ptr, None, N, Ci, H, W, Co, kH, kW, dt), "same forward")
    y_nb = torch.nn.functional.conv2d(xt, wt, None, padding=p).numpy()
    assert oracle.rel_err(oracle.to_f64(dy_.numpy(), dt), y_nb) <= _one_rounding(dt, Ci * kH * kW)
    # gradient with respect to the input (C_out in whole k slabs of the dtype's kernel)
    dx_ok = L.rp_hip_conv2d_same_supported(Co, H, W, kH, kW, dt) == 1
    assert dx_ok == (Co % {BF16: 64, F16: 64, F32: 32, F64: 16}[dt] == 0)
    if dx_ok:
        g = rand_storage(rng, (N, Co, H, W), dt)
        dg_, dgx_ = Dev(g, dt), Dev.empty((N, Ci, H, W), dt)
        capi.check(L.rp_hip_conv2d_same_backward_input(dgx_.ptr, dg_.ptr, dw_.ptr, N, Ci, H, W, Co, kH, kW, dt), "same backward")
        dx_ref, _, _ = oracle.conv2d_backward(x, w, g, s, p, d, dt, with_bias=False)
        dx_exact = torch.nn.grad.conv2d_input((N, Ci, H, W), wt, torch.tensor(oracle.to_f64(g, dt)), padding=p).numpy()
        got = oracle.to_f64(dgx_.numpy(), dt)
        assert oracle.rel_err(got, oracle.to_f64(dx_ref, dt)) <= tol(dt, Co * kH * kW)
        assert oracle.rel_err(got, dx_exact) <= _one_rounding(dt, Co * kH * kW)
    else:
        g = rand_storage(rng, (N, Co, H, W), dt)
        dg_ = Dev(g, dt)
    # gradient with respect to the weights (any channel counts), alone and together with the input gradient
    assert L.rp_hip_conv2d_same_supported(0, H, W, kH, kW, dt) == 1
    dgw_ = Dev.empty((Co, Ci, kH, kW), dt)
    capi.check(L.rp_hip_conv2d_same_backward(None, dgw_.ptr, dg_.ptr, dx_.ptr, None, N, Ci, H, W, Co, kH, kW, dt), "same backward (weights)")
    _, dw_ref, _ = oracle.conv2d_backward(x, w, g, s, p, d, dt, with_bias=False)
    dw_exact = torch.nn.grad.conv2d_weight(xt, (Co, Ci, kH, kW), torch.tensor(oracle.to_f64(g, dt)), padding=p).numpy()
    got_w = oracle.to_f64(dgw_.numpy(), dt)
    assert oracle.rel_err(got_w, oracle.to_f64(dw_ref, dt).reshape(got_w.shape)) <= tol(dt, N * H * W)
    assert oracle.rel_err(got_w, dw_exact) <= tol(dt, N * H * W)
    if dx_ok:
        both_x, both_w = Dev.empty((N, Ci, H, W), dt), Dev.empty((Co, Ci, kH, kW), dt)
        capi.check(L.rp_hip_conv2d_same_backward(both_x.ptr, both_w.ptr, dg_.ptr, dx_.ptr, dw_.ptr, N, Ci, H, W, Co, kH, kW, dt), "same backward (both)")
        assert np.array_equal(both_x.numpy(), dgx_.numpy()) and np.array_equal(both_w.numpy(), dgw_.numpy())


def test_same_convolution_in_chunks_of_the_batch(monkeypatch):
    """With room for two samples at a time a batch of five goes in three chunks: same bits as in one piece (the weight
    gradient adds its chunks in fp32 and rounds after each, so it is compared to tolerance)."""
    dt, (N, Ci, H, W, Co, kH, kW) = BF16, (5, 64, 6, 8, 64, 3, 3)
    L = capi.lib()
    rng = np.random.default_rng(84)
    x, w, g = rand_storage(rng, (N, Ci, H, W), dt), oracle.to_storage(rng.standard_normal((Co, Ci, kH, kW)) * 0.2, dt), rand_storage(rng, (N, Co, H, W), dt)
    dx_, dw_, dg_ = Dev(x, dt), Dev(w, dt), Dev(g, dt)

    def run():
        y, gx, gw = Dev.empty((N, Co, H, W), dt), Dev.empty((N, Ci, H, W), dt), Dev.empty((Co, Ci, kH, kW), dt)
        capi.check(L.rp_hip_conv2d_same_forward(y.ptr, dx_.ptr, dw_.ptr, None, N, Ci, H, W, Co, kH, kW, dt), "same forward")
        capi.check(L.rp_hip_conv2d_same_backward(gx.ptr, gw.ptr, dg_.ptr, dx_.ptr, dw_.ptr, N, Ci, H, W, Co, kH, kW, dt), "same backward")
        return y.numpy(), gx.numpy(), gw.numpy()

    whole = run()
    per_sample = (2 * 64 * (8 * 16 + 16) + 64 * 64 * 9) * 2          # padded dy and x planes plus the larger product, bytes
    monkeypatch.setenv("RP_CONV_WORKSPACE_BYTES", str(2 * per_sample + 64))
    parts = run()
    assert np.array_equal(whole[0], parts[0]) and np.array_equal(whole[1], parts[1])
    assert oracle.rel_err(oracle.to_f64(parts[2], dt), oracle.to_f64(whole[2], dt)) <= 2.0 ** -7
    forward_per_sample = (64 * (8 * 16 + 16) + 64 * 6 * 16) * 2      # the forward holds less per sample: give it room for two as well
    monkeypatch.setenv("RP_CONV_WORKSPACE_BYTES", str(2 * forward_per_sample + 64))
    assert np.array_equal(whole[0], run()[0])


def test_same_convolution_rejects_other_shapes():
    L = capi.lib()
    assert L.rp_hip_conv2d_same_supported(48, 8, 8, 3, 3, BF16) == 0           # channels in whole k slabs: 64 for 16-bit types,
    assert L.rp_hip_conv2d_same_supported(48, 8, 8, 3, 3, F32) == 0            # 32 for float32,
    assert L.rp_hip_conv2d_same_supported(32, 8, 8, 3, 3, F32) == 1
    assert L.rp_hip_conv2d_same_supported(24, 8, 8, 3, 3, F64) == 0            # 16 for float64
    assert L.rp_hip_conv2d_same_supported(48, 8, 8, 3, 3, F64) == 1
    assert L.rp_hip_conv2d_same_supported(64, 8, 8, 3, 3, 99) == 0             # no such dtype
    assert L.rp_hip_conv2d_same_supported(64, 8, 8, 2, 2, BF16) == 0           # odd kernels only
    assert L.rp_hip_conv2d_same_supported(64, 8, 8, 1, 1, BF16) == 0           # 1 x 1 needs no lowering in the first place
    d = Dev.empty((64 * 64,), BF16)
    assert L.rp_hip_conv2d_same_forward(d.ptr, d.ptr, d.ptr, None, 1, 48, 8, 8, 64, 3, 3, BF16) == -1
    assert b"rp_hip_conv2d_same_supported" in L.rp_hip_last_error()


# ---- through the drop-in module -------------------------------------------------------------------------------
def _dev(arr, dt, grad=False):
    """storage array -> device tensor (16-bit values travel as float32, exactly)."""
    vals = oracle.to_f64(arr, dt)
    t = rp.from_numpy(np.ascontiguousarray(vals, dtype=np.float64 if dt == F64 else np.float32)).to(device="cuda", dtype=DT_NAME[dt])
    return t.requires_grad_(True) if grad else t


def _host(t):
    return t.to(device="cpu", dtype="float64").to_numpy()


def _run_conv(x, w, b, dy, s, p, d, dt):
    tx, tw = _dev(x, dt, True), _dev(w, dt, True)
    tb = _dev(b, dt, True) if b is not None else None
    y = tx.op_conv2d(tw, bias=tb, stride_h=s[0], stride_w=s[1], pad_h=p[0], pad_w=p[1], dilation_h=d[0], dilation_w=d[1])
    # upstream gradient dy: loss = y_flat . dy_flat
    n = int(np.prod(y.shape))
    y.reshape([1, n]).op_matmul(_dev(dy, dt).reshape([n, 1])).op_sum_all().backward()
    return _host(y), _host(tx.grad), _host(tw.grad), (_host(tb.grad) if tb is not None else None)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c[0])) + "_k" + "x".join(map(str, c[1][2:])))
def test_conv2d_forward_and_backward(dt, case, monkeypatch):
    import torch
    xs, ws, s, p, d, has_bias = case
    rng = np.random.default_rng(82)
    x, w = rand_storage(rng, xs, dt), oracle.to_storage(rng.standard_normal(ws) * 0.3, dt)
    b = rand_storage(rng, (ws[0],), dt) if has_bias else None
    y_ref = oracle.conv2d_forward(x, w, b, s, p, d, dt)
    dy = rand_storage(rng, y_ref.shape, dt)
    got = _run_conv(x, w, b, dy, s, p, d, dt)
    dx_ref, dw_ref, db_ref = oracle.conv2d_backward(x, w, dy, s, p, d, dt, with_bias=has_bias)
    k_fwd, k_dx, k_dw = xs[1] * ws[2] * ws[3], ws[0], y_ref.shape[2] * y_ref.shape[3] * xs[0]
    names = ("y", "dx", "dw", "db")
    refs = (y_ref, dx_ref, dw_ref, db_ref)
    ks = (k_fwd, k_dx, k_dw, k_dw)
    for name, g, r, k in zip(names, got, refs, ks):
        if r is None:
            continue
        assert g.shape == r.shape, name
        assert oracle.rel_err(g, oracle.to_f64(r, dt)) <= tol(dt, k), name
    # the same against an independent float64 implementation
    xt = torch.tensor(oracle.to_f64(x, dt), requires_grad=True); wt = torch.tensor(oracle.to_f64(w, dt), requires_grad=True)
    bt = torch.tensor(oracle.to_f64(b, dt), requires_grad=True) if has_bias else None
    yt = torch.nn.functional.conv2d(xt, wt, bt, stride=s, padding=p, dilation=d)
    yt.backward(torch.tensor(oracle.to_f64(dy, dt)))
    exact = (yt.detach().numpy(), xt.grad.numpy(), wt.grad.numpy(), bt.grad.numpy() if has_bias else None)
    for name, g, r, k in zip(names, got, exact, ks):
        if r is not None:
            assert oracle.rel_err(g, r) <= tol(dt, k), name
    # with the lowered matrix limited to one sample at a time the batch goes in chunks of one: the GEMMs then run
    # unbatched (a different kernel and split of k may be chosen), so the comparison is to tolerance, not to the bit
    monkeypatch.setenv("RP_CONV_COL_BYTES", "1")
    monkeypatch.setenv("RP_CONV_NO_DIRECT", "1")           # and always through the lowered matrix
    again = _run_conv(x, w, b, dy, s, p, d, dt)
    for name, g, r, k in zip(names, again, refs, ks):
        if r is not None:
            assert oracle.rel_err(g, oracle.to_f64(r, dt)) <= tol(dt, k), name + " (chunked)"


@pytest.mark.parametrize("dtype", ["float32", "float64", "float16", "bfloat16"])
def test_conv2d_reference_known_answers(dtype):
    """reference tests/autograd/test_conv2d.py:46-152, 188-216 with device='cuda'."""
    for case in GOLD["conv2d_known_answers"]["cases"]:
        x = rp.ones(case["x_shape"], dtype=dtype, device="cuda").requires_grad_(True)
        w = rp.ones(case["w_shape"], dtype=dtype, device="cuda").requires_grad_(True)
        b = rp.values(case["bias"], dtype=dtype, device="cuda").requires_grad_(True) if "bias" in case else None
        s, p = case.get("stride", (1, 1)), case.get("pad", (0, 0))
        y = x.op_conv2d(w, bias=b, stride_h=s[0], stride_w=s[1], pad_h=p[0], pad_w=p[1])
        assert list(y.shape) == case["out_shape"] and y.dtype == dtype
        if "out_sum" in case:
            assert _host(y).sum() == case["out_sum"]
        y.op_sum_all().backward()
        assert x.has_grad and x.grad.shape == tuple(case["x_shape"])
        assert w.has_grad and w.grad.shape == tuple(case["w_shape"])
        if "bias_grad_of_sum" in case:
            assert b.grad.shape == (1,) and list(_host(b.grad)) == case["bias_grad_of_sum"]


def test_conv2d_weight_gradient_vs_central_differences():
    """reference tests/autograd/test_conv2d.py:154-186."""
    g = GOLD["conv2d_known_answers"]["weight_gradcheck"]
    x = np.array(g["x"], dtype=np.float64).reshape(g["x_shape"]); w = np.array(g["w"], dtype=np.float64).reshape(g["w_shape"])
    tw = _dev(w, F64, True)
    _dev(x, F64).op_conv2d(tw).op_sum_all().backward()
    eps = 1e-3
    for i in range(9):
        wp, wm = w.copy().reshape(-1), w.copy().reshape(-1)
        wp[i] += eps; wm[i] -= eps
        num = (_host(_dev(x, F64).op_conv2d(_dev(wp.reshape(w.shape), F64))).sum() - _host(_dev(x, F64).op_conv2d(_dev(wm.reshape(w.shape), F64))).sum()) / (2 * eps)
        assert abs(_host(tw.grad).reshape(-1)[i] - num) <= 1e-2 * max(1.0, abs(num))


def test_conv2d_module_and_argument_errors():
    """reference recpulse/module.py:117-155 (layout of the parameters, int or pair arguments) and ops/ops.c:4726-4742 (rejections)."""
    rp.manual_seed(3)
    layer = Conv2d(3, 8, 3, stride=(2, 1), padding=1).to(device="cuda")
    assert layer.weight.shape == (8, 3, 3, 3) and layer.bias.shape == (8,) and set(layer.tracked) == {"weight", "bias"}
    assert layer.kernel_size == (3, 3) and layer.stride == (2, 1) and layer.padding == (1, 1) and layer.dilation == (1, 1)
    w = _host(layer.weight)
    assert abs(w.std() - 1.0 / np.sqrt(27)) < 0.05 and np.all(_host(layer.bias) == 0)
    x = rp.randn([2, 3, 9, 8], device="cuda")
    y = layer(x)
    assert y.shape == (2, 8, 5, 8)
    y.op_sum_all().backward()
    assert layer.weight.has_grad and layer.bias.has_grad and np.all(_host(layer.bias.grad) == 2 * 5 * 8)
    assert Conv2d(3, 4, (1, 2), bias=False).bias is None
    with pytest.raises(RuntimeError):
        x.op_conv2d(rp.ones([4, 2, 3, 3], device="cuda"))            # channel mismatch
    with pytest.raises(RuntimeError):
        x.op_conv2d(rp.ones([4, 3, 11, 3], device="cuda"))           # kernel taller than the input
    with pytest.raises(RuntimeError):
        x.op_conv2d(rp.ones([4, 3, 3, 3], device="cuda"), stride_h=0)
    with pytest.raises(RuntimeError):
        x.reshape([6, 9, 8]).op_conv2d(rp.ones([4, 3, 3, 3], device="cuda"))
