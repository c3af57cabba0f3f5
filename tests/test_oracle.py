"""Pins for the CPU oracle (oracle/rp_oracle.c).

Nothing here retypes the oracle's formulas.  Each restated function is held to
(1) the known answers in the reference's own tests (tests/golden/), (2) bit
equality with the reference's own host kernels compiled unchanged into
oracle/_ref (skipped only if that library was never built), (3) independent
implementations: numpy float64 closed forms, numpy/torch casts, torch autograd,
and scalar Python loops in np.float32 that fix the accumulation order.
"""
import json
import os

import numpy as np
import pytest

import oracle
from oracle import F32, F64, F16, BF16

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))
REF = oracle.load_reference()
needs_ref = pytest.mark.skipif(REF is None, reason="oracle/_ref was not built (reference tree absent at build time)")
ALL = [F32, F64, F16, BF16]


def _st(x, dt):
    return oracle.to_storage(np.array(x, dtype=np.float64), dt)


# --------------------------------------------------------------------------- converters
def test_f16_widen_exhaustive_vs_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.widen(bits, F16)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_bf16_widen_exhaustive_is_shift():
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.widen(bits, BF16).view(np.uint32)
    assert np.array_equal(got, bits.astype(np.uint32) << 16)


@pytest.mark.parametrize("dt", [F16, BF16])
def test_narrow_roundtrip_exhaustive(dt):
    bits = np.arange(65536, dtype=np.uint16)
    w = oracle.widen(bits, dt)
    ok = ~np.isnan(w)
    assert np.array_equal(oracle.narrow(w[ok], dt), bits[ok])


def test_f16_narrow_matches_numpy_off_ties_and_rounds_ties_away():
    rng = np.random.default_rng(10)
    x = np.concatenate([rng.normal(0, 1, 200000), rng.normal(0, 300, 50000),
                        rng.uniform(-1e-5, 1e-5, 50000)]).astype(np.float32)
    x = x[np.abs(x) < 65000]
    u = x.view(np.uint32)
    normal = np.abs(x) >= 2.0 ** -14
    tie = (u & 0x1FFF) == 0x1000
    sel = normal & ~tie
    assert np.array_equal(oracle.narrow(x[sel], F16), x[sel].astype(np.float16).view(np.uint16))
    # exact midpoints between neighbouring fp16 values go away from zero
    h = np.arange(0x0400, 0x7BFF, 7, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64); hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    assert np.array_equal(oracle.narrow(mid, F16), h + 1)
    assert np.array_equal(oracle.narrow(-mid, F16), (h + 1) | 0x8000)
    below = np.nextafter(mid, np.float32(0))
    assert np.array_equal(oracle.narrow(below, F16), h)
    # subnormal results: agree with numpy off ties
    sub = rng.uniform(-6e-5, 6e-5, 100000).astype(np.float32)
    got = oracle.narrow(sub, F16).view(np.float16).astype(np.float64)
    want = sub.astype(np.float16).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2.0 ** -24          # never more than one subnormal step apart
    assert np.mean(got == want) > 0.999
    assert oracle.narrow(np.array([1e6, -1e6, np.inf], np.float32), F16).tolist() == [0x7C00, 0xFC00, 0x7C00]


def test_bf16_narrow_matches_torch_off_ties_and_rounds_ties_away():
    import torch
    rng = np.random.default_rng(11)
    x = rng.normal(0, 10, 300000).astype(np.float32)
    tie = (x.view(np.uint32) & 0xFFFF) == 0x8000
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.narrow(x, BF16)
    assert np.array_equal(got[~tie], want[~tie])
    h = np.arange(0x0080, 0x7F00, 5, dtype=np.uint16)
    mid = ((h.astype(np.uint32) << 16) | 0x8000).view(np.float32)
    assert np.array_equal(oracle.narrow(mid, BF16), h + 1)
    assert np.array_equal(oracle.narrow(-mid, BF16), (h + 1) | 0x8000)
    assert np.array_equal(oracle.narrow(np.nextafter(mid, np.float32(0)), BF16), h)


# --------------------------------------------------------------------------- matmul
@pytest.mark.parametrize("dt", ALL)
def test_matmul_reference_known_answers(dt):
    for key in ("matmul_2x3_3x2", "matmul_identity"):
        g = GOLD[key]
        c = oracle.matmul(_st(g["a"], dt), _st(g["b"], dt), dt)
        assert np.array_equal(oracle.to_f64(c, dt), np.array(g["c"], dtype=np.float64)), key
    assert oracle.to_f64(c, dt).shape == (2, 2)
    g = GOLD["matmul_2x3_3x2"]
    c = oracle.matmul(_st(g["a"], dt), _st(g["b"], dt), dt)
    assert oracle.to_f64(oracle.sum_all(c, dt), dt)[0] == g["c_sum"]


@pytest.mark.parametrize("dt", ALL)
def test_matmul_backward_reference_known_answers(dt):
    for key in ("backward_a", "backward_both_2x2", "backward_nonsquare_2x4_4x3"):
        g = GOLD[key]
        a, b = _st(g["a"], dt), _st(g["b"], dt)
        dc = _st(np.ones((len(g["a"]), len(g["b"][0]))), dt)
        da, db = oracle.matmul_backward(a, b, dc, dt)
        assert np.array_equal(oracle.to_f64(da, dt), np.array(g["da"], dtype=np.float64)), key
        assert np.array_equal(oracle.to_f64(db, dt), np.array(g["db"], dtype=np.float64)), key


def test_matmul_backward_f64_known_answer():
    g = GOLD["backward_f64_2x2"]
    a, b = _st(g["a"], F64), _st(g["b"], F64)
    c = oracle.matmul(a, b, F64)
    assert abs(oracle.sum_all(c, F64)[0] - g["c_sum"]) < 1e-10
    da, db = oracle.matmul_backward(a, b, np.ones((2, 2)), F64)
    assert np.max(np.abs(da - np.array(g["da"]))) < 1e-10
    assert np.max(np.abs(db - np.array(g["db"]))) < 1e-10


def test_matmul_parity_shapes_f64_vs_numpy():
    rng = np.random.default_rng(12)
    g = GOLD["parity_shapes"]
    for m, k, n in g["mkn"]:
        a = rng.uniform(-1, 1, (m, k)); b = rng.uniform(-1, 1, (k, n))
        np.testing.assert_allclose(oracle.matmul(a, b, F64), a @ b, rtol=g["rtol"], atol=g["atol"])


def _loop_matmul(a, b, ty):
    """Scalar reference of the accumulation order: C[i,j] built left to right in `ty`."""
    m, k = a.shape; n = b.shape[1]
    c = np.zeros((m, n), dtype=ty)
    for i in range(m):
        for j in range(n):
            acc = ty(0)
            for l in range(k):
                acc = ty(acc + ty(a[i, l] * b[l, j]))
            c[i, j] = acc
    return c


@pytest.mark.parametrize("dt,ty", [(F32, np.float32), (F64, np.float64)])
def test_matmul_accumulation_order_and_type(dt, ty):
    rng = np.random.default_rng(13)
    # magnitudes spread over many binades: any reordering, widening of the
    # accumulator or fused multiply-add changes low bits somewhere
    a = (rng.normal(0, 1, (5, 37)) * 10.0 ** rng.integers(-4, 5, (5, 37))).astype(ty)
    b = (rng.normal(0, 1, (37, 6)) * 10.0 ** rng.integers(-4, 5, (37, 6))).astype(ty)
    got = oracle.matmul(a, b, dt)
    want = _loop_matmul(a, b, ty)
    assert np.array_equal(got.view(np.uint32 if dt == F32 else np.uint64),
                          want.view(np.uint32 if dt == F32 else np.uint64))


@needs_ref
@pytest.mark.parametrize("dt", [F32, F64])
def test_matmul_bit_equal_to_reference_kernel(dt):
    rng = np.random.default_rng(14)
    for m, k, n in [(1, 1, 1), (3, 4, 5), (1, 7, 1), (16, 32, 8), (64, 64, 64), (128, 784, 256), (33, 257, 19)]:
        a = oracle.to_storage(rng.normal(0, 1, (m, k)), dt)
        b = oracle.to_storage(rng.normal(0, 1, (k, n)), dt)
        assert oracle.matmul(a, b, dt).tobytes() == oracle.reference_matmul(REF, a, b, dt).tobytes()


@pytest.mark.parametrize("dt", [F16, BF16])
def test_matmul_16bit_is_fp32_pivot_then_one_narrowing(dt):
    rng = np.random.default_rng(15)
    a = oracle.to_storage(rng.normal(0, 1, (9, 40)), dt)
    b = oracle.to_storage(rng.normal(0, 1, (40, 11)), dt)
    c = oracle.matmul(a, b, dt)
    c32 = _loop_matmul(oracle.widen(a, dt), oracle.widen(b, dt), np.float32)
    assert np.array_equal(c, oracle.narrow(c32, dt))
    assert oracle.rel_err(oracle.to_f64(c, dt), oracle.matmul_f64(a, b, dt)) < 2e-2


def test_matmul_rejects_bad_arguments():
    a = np.zeros((2, 2), np.float32)
    with pytest.raises(RuntimeError):
        oracle._check(oracle._matmul(None, oracle._ptr(a), oracle._ptr(a), 2, 2, 2, F32), "matmul")
    with pytest.raises(RuntimeError):
        oracle._check(oracle._matmul(oracle._ptr(a), oracle._ptr(a), oracle._ptr(a), 0, 2, 2, F32), "matmul")
    with pytest.raises(RuntimeError):
        oracle._check(oracle._matmul(oracle._ptr(a), oracle._ptr(a), oracle._ptr(a), 2, 2, 2, 9), "matmul")


# --------------------------------------------------------------------------- strided / batched / epilogue
@pytest.mark.parametrize("dt", ALL)
def test_gemm_strided_batched_views_bias_accumulate(dt):
    rng = np.random.default_rng(16)
    batch, m, k, n = 3, 5, 7, 4
    A = oracle.to_storage(rng.normal(0, 1, (batch, k, m)), dt)        # stored transposed: view is [m,k] with strides (1, m)
    B = oracle.to_storage(rng.normal(0, 1, (batch, n, k)), dt)        # stored transposed: view is [k,n] with strides (1, k)
    bias = oracle.to_storage(rng.normal(0, 1, (n,)), dt)
    C0 = oracle.to_storage(rng.normal(0, 1, (batch, m, n)), dt)
    C = C0.copy()
    oracle.gemm_strided_batched(C, A, B, bias, batch, m, k, n, (k * m, 1, m), (n * k, 1, k), (m * n, n, 1), True, dt)
    for z in range(batch):
        az = np.ascontiguousarray(A[z].T); bz = np.ascontiguousarray(B[z].T)
        y = oracle.bias_add(oracle.matmul(az, bz, dt), bias, dt)
        want = oracle.add(C0[z], y, dt)
        assert np.array_equal(C[z], want)
    # float64 closed form
    want64 = np.einsum("zkm,znk->zmn", oracle.to_f64(A, dt), oracle.to_f64(B, dt)) + oracle.to_f64(bias, dt) + oracle.to_f64(C0, dt)
    tol = {F32: 1e-5, F64: 1e-13, F16: 2e-2, BF16: 2e-2}[dt]
    assert oracle.rel_err(oracle.to_f64(C, dt), want64) < tol


def test_contiguous_copy_is_view_indexing():
    rng = np.random.default_rng(17)
    base = rng.normal(0, 1, (4, 5, 6)).astype(np.float32)
    view = base.transpose(2, 0, 1)[1:, ::2]
    strides = [s // 4 for s in view.strides]
    off = (view.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // 4
    got = oracle.contiguous_copy(base, view.shape, strides, F32, offset=off)
    assert np.array_equal(got, view)


# --------------------------------------------------------------------------- element-wise neighbours
@needs_ref
def test_elementwise_bit_equal_to_reference_kernels():
    import ctypes
    rng = np.random.default_rng(18)
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    x = rng.normal(0, 2, (7, 33)).astype(np.float32)
    out = np.empty_like(x)
    REF.softmax_kernel_host_f32.argtypes = [vp, vp, sz, sz, sz]
    REF.log_softmax_kernel_host_f32.argtypes = [vp, vp, sz, sz, sz]
    REF.softmax_kernel_host_f32(oracle._ptr(out), oracle._ptr(x), 7, 33, 1)
    assert np.array_equal(out, oracle.softmax(x, F32))
    REF.log_softmax_kernel_host_f32(oracle._ptr(out), oracle._ptr(x), 7, 33, 1)
    assert np.array_equal(out, oracle.softmax(x, F32, log=True))
    # softmax over a middle axis
    x3 = rng.normal(0, 2, (3, 5, 4)).astype(np.float32); o3 = np.empty_like(x3)
    REF.softmax_kernel_host_f32(oracle._ptr(o3), oracle._ptr(x3), 3, 5, 4)
    assert np.array_equal(o3, oracle.softmax(x3, F32, dim=1))
    REF.relu_kernel_host_f32.argtypes = [vp, vp, sz]
    REF.relu_kernel_host_f32(oracle._ptr(out), oracle._ptr(x), x.size)
    assert np.array_equal(out, oracle.relu(x, F32))
    g = rng.normal(0, 1, x.shape).astype(np.float32)
    REF.backwards_relu_host.argtypes = [vp, vp, vp, sz, ctypes.c_int]
    for dt in ALL:
        xs, gs = oracle.to_storage(x, dt), oracle.to_storage(g, dt)
        o = np.empty_like(xs)
        assert REF.backwards_relu_host(oracle._ptr(gs), oracle._ptr(xs), oracle._ptr(o), xs.size, dt) == 0
        assert np.array_equal(o, oracle.backwards_relu(gs, xs, dt)), dt
    REF.backwards_softmax_host.argtypes = [vp, vp, vp, sz, sz, sz, ctypes.c_int]
    for dt in ALL:
        ys = oracle.softmax(oracle.to_storage(x, dt), dt); gs = oracle.to_storage(g, dt)
        o = np.empty_like(ys)
        assert REF.backwards_softmax_host(oracle._ptr(gs), oracle._ptr(ys), oracle._ptr(o), 7, 33, 1, dt) == 0
        assert np.array_equal(o, oracle.backwards_softmax(gs, ys, dt)), dt
    REF.backwards_log_softmax_host.argtypes = [vp, vp, vp, sz, sz, sz, ctypes.c_int]
    for dt in ALL:
        ls = oracle.softmax(oracle.to_storage(x, dt), dt, log=True); gs = oracle.to_storage(g, dt)
        o = np.empty_like(ls)
        assert REF.backwards_log_softmax_host(oracle._ptr(gs), oracle._ptr(ls), oracle._ptr(o), 7, 33, 1, dt) == 0
        assert np.array_equal(o, oracle.backwards_log_softmax(gs, ls, dt)), dt
    # broadcasting add, the Linear bias case
    y = rng.normal(0, 1, (6, 9)).astype(np.float32); b = rng.normal(0, 1, (9,)).astype(np.float32)
    o = np.empty_like(y)
    ip = ctypes.POINTER(ctypes.c_int)
    REF.add_strided_kernel_host_f32.argtypes = [vp, vp, vp, ctypes.c_int, ip, ip, ip, sz]
    arr = lambda *v: (ctypes.c_int * len(v))(*v)
    REF.add_strided_kernel_host_f32(oracle._ptr(o), oracle._ptr(y), oracle._ptr(b), 2, arr(6, 9), arr(9, 1), arr(0, 1), y.size)
    assert np.array_equal(o, oracle.bias_add(y, b, F32))
    REF.sum_all_kernel_host_f32.argtypes = [vp, sz]; REF.sum_all_kernel_host_f32.restype = ctypes.c_float
    assert np.float32(REF.sum_all_kernel_host_f32(oracle._ptr(x), x.size)) == oracle.sum_all(x, F32)[0]


@pytest.mark.parametrize("dt", ALL)
def test_elementwise_closed_forms(dt):
    import torch
    rng = np.random.default_rng(19)
    tol = {F32: 2e-6, F64: 1e-14, F16: 2e-3, BF16: 1.6e-2}[dt]
    x = oracle.to_storage(rng.normal(0, 2, (6, 17)), dt); x64 = oracle.to_f64(x, dt)
    g = oracle.to_storage(rng.normal(0, 1, (6, 17)), dt); g64 = oracle.to_f64(g, dt)
    assert np.array_equal(oracle.to_f64(oracle.relu(x, dt), dt), np.maximum(x64, 0))
    assert np.array_equal(oracle.to_f64(oracle.backwards_relu(g, x, dt), dt), np.where(x64 > 0, g64, 0))
    t = torch.from_numpy(x64)
    assert oracle.rel_err(oracle.to_f64(oracle.softmax(x, dt), dt), torch.softmax(t, -1).numpy()) < tol
    assert oracle.rel_err(oracle.to_f64(oracle.softmax(x, dt, log=True), dt), torch.log_softmax(t, -1).numpy()) < tol
    y = oracle.softmax(x, dt); y64 = oracle.to_f64(y, dt)
    want = y64 * (g64 - (g64 * y64).sum(-1, keepdims=True))
    assert oracle.rel_err(oracle.to_f64(oracle.backwards_softmax(g, y, dt), dt), want) < 4 * tol
    assert oracle.rel_err(oracle.to_f64(oracle.mul_scalar(x, 0.125, dt), dt), x64 * 0.125) < tol
    assert oracle.rel_err(oracle.to_f64(oracle.add(x, g, dt), dt), x64 + g64) < tol
    b = oracle.to_storage(rng.normal(0, 1, (17,)), dt)
    assert oracle.rel_err(oracle.to_f64(oracle.bias_add(x, b, dt), dt), x64 + oracle.to_f64(b, dt)) < tol
    assert oracle.rel_err(oracle.to_f64(oracle.reduce_rows(g, dt), dt), g64.sum(0)) < 4 * tol
    assert abs(oracle.to_f64(oracle.sum_all(g, dt), dt)[0] - g64.sum()) < 40 * tol * np.abs(g64).sum() / 10


def test_reduce_rows_order_top_to_bottom_in_fp32():
    g = np.array([[1e8, 1.0], [1.0, 1e8], [-1e8, 1.0], [1.0, -1e8]], dtype=np.float32)
    want = np.zeros(2, np.float32)
    for i in range(4):
        for j in range(2):
            want[j] = np.float32(want[j] + g[i, j])
    assert np.array_equal(oracle.reduce_rows(g, F32), want)
    assert want.tolist() == [1.0, 0.0]            # a pairwise or fp64 accumulator would give [2, 2]


@pytest.mark.parametrize("dt,tdt,tol", [(F32, "float32", 2e-6), (F64, "float64", 1e-13)])
def test_cross_entropy_vs_torch(dt, tdt, tol):
    import torch
    rng = np.random.default_rng(20)
    logits = oracle.to_storage(rng.normal(0, 3, (32, 10)), dt)
    targets = rng.integers(0, 10, 32)
    loss, grad = oracle.cross_entropy_mean(logits, targets, dt, upstream=1.0)
    t = torch.tensor(logits, dtype=torch.float64, requires_grad=True)
    l = torch.nn.functional.cross_entropy(t, torch.tensor(targets))
    l.backward()
    assert abs(float(loss[0]) - float(l.detach())) < tol * max(1.0, abs(float(l.detach())))
    assert oracle.rel_err(grad, t.grad.numpy()) < tol
    _, grad3 = oracle.cross_entropy_mean(logits, targets, dt, upstream=3.0)
    assert oracle.rel_err(grad3, 3 * t.grad.numpy()) < tol
    with pytest.raises(RuntimeError):
        oracle.cross_entropy_mean(logits, np.full(32, 10), dt)


# --------------------------------------------------------------------------- compositions
@pytest.mark.parametrize("dt,tol", [(F32, 2e-5), (F64, 1e-12)])
def test_mlp_step_vs_torch_autograd(dt, tol):
    import torch
    rng = np.random.default_rng(21)
    dims = [20, 16, 12, 5]
    x = oracle.to_storage(rng.uniform(0, 1, (8, dims[0])), dt)
    ws = [oracle.to_storage(rng.normal(0, np.sqrt(2 / dims[i]), (dims[i], dims[i + 1])), dt) for i in range(3)]
    bs = [oracle.to_storage(rng.normal(0, 0.1, (dims[i + 1],)), dt) for i in range(3)]
    y = rng.integers(0, dims[-1], 8)
    got = oracle.mlp_step(x, ws, bs, y, dt)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tw = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in ws]
    tb = [torch.tensor(b, dtype=torch.float64, requires_grad=True) for b in bs]
    h = tx
    for i in range(3):
        h = h @ tw[i] + tb[i]
        if i < 2:
            h = torch.relu(h)
    loss = torch.nn.functional.cross_entropy(h, torch.tensor(y))
    loss.backward()
    assert abs(float(got["loss"][0]) - float(loss)) < tol * 10
    assert oracle.rel_err(got["dX"], tx.grad.numpy()) < tol
    for i in range(3):
        assert oracle.rel_err(got["dW"][i], tw[i].grad.numpy()) < tol
        assert oracle.rel_err(got["db"][i], tb[i].grad.numpy()) < tol


@pytest.mark.parametrize("dt,tol", [(F32, 2e-5), (F64, 1e-12), (BF16, 3e-2)])
def test_attention_slice_vs_torch_autograd(dt, tol):
    import torch
    rng = np.random.default_rng(22)
    q, k, v, do = [oracle.to_storage(rng.normal(0, 1, (24, 16)), dt) for _ in range(4)]
    got = oracle.attention(q, k, v, dt, scale=0.25, d_out=do)
    tq, tk, tv = [torch.tensor(oracle.to_f64(t, dt), requires_grad=True) for t in (q, k, v)]
    o = torch.softmax((tq @ tk.T) * 0.25, -1) @ tv
    o.backward(torch.tensor(oracle.to_f64(do, dt)))
    assert oracle.rel_err(oracle.to_f64(got["O"], dt), o.detach().numpy()) < tol
    for name, t in (("dQ", tq), ("dK", tk), ("dV", tv)):
        assert oracle.rel_err(oracle.to_f64(got[name], dt), t.grad.numpy()) < tol, name


# --------------------------------------------------------------------------- conv2d lowering
CONV_CASES = [tuple(tuple(v) if isinstance(v, list) else v for v in c) for c in GOLD["conv2d_parity_shapes"]["cases"]]


def _ref_lowering(name, dst, src, C, H, W, k, s, p, d, oH, oW):
    fn = getattr(REF, name)
    assert fn(dst.ctypes.data, src.ctypes.data, C, H, W, k[0], k[1], s[0], s[1], p[0], p[1], d[0], d[1], oH, oW) == 0


@needs_ref
@pytest.mark.parametrize("dt,ty", [(F32, np.float32), (F64, np.float64)])
@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c[0])))
def test_im2col_col2im_bit_equal_to_reference_kernels(dt, ty, case):
    (N, C, H, W), (Co, _, kH, kW), s, p, d, _ = case
    rng = np.random.default_rng(70)
    oH, oW = oracle.conv_out_size(H, kH, s[0], p[0], d[0]), oracle.conv_out_size(W, kW, s[1], p[1], d[1])
    im = rng.standard_normal((C, H, W)).astype(ty)
    col = oracle.im2col(im, (kH, kW), s, p, d, dt)
    want = np.empty_like(col)
    _ref_lowering("im2col_kernel_host_f32" if dt == F32 else "im2col_kernel_host_f64", want, im, C, H, W, (kH, kW), s, p, d, oH, oW)
    assert np.array_equal(col, want)
    # col2im adds into an image that already holds values
    c2 = rng.standard_normal(col.shape).astype(ty)
    base = rng.standard_normal((C, H, W)).astype(ty)
    got = oracle.col2im(base, c2, (kH, kW), s, p, d, dt)
    want_im = base.copy()
    _ref_lowering("col2im_kernel_host_f32" if dt == F32 else "col2im_kernel_host_f64", want_im, c2, C, H, W, (kH, kW), s, p, d, oH, oW)
    assert np.array_equal(got, want_im)


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c[0])))
def test_col2im_is_the_adjoint_of_im2col(case):
    """<im2col(x), c> == <x, col2im(c)> for any x and c: fixes every index of the gather against the scatter."""
    (N, C, H, W), (Co, _, kH, kW), s, p, d, _ = case
    rng = np.random.default_rng(71)
    x = rng.standard_normal((C, H, W))
    col = oracle.im2col(x, (kH, kW), s, p, d, F64)
    c = rng.standard_normal(col.shape)
    back = oracle.col2im(np.zeros((C, H, W)), c, (kH, kW), s, p, d, F64)
    assert abs((col * c).sum() - (x * back).sum()) <= 1e-10 * max(1.0, abs((col * c).sum()))


@pytest.mark.parametrize("dt", [F16, BF16])
def test_lowering_16bit_is_fp32_pivot_then_one_narrowing(dt):
    rng = np.random.default_rng(72)
    C, H, W, k, s, p, d = 3, 7, 6, (3, 2), (2, 1), (1, 1), (1, 2)
    im = oracle.to_storage(rng.standard_normal((C, H, W)), dt)
    col = oracle.im2col(im, k, s, p, d, dt)
    assert np.array_equal(col, oracle.narrow(oracle.im2col(oracle.widen(im, dt), k, s, p, d, F32), dt))
    c2 = oracle.to_storage(rng.standard_normal(col.shape), dt)
    got = oracle.col2im(im, c2, k, s, p, d, dt)
    assert np.array_equal(got, oracle.narrow(oracle.col2im(oracle.widen(im, dt), oracle.widen(c2, dt), k, s, p, d, F32), dt))


@pytest.mark.parametrize("dt", ALL)
def test_conv2d_reference_known_answers(dt):
    for case in GOLD["conv2d_known_answers"]["cases"]:
        x = _st(np.ones(case["x_shape"]), dt); w = _st(np.ones(case["w_shape"]), dt)
        bias = _st(case["bias"], dt) if "bias" in case else None
        s, p = tuple(case.get("stride", (1, 1))), tuple(case.get("pad", (0, 0)))
        y = oracle.conv2d_forward(x, w, bias, s, p, (1, 1), dt)
        assert list(y.shape) == case["out_shape"]
        if "out_sum" in case:
            assert oracle.to_f64(y, dt).sum() == case["out_sum"]
        if "bias_grad_of_sum" in case:
            _, _, db = oracle.conv2d_backward(x, w, _st(np.ones(y.shape), dt), s, p, (1, 1), dt)
            assert list(oracle.to_f64(db, dt)) == case["bias_grad_of_sum"]


def test_conv2d_weight_gradient_vs_central_differences():
    g = GOLD["conv2d_known_answers"]["weight_gradcheck"]
    x = np.array(g["x"], dtype=np.float64).reshape(g["x_shape"]); w = np.array(g["w"], dtype=np.float64).reshape(g["w_shape"])
    y = oracle.conv2d_forward(x, w, None, (1, 1), (0, 0), (1, 1), F64)
    _, dw, _ = oracle.conv2d_backward(x, w, np.ones_like(y), (1, 1), (0, 0), (1, 1), F64, with_bias=False)
    eps = 1e-3
    for i in range(9):
        wp, wm = w.copy().reshape(-1), w.copy().reshape(-1)
        wp[i] += eps; wm[i] -= eps
        num = (oracle.conv2d_forward(x, wp.reshape(w.shape), None, (1, 1), (0, 0), (1, 1), F64).sum()
               - oracle.conv2d_forward(x, wm.reshape(w.shape), None, (1, 1), (0, 0), (1, 1), F64).sum()) / (2 * eps)
        assert abs(dw.reshape(-1)[i] - num) <= 1e-2 * max(1.0, abs(num))


@pytest.mark.parametrize("dt,tdt,tol", [(F32, "float32", 2e-5), (F64, "float64", 1e-12), (BF16, None, 3e-2), (F16, None, 4e-3)])
@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c[0])))
def test_conv2d_vs_torch_autograd(dt, tdt, tol, case):
    """Forward and all three gradients against torch.nn.functional.conv2d in float64 (an independent implementation)."""
    import torch
    xs, ws, s, p, d, has_bias = case
    rng = np.random.default_rng(73)
    x, w = oracle.to_storage(rng.standard_normal(xs), dt), oracle.to_storage(rng.standard_normal(ws) * 0.3, dt)
    b = oracle.to_storage(rng.standard_normal(ws[0]), dt) if has_bias else None
    y = oracle.conv2d_forward(x, w, b, s, p, d, dt)
    dy = oracle.to_storage(rng.standard_normal(y.shape), dt)
    dx, dw, db = oracle.conv2d_backward(x, w, dy, s, p, d, dt, with_bias=has_bias)
    xt = torch.tensor(oracle.to_f64(x, dt), requires_grad=True); wt = torch.tensor(oracle.to_f64(w, dt), requires_grad=True)
    bt = torch.tensor(oracle.to_f64(b, dt), requires_grad=True) if has_bias else None
    yt = torch.nn.functional.conv2d(xt, wt, bt, stride=s, padding=p, dilation=d)
    yt.backward(torch.tensor(oracle.to_f64(dy, dt)))
    assert oracle.rel_err(oracle.to_f64(y, dt), yt.detach().numpy()) <= tol
    assert oracle.rel_err(oracle.to_f64(dx, dt), xt.grad.numpy()) <= tol
    assert oracle.rel_err(oracle.to_f64(dw, dt), wt.grad.numpy()) <= tol
    if has_bias:
        assert oracle.rel_err(oracle.to_f64(db, dt), bt.grad.numpy()) <= tol


# --------------------------------------------------------------------------- LSTM / GRU cells
@needs_ref
@pytest.mark.parametrize("dt,ty", [(F32, np.float32), (F64, np.float64)])
def test_sigmoid_tanh_bit_equal_to_reference_kernels(dt, ty):
    rng = np.random.default_rng(90)
    x = np.concatenate([rng.standard_normal(4000) * 4, [0.0, -0.0, 30.0, -30.0, 100.0, -100.0, 1e-8]]).astype(ty)
    sfx = "f32" if dt == F32 else "f64"
    for mine, name in ((oracle.sigmoid, "sigmoid_kernel_host_" + sfx), (oracle.tanh, "tanh_kernel_host_" + sfx)):
        want = np.empty_like(x)
        assert getattr(REF, name)(want.ctypes.data, x.ctypes.data, x.size) == 0
        assert np.array_equal(mine(x, dt), want), name


@pytest.mark.parametrize("dt", [F16, BF16])
def test_sigmoid_tanh_16bit_is_fp32_pivot_then_one_narrowing(dt):
    rng = np.random.default_rng(91)
    x = oracle.to_storage(rng.standard_normal(3000) * 3, dt)
    assert np.array_equal(oracle.sigmoid(x, dt), oracle.narrow(oracle.sigmoid(oracle.widen(x, dt), F32), dt))
    assert np.array_equal(oracle.tanh(x, dt), oracle.narrow(oracle.tanh(oracle.widen(x, dt), F32), dt))


def _cell_inputs(rng, B, I, H, gates, dt):
    st = lambda a: oracle.to_storage(a, dt)
    return (st(rng.standard_normal((B, I))), st(rng.standard_normal((B, H)) * 0.5), st(rng.standard_normal((B, H)) * 0.5),
            st(rng.standard_normal((I, gates * H)) / np.sqrt(H)), st(rng.standard_normal((H, gates * H)) / np.sqrt(H)),
            st(rng.standard_normal(gates * H) * 0.1), st(rng.standard_normal(gates * H) * 0.1))


@pytest.mark.parametrize("dt,tol", [(F32, 2e-6), (F64, 1e-13), (BF16, 2e-2), (F16, 3e-3)])
@pytest.mark.parametrize("bias", [True, False])
def test_lstm_cell_vs_torch(dt, tol, bias):
    """torch.nn.LSTMCell in float64 (same gate order i, f, g, o; its weights are the transposes) and its autograd."""
    import torch
    rng = np.random.default_rng(92)
    B, I, H = 5, 7, 6
    x, h, c, w_ih, w_hh, b_ih, b_hh = _cell_inputs(rng, B, I, H, 4, dt)
    if not bias:
        b_ih = b_hh = None
    hn, cn, saved = oracle.lstm_cell_forward(x, h, c, w_ih, w_hh, b_ih, b_hh, dt)
    dh, dc = oracle.to_storage(rng.standard_normal((B, H)), dt), oracle.to_storage(rng.standard_normal((B, H)), dt)
    got = oracle.lstm_cell_backward(x, h, c, w_ih, w_hh, saved, dh, dc, dt)
    T = lambda a: torch.tensor(oracle.to_f64(a, dt), requires_grad=True)
    tx, th, tc, tw1, tw2 = T(x), T(h), T(c), T(w_ih), T(w_hh)
    tb1, tb2 = (T(b_ih), T(b_hh)) if bias else (None, None)
    gates = tx @ tw1 + th @ tw2 + ((tb1 + tb2) if bias else 0)
    i_g, f_g, g_g, o_g = gates.chunk(4, 1)
    cn_t = torch.sigmoid(f_g) * tc + torch.sigmoid(i_g) * torch.tanh(g_g)
    hn_t = torch.sigmoid(o_g) * torch.tanh(cn_t)
    cell = torch.nn.LSTMCell(I, H, bias=bias, dtype=torch.float64)                    # the library's own cell agrees with the formula above
    with torch.no_grad():
        cell.weight_ih.copy_(tw1.T); cell.weight_hh.copy_(tw2.T)
        if bias:
            cell.bias_ih.copy_(tb1); cell.bias_hh.copy_(tb2)
    lib_h, lib_c = cell(tx.detach(), (th.detach(), tc.detach()))
    assert torch.allclose(lib_h, hn_t, atol=1e-12) and torch.allclose(lib_c, cn_t, atol=1e-12)
    (hn_t * torch.tensor(oracle.to_f64(dh, dt))).sum().add((cn_t * torch.tensor(oracle.to_f64(dc, dt))).sum()).backward()
    assert oracle.rel_err(oracle.to_f64(hn, dt), hn_t.detach().numpy()) <= tol
    assert oracle.rel_err(oracle.to_f64(cn, dt), cn_t.detach().numpy()) <= tol
    want = [tx.grad, th.grad, tc.grad, tw1.grad, tw2.grad] + ([tb1.grad] if bias else [])
    for name, g, w in zip(("dx", "dh", "dc", "dw_ih", "dw_hh", "db"), got, want):
        assert oracle.rel_err(oracle.to_f64(g, dt), w.numpy()) <= 3 * tol, name


@pytest.mark.parametrize("dt,tol", [(F32, 2e-6), (F64, 1e-13), (BF16, 2e-2), (F16, 3e-3)])
@pytest.mark.parametrize("bias", [True, False])
def test_gru_cell_vs_torch(dt, tol, bias):
    """torch.nn.GRUCell in float64 (gate order r, z, n; n = tanh(i_n + r * (h_n + b_hn)); h' = (1 - z) n + z h)."""
    import torch
    rng = np.random.default_rng(93)
    B, I, H = 4, 6, 5
    x, h, _, w_ih, w_hh, b_ih, b_hh = _cell_inputs(rng, B, I, H, 3, dt)
    if not bias:
        b_ih = b_hh = None
    hn, saved = oracle.gru_cell_forward(x, h, w_ih, w_hh, b_ih, b_hh, dt)
    dh = oracle.to_storage(rng.standard_normal((B, H)), dt)
    got = oracle.gru_cell_backward(x, h, w_ih, w_hh, saved, dh, dt)
    T = lambda a: torch.tensor(oracle.to_f64(a, dt), requires_grad=True)
    tx, th, tw1, tw2 = T(x), T(h), T(w_ih), T(w_hh)
    tb1, tb2 = (T(b_ih), T(b_hh)) if bias else (None, None)
    cell = torch.nn.GRUCell(I, H, bias=bias, dtype=torch.float64)
    params = {"weight_ih": tw1.T, "weight_hh": tw2.T}
    if bias:
        params.update({"bias_ih": tb1, "bias_hh": tb2})
    hn_t = torch.func.functional_call(cell, params, (tx, th))
    (hn_t * torch.tensor(oracle.to_f64(dh, dt))).sum().backward()
    assert oracle.rel_err(oracle.to_f64(hn, dt), hn_t.detach().numpy()) <= tol
    want = [tx.grad, th.grad, tw1.grad, tw2.grad] + ([tb1.grad, tb2.grad] if bias else [])
    for name, g, w in zip(("dx", "dh", "dw_ih", "dw_hh", "db_ih", "db_hh"), got, want):
        assert oracle.rel_err(oracle.to_f64(g, dt), w.numpy()) <= 3 * tol, name


# ---- cross-entropy with every reduction, on logits and on probabilities (reference ops/ops.c:5545-5643, 5412-5543),
# and the gradient of log_softmax (ops/grad_host.c:1428-1500): against torch in float64 and against closed forms
@pytest.mark.parametrize("dt,tdt,tol", [(F32, "float32", 2e-6), (F64, "float64", 1e-13)])
@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_cross_entropy_every_reduction_vs_torch(dt, tdt, tol, reduction):
    import torch
    rng = np.random.default_rng(29)
    batch, classes = 37, 11
    logits = rng.normal(0, 2, (batch, classes)).astype(oracle.NP_STORAGE[dt])
    targets = rng.integers(0, classes, batch)
    up = rng.normal(0, 1, batch if reduction == "none" else 1).astype(oracle.NP_STORAGE[dt])
    t = torch.tensor(logits.astype(np.float64), requires_grad=True)
    l = torch.nn.functional.cross_entropy(t, torch.tensor(targets), reduction=reduction)
    (l * torch.tensor(up.astype(np.float64))).sum().backward()
    loss, grad = oracle.cross_entropy(logits, targets, dt, reduction, True, upstream=up)
    assert loss.shape == ((batch,) if reduction == "none" else (1,))
    np.testing.assert_allclose(loss, l.detach().numpy().reshape(loss.shape), rtol=tol * 10, atol=tol)
    np.testing.assert_allclose(grad, t.grad.numpy(), rtol=tol * 50, atol=tol * 5)
    # the same loss from probabilities: log(p) instead of log_softmax(x), gradient -1 / p at the target only
    probs = oracle.softmax(logits, dt)
    tp = torch.tensor(probs.astype(np.float64), requires_grad=True)
    lp = torch.nn.functional.nll_loss(torch.log(tp), torch.tensor(targets), reduction=reduction)
    (lp * torch.tensor(up.astype(np.float64))).sum().backward()
    loss_p, grad_p = oracle.cross_entropy(probs, targets, dt, reduction, False, upstream=up)
    np.testing.assert_allclose(loss_p, lp.detach().numpy().reshape(loss_p.shape), rtol=tol * 10, atol=tol)
    np.testing.assert_allclose(grad_p, tp.grad.numpy(), rtol=tol * 50, atol=tol * 5)
    assert np.count_nonzero(grad_p) <= batch                 # one entry per row
    if reduction == "mean":                                     # the mean-on-logits path is the older entry, bit for bit
        l0, g0 = oracle.cross_entropy_mean(logits, targets, dt, upstream=float(up[0]))
        assert np.array_equal(l0, loss) and np.array_equal(g0, grad)
    with pytest.raises(RuntimeError):
        oracle.cross_entropy(logits, np.full(batch, classes), dt, reduction)


@pytest.mark.parametrize("dt", ALL)
def test_backwards_log_softmax_vs_torch_and_closed_form(dt):
    import torch
    rng = np.random.default_rng(31)
    x = oracle.to_storage(rng.normal(0, 2, (3, 9, 4)), dt); g = oracle.to_storage(rng.normal(0, 1, (3, 9, 4)), dt)
    for dim in (1, 2, -1):
        y = oracle.softmax(x, dt, dim=dim, log=True)
        got = oracle.to_f64(oracle.backwards_log_softmax(g, y, dt, dim=dim), dt)
        t = torch.tensor(oracle.to_f64(x, dt), requires_grad=True)
        torch.log_softmax(t, dim).backward(torch.tensor(oracle.to_f64(g, dt)))
        tol = {F32: 2e-6, F64: 1e-13, F16: 4e-3, BF16: 3e-2}[dt]
        np.testing.assert_allclose(got, t.grad.numpy(), rtol=tol * 10, atol=tol * 4)
    # a gradient that is constant along the axis: gx = g (1 - n p), and the rows of gx sum to 0 when g sums against p... closed form on one row
    yrow = oracle.softmax(oracle.to_storage(np.array([[0.0, np.log(3.0)]]), dt), dt, log=True)          # p = (1/4, 3/4)
    gx = oracle.to_f64(oracle.backwards_log_softmax(oracle.to_storage(np.array([[1.0, 1.0]]), dt), yrow, dt), dt)
    np.testing.assert_allclose(gx, [[1 - 2 * 0.25, 1 - 2 * 0.75]], rtol=2e-2 if dt in (F16, BF16) else 1e-6)
