"""LSTM and GRU cells on the GPU: the fused element-wise kernels through the C ABI, and op_lstm_cell / op_gru_cell /
LSTMCell / GRUCell through the drop-in module, against the CPU oracle's restatement of the reference's op chain
(recpulse/module.py:255-351) and against torch's cells in float64.

The GEMM tolerances apply (1e-5*sqrt(K) fp32, 1e-12 fp64, 2e-2 for the 16-bit types): the device's expf / tanhf are
not glibc's to the last bit, so nothing here is compared bit for bit except the scatter behind the slice gradient.
"""
import numpy as np
import pytest

import oracle
import recpulse_cuda as rp
from recpulse.module import GRUCell, LSTMCell
from recpulse_amd import capi
from devhelp import ALL, BF16, F16, F32, F64, NAMES, Dev, rand_storage, tol

pytestmark = pytest.mark.gpu
DT_NAME = {F32: "float32", F64: "float64", F16: "float16", BF16: "bfloat16"}
EW_TOL = {F32: 2e-6, F64: 1e-14, F16: 2e-3, BF16: 1e-2}          # element-wise kernels: transcendental ulps and one 16-bit rounding


def _inputs(rng, B, I, H, gates, dt):
    st = lambda a: oracle.to_storage(a, dt)
    return (st(rng.standard_normal((B, I))), st(rng.standard_normal((B, H)) * 0.5), st(rng.standard_normal((B, H)) * 0.5),
            st(rng.standard_normal((I, gates * H)) / np.sqrt(H)), st(rng.standard_normal((H, gates * H)) / np.sqrt(H)),
            st(rng.standard_normal(gates * H) * 0.1), st(rng.standard_normal(gates * H) * 0.1))


def _close(got, want, dt, bound, what):
    assert got.shape == want.shape, what
    assert oracle.rel_err(oracle.to_f64(got, dt), oracle.to_f64(want, dt)) <= bound, what


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("shape", [(5, 6), (33, 128), (64, 520)], ids=lambda s: "x".join(map(str, s)))
def test_lstm_elementwise_kernels(dt, shape):
    B, H = shape
    rng = np.random.default_rng(100)
    gates, c = rand_storage(rng, (B, 4 * H), dt), rand_storage(rng, (B, H), dt)
    b1, b2 = oracle.to_storage(rng.standard_normal(4 * H) * 0.1, dt), oracle.to_storage(rng.standard_normal(4 * H) * 0.1, dt)
    L = capi.lib()
    d_hc, d_act = Dev.empty((B, 2 * H), dt), Dev.empty((B, 4 * H), dt)
    d_g, d_c, d_b1, d_b2 = Dev(gates, dt), Dev(c, dt), Dev(b1, dt), Dev(b2, dt)
    capi.check(L.rp_hip_lstm_cell_forward(d_hc.ptr, d_act.ptr, d_g.ptr, d_b1.ptr, d_b2.ptr, d_c.ptr, H, B, H, dt), "rp_hip_lstm_cell_forward")
    # the reference chain from the pre-activations on
    pre = oracle.add(oracle.add(gates, np.ascontiguousarray(np.broadcast_to(b1, gates.shape)), dt), np.ascontiguousarray(np.broadcast_to(b2, gates.shape)), dt)
    q = [np.ascontiguousarray(pre[:, k * H:(k + 1) * H]) for k in range(4)]
    i_g, f_g, g_g, o_g = oracle.sigmoid(q[0], dt), oracle.sigmoid(q[1], dt), oracle.tanh(q[2], dt), oracle.sigmoid(q[3], dt)
    c_next = oracle.add(oracle.mul(f_g, c, dt), oracle.mul(i_g, g_g, dt), dt)
    tc = oracle.tanh(c_next, dt)
    h_next = oracle.mul(o_g, tc, dt)
    hc, act = d_hc.numpy(), d_act.numpy()
    _close(act, np.concatenate([i_g, f_g, g_g, o_g], axis=1), dt, EW_TOL[dt], "activated gates")
    _close(hc[:, :H], h_next, dt, 2 * EW_TOL[dt], "h_next")
    _close(hc[:, H:], c_next, dt, 2 * EW_TOL[dt], "c_next")
    # backward from the device's own saved values, so that only the backward arithmetic is compared
    dhc = rand_storage(rng, (B, 2 * H), dt)
    d_dg, d_dc, d_dhc = Dev.empty((B, 4 * H), dt), Dev.empty((B, H), dt), Dev(dhc, dt)
    capi.check(L.rp_hip_lstm_cell_backward(d_dg.ptr, d_dc.ptr, d_dhc.ptr, d_act.ptr, d_hc.ptr, d_c.ptr, H, B, H, dt), "rp_hip_lstm_cell_backward")
    a = [np.ascontiguousarray(act[:, k * H:(k + 1) * H]) for k in range(4)]
    saved = (a[0], a[1], a[2], a[3], oracle.tanh(np.ascontiguousarray(hc[:, H:]), dt))
    eye = oracle.to_storage(np.eye(H), dt)                     # identity weights: dx of the oracle's backward is dgates . I^T
    zero_x = oracle.to_storage(np.zeros((B, 4 * H)), dt)
    dh, dc = np.ascontiguousarray(dhc[:, :H]), np.ascontiguousarray(dhc[:, H:])
    want = oracle.lstm_cell_backward(zero_x, np.ascontiguousarray(hc[:, :H]), c, oracle.to_storage(np.eye(4 * H), dt), np.tile(eye, (1, 4)), saved, dh, dc, dt)
    _close(d_dg.numpy(), want[0], dt, 4 * EW_TOL[dt], "dgates")
    _close(d_dc.numpy(), want[2], dt, 4 * EW_TOL[dt], "dc_prev")


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_scatter_strided_places_a_block(dt):
    rng = np.random.default_rng(101)
    full = np.zeros((4, 6, 10), dtype=capi.NP_STORAGE[dt])
    block = rand_storage(rng, (2, 3, 4), dt)
    d_full, d_block = Dev(full, dt), Dev(block, dt)
    import ctypes
    shp = (ctypes.c_int * 3)(2, 3, 4)
    strides = (ctypes.c_longlong * 3)(60 * 1, 10 * 2, 1 * 2)                 # steps 1, 2, 2 over dense strides 60, 10, 1
    off = (1 * 60 + 0 * 10 + 1) * capi.DTYPE_SIZE[dt]
    capi.check(capi.lib().rp_hip_scatter_strided(d_full.buf.at(off), d_block.ptr, 3, shp, strides, block.size, dt), "rp_hip_scatter_strided")
    full[1:3, 0:6:2, 1:9:2] = block
    assert np.array_equal(d_full.numpy(), full)
    assert capi.lib().rp_hip_scatter_strided(d_full.ptr, d_block.ptr, 3, shp, strides, block.size + 1, dt) == -1


# ---- through the drop-in module -------------------------------------------------------------------------------
def _dev(arr, dt, grad=False):
    vals = oracle.to_f64(arr, dt)
    t = rp.from_numpy(np.ascontiguousarray(vals, dtype=np.float64 if dt == F64 else np.float32)).to(device="cuda", dtype=DT_NAME[dt])
    return t.requires_grad_(True) if grad else t


def _host(t):
    return t.to(device="cpu", dtype="float64").to_numpy()


def _seed_loss(outs, ups, dt):
    """sum_k <out_k, up_k> as one scalar, so that out_k receives the upstream gradient up_k."""
    total = None
    for o, u in zip(outs, ups):
        n = int(np.prod(o.shape))
        term = o.reshape([1, n]).op_matmul(_dev(u, dt).reshape([n, 1]))
        total = term if total is None else total.op_add(term)
    return total.op_sum_all()


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("dims", [(5, 7, 8), (32, 64, 128), (3, 40, 24), (16, 64, 64), (64, 512, 512)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("bias", [True, False], ids=["bias", "nobias"])
def test_lstm_cell_step(dt, dims, bias):
    B, I, H = dims
    rng = np.random.default_rng(102)
    x, h, c, w_ih, w_hh, b_ih, b_hh = _inputs(rng, B, I, H, 4, dt)
    if not bias:
        b_ih = b_hh = None
    tx, th, tc, tw1, tw2 = (_dev(a, dt, True) for a in (x, h, c, w_ih, w_hh))
    tb1, tb2 = (_dev(b_ih, dt, True), _dev(b_hh, dt, True)) if bias else (None, None)
    hc = tx.op_lstm_cell(th, tc, tw1, tw2, tb1, tb2)
    assert hc.shape == (B, 2 * H)
    hn, cn = hc.slice([0, 0], [B, H]), hc.slice([0, H], [B, 2 * H])
    want_h, want_c, saved = oracle.lstm_cell_forward(x, h, c, w_ih, w_hh, b_ih, b_hh, dt)
    k = max(I, H)
    assert oracle.rel_err(_host(hn), oracle.to_f64(want_h, dt)) <= tol(dt, k)
    assert oracle.rel_err(_host(cn), oracle.to_f64(want_c, dt)) <= tol(dt, k)
    dh, dc = rand_storage(rng, (B, H), dt), rand_storage(rng, (B, H), dt)
    _seed_loss([hn, cn], [dh, dc], dt).backward()
    want = oracle.lstm_cell_backward(x, h, c, w_ih, w_hh, saved, dh, dc, dt)
    got = [tx.grad, th.grad, tc.grad, tw1.grad, tw2.grad] + ([tb1.grad, tb2.grad] if bias else [])
    names = ("dx", "dh", "dc", "dw_ih", "dw_hh", "db_ih", "db_hh")
    wants = list(want[:5]) + ([want[5], want[5]] if bias else [])
    for name, g, w in zip(names, got, wants):
        assert g.shape == tuple(w.shape), name
        assert oracle.rel_err(_host(g), oracle.to_f64(w, dt)) <= 2 * tol(dt, max(k, 4 * H, B)), name


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("dims", [(5, 7, 8), (32, 64, 128), (3, 40, 24), (16, 64, 64), (64, 512, 512)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("bias", [True, False], ids=["bias", "nobias"])
def test_gru_cell_step(dt, dims, bias):
    B, I, H = dims
    rng = np.random.default_rng(103)
    x, h, _, w_ih, w_hh, b_ih, b_hh = _inputs(rng, B, I, H, 3, dt)
    if not bias:
        b_ih = b_hh = None
    tx, th, tw1, tw2 = (_dev(a, dt, True) for a in (x, h, w_ih, w_hh))
    tb1, tb2 = (_dev(b_ih, dt, True), _dev(b_hh, dt, True)) if bias else (None, None)
    hn = tx.op_gru_cell(th, tw1, tw2, tb1, tb2)
    want_h, saved = oracle.gru_cell_forward(x, h, w_ih, w_hh, b_ih, b_hh, dt)
    k = max(I, H)
    assert hn.shape == (B, H)
    assert oracle.rel_err(_host(hn), oracle.to_f64(want_h, dt)) <= tol(dt, k)
    dh = rand_storage(rng, (B, H), dt)
    _seed_loss([hn], [dh], dt).backward()
    want = oracle.gru_cell_backward(x, h, w_ih, w_hh, saved, dh, dt)
    got = [tx.grad, th.grad, tw1.grad, tw2.grad] + ([tb1.grad, tb2.grad] if bias else [])
    for name, g, w in zip(("dx", "dh", "dw_ih", "dw_hh", "db_ih", "db_hh"), got, want):
        assert g.shape == tuple(w.shape), name
        assert oracle.rel_err(_host(g), oracle.to_f64(w, dt)) <= 2 * tol(dt, max(k, 3 * H, B)), name


@pytest.mark.parametrize("kind", ["lstm", "gru"])
@pytest.mark.parametrize("sizes", [(10, 16), (16, 16)], ids=["in10_hid16", "in16_hid16"])
@pytest.mark.parametrize("dt,bound", [(F64, 1e-11), (F32, 1e-4), (BF16, 5e-2)], ids=["f64", "f32", "bf16"])
def test_unrolled_sequence_vs_torch(kind, dt, bound, sizes):
    """Six time steps through the module (state fed back as views of the packed output for the LSTM), loss on every
    step's h: forward values and every parameter gradient against torch's cell in float64.  With input size = hidden
    size the backward issues its gradient products in pairs, from the second step on accumulating into the weights'
    existing gradients."""
    import torch
    rng = np.random.default_rng(104)
    B, (I, H), steps = 4, sizes, 6
    rp.manual_seed(5)
    cell = (LSTMCell if kind == "lstm" else GRUCell)(I, H).to(device="cuda", dtype=DT_NAME[dt])
    for b in (cell.bias_ih, cell.bias_hh):
        b.copy_(_dev(oracle.to_storage(rng.standard_normal(b.shape[0]) * 0.1, dt), dt)); b.requires_grad_(True)
    xs = [oracle.to_storage(rng.standard_normal((B, I)), dt) for _ in range(steps)]
    ups = [oracle.to_storage(rng.standard_normal((B, H)), dt) for _ in range(steps)]
    state, outs = None, []
    for x in xs:
        if kind == "lstm":
            state = cell(_dev(x, dt), state); outs.append(state[0])
        else:
            state = cell(_dev(x, dt), state); outs.append(state)
    _seed_loss(outs, ups, dt).backward()
    tc = (torch.nn.LSTMCell if kind == "lstm" else torch.nn.GRUCell)(I, H, dtype=torch.float64)
    with torch.no_grad():
        tc.weight_ih.copy_(torch.tensor(_host(cell.weight_ih)).T); tc.weight_hh.copy_(torch.tensor(_host(cell.weight_hh)).T)
        tc.bias_ih.copy_(torch.tensor(_host(cell.bias_ih))); tc.bias_hh.copy_(torch.tensor(_host(cell.bias_hh)))
    tstate, loss = None, 0
    for x, u, o in zip(xs, ups, outs):
        tstate = tc(torch.tensor(oracle.to_f64(x, dt)), tstate)
        th = tstate[0] if kind == "lstm" else tstate
        assert oracle.rel_err(_host(o), th.detach().numpy()) <= bound
        loss = loss + (th * torch.tensor(oracle.to_f64(u, dt))).sum()
    loss.backward()
    assert oracle.rel_err(_host(cell.weight_ih.grad), tc.weight_ih.grad.T.numpy()) <= bound
    assert oracle.rel_err(_host(cell.weight_hh.grad), tc.weight_hh.grad.T.numpy()) <= bound
    assert oracle.rel_err(_host(cell.bias_ih.grad), tc.bias_ih.grad.numpy()) <= bound
    assert oracle.rel_err(_host(cell.bias_hh.grad), tc.bias_hh.grad.numpy()) <= bound


def test_cell_modules_and_argument_errors():
    """reference recpulse/module.py:255-351: parameter names, layouts and initial scale; missing state is zeros."""
    rp.manual_seed(9)
    lstm, gru = LSTMCell(12, 32).to(device="cuda"), GRUCell(12, 32, bias=False).to(device="cuda")
    assert set(lstm.tracked) == {"weight_ih", "weight_hh", "bias_ih", "bias_hh"} and set(gru.tracked) == {"weight_ih", "weight_hh"}
    assert lstm.weight_ih.shape == (12, 128) and lstm.weight_hh.shape == (32, 128) and lstm.bias_ih.shape == (128,)
    assert gru.weight_ih.shape == (12, 96) and gru.weight_hh.shape == (32, 96) and gru.bias_ih is None
    assert abs(_host(lstm.weight_hh).std() - 1 / np.sqrt(32)) < 0.03 and np.all(_host(lstm.bias_hh) == 0)
    x = rp.randn([5, 12], device="cuda")
    h, c = lstm(x)
    zeros = rp.zeros([5, 32], device="cuda")
    h2, c2 = lstm(x, (zeros, zeros))
    assert h.shape == (5, 32) and c.shape == (5, 32) and np.array_equal(_host(h), _host(h2)) and np.array_equal(_host(c), _host(c2))
    assert np.array_equal(_host(gru(x)), _host(gru(x, zeros)))
    with pytest.raises(RuntimeError):
        x.op_lstm_cell(zeros, zeros, gru.weight_ih, lstm.weight_hh, None, None)         # 3H columns where 4H are due
    with pytest.raises(RuntimeError):
        x.op_gru_cell(zeros, gru.weight_ih, gru.weight_hh, lstm.bias_ih, None)           # one bias only
    with pytest.raises(RuntimeError):
        rp.randn([4, 12], device="cuda").op_gru_cell(zeros, gru.weight_ih, gru.weight_hh, None, None)     # batch mismatch


def test_slice_gradient_lands_in_place():
    """reference ops/ops.c:7536-7600: the gradient of a slice is zero outside the slice."""
    x = _dev(np.arange(24, dtype=np.float64).reshape(4, 6), F32, True)
    x.slice([1, 1], [4, 6], [2, 2]).op_sum_all().backward()
    want = np.zeros((4, 6)); want[1:4:2, 1:6:2] = 1
    assert np.array_equal(_host(x.grad), want)
    y = _dev(np.ones((3, 8)), F64, True)
    a, b = y.slice([0, 0], [3, 4]), y.slice([0, 4], [3, 8])
    a.op_mul_scalar(2.0).op_sum_all().op_add(b.op_mul_scalar(3.0).op_sum_all()).backward()
    assert np.array_equal(_host(y.grad), np.concatenate([np.full((3, 4), 2.0), np.full((3, 4), 3.0)], axis=1))
