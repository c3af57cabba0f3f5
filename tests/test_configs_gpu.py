"""The five benchmark configurations at their real sizes, through the C ABI.

Full results are compared with a float64 oracle; the CPU oracle (the
restatement of the reference's own loops) is run in full where it finishes in
seconds and on row slabs elsewhere (every output row is an independent set of
length-K dot products, so a slab is an exact sub-problem).  Size-independent
checks (row-sum checksums, determinism) cover what sampling leaves open.
"""
import ctypes

import numpy as np
import pytest

import oracle
from recpulse_amd import capi
from devhelp import BF16, F16, F32, F64, NAMES, Dev, device_gemm, f64_gemm, rand_storage, scalar_arg, tol

pytestmark = pytest.mark.gpu
L = capi.lib


def _gemm(c, a, b, m, k, n, a_st, b_st, dt, bias=None, batch=1, c_bs=None, accumulate=False):
    capi.gemm(c.ptr, a.ptr, b.ptr, bias.ptr if bias is not None else None, batch, m, k, n, a_st, b_st,
              (m * n if c_bs is None else c_bs, n, 1), accumulate, dt)


# ------------------------------------------------------------------ config 1
def test_config1_linear_forward_fp32():
    rng = np.random.default_rng(0)
    m, k, n = 128, 784, 256
    x = rng.uniform(0, 1, (m, k)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / k), (k, n)).astype(np.float32)
    b = rng.normal(0, 0.1, (n,)).astype(np.float32)
    got = device_gemm(x, w, F32, bias=b)
    want = oracle.linear_forward(x, w, b, F32)
    assert oracle.rel_err(got, want) <= tol(F32, k)
    assert oracle.rel_err(got, x.astype(np.float64) @ w.astype(np.float64) + b) <= tol(F32, k)
    # two-op form (matmul, then the broadcasting add) agrees with the fused epilogue bit for bit
    dx, dw, db = Dev(x, F32), Dev(w, F32), Dev(b, F32)
    y0, y1 = Dev.empty((m, n), F32), Dev.empty((m, n), F32)
    capi.check(L().matmul_kernel_device(y0.ptr, dx.ptr, dw.ptr, m, k, n, F32), "matmul")
    arr = lambda *v: (ctypes.c_int * len(v))(*v)
    capi.check(L().add_strided_kernel_device(y1.ptr, y0.ptr, db.ptr, 2, arr(m, n), arr(n, 1), arr(0, 1), m * n, F32), "add")
    assert np.array_equal(y1.numpy(), got)


# ------------------------------------------------------------------ config 2
def _device_mlp_step(x, ws, bs, y, dt):
    dims = [x.shape[1]] + [w.shape[1] for w in ws]
    batch = x.shape[0]
    nl = len(ws)
    d_x = Dev(x, dt); d_w = [Dev(w, dt) for w in ws]; d_b = [Dev(b, dt) for b in bs]
    d_y = capi.DeviceBuffer.from_numpy(y.astype(np.int32))
    d_z = [Dev.empty((batch, dims[i + 1]), dt) for i in range(nl)]
    d_h = [Dev.empty((batch, dims[i + 1]), dt) for i in range(nl - 1)]
    d_g = [Dev.empty((batch, dims[i + 1]), dt) for i in range(nl)]
    d_gh = [Dev.empty((batch, dims[i + 1]), dt) for i in range(nl - 1)]
    d_dw = [Dev.empty(w.shape, dt) for w in ws]; d_db = [Dev.empty(b.shape, dt) for b in bs]
    d_dx = Dev.empty(x.shape, dt); d_loss = Dev.empty((1,), dt)
    h = d_x
    for i in range(nl):
        m, k, n = batch, dims[i], dims[i + 1]
        _gemm(d_z[i], h, d_w[i], m, k, n, (0, k, 1), (0, n, 1), dt, bias=d_b[i])
        if i + 1 < nl:
            capi.check(L().relu_kernel_device(d_h[i].ptr, d_z[i].ptr, m * n, dt), "relu")
            h = d_h[i]
    capi.check(L().rp_hip_cross_entropy_mean(d_loss.ptr, d_g[-1].ptr, d_z[-1].ptr, d_y.ptr, batch, dims[-1], 1.0, dt), "ce")
    for i in reversed(range(nl)):
        m, k, n = batch, dims[i], dims[i + 1]
        inp = d_x if i == 0 else d_h[i - 1]
        capi.check(L().rp_hip_reduce_rows(d_db[i].ptr, d_g[i].ptr, m, n, 0, dt), "reduce_rows")
        _gemm(d_dw[i], inp, d_g[i], k, m, n, (0, 1, k), (0, n, 1), dt)                    # dW = inpᵀ · g  (view, no copy)
        dst = d_dx if i == 0 else d_gh[i - 1]
        _gemm(dst, d_g[i], d_w[i], m, n, k, (0, n, 1), (0, 1, n), dt)                     # dIn = g · Wᵀ (view, no copy)
        if i > 0:
            capi.check(L().backwards_relu_device(d_gh[i - 1].ptr, d_z[i - 1].ptr, d_g[i - 1].ptr, m * k, dt), "backwards_relu")
    return {"loss": d_loss.numpy(), "logits": d_z[-1].numpy(), "dW": [t.numpy() for t in d_dw],
            "db": [t.numpy() for t in d_db], "dX": d_dx.numpy()}


def test_config2_mlp_forward_backward_fp32():
    rng = np.random.default_rng(1)
    dims = [784, 256, 128, 10]; batch = 256
    x = rng.uniform(0, 1, (batch, dims[0])).astype(np.float32)
    ws = [rng.normal(0, np.sqrt(2.0 / dims[i]), (dims[i], dims[i + 1])).astype(np.float32) for i in range(3)]
    bs = [np.zeros(dims[i + 1], np.float32) for i in range(3)]
    y = rng.integers(0, 10, batch)
    got = _device_mlp_step(x, ws, bs, y, F32)
    want = oracle.mlp_step(x, ws, bs, y, F32)
    t = 1e-5 * np.sqrt(784)
    assert abs(float(got["loss"][0]) - float(want["loss"][0])) <= 1e-5 * abs(float(want["loss"][0]))
    assert oracle.rel_err(got["logits"], want["logits"]) <= t
    assert oracle.rel_err(got["dX"], want["dX"]) <= t
    for i in range(3):
        assert oracle.rel_err(got["dW"][i], want["dW"][i]) <= t, i
        assert oracle.rel_err(got["db"][i], want["db"][i]) <= t, i
    # float64 reference of the same step (torch autograd)
    import torch
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
    assert abs(float(got["loss"][0]) - float(loss.detach())) <= 1e-5 * float(loss.detach())
    assert oracle.rel_err(got["dX"], tx.grad.numpy()) <= t
    for i in range(3):
        assert oracle.rel_err(got["dW"][i], tw[i].grad.numpy()) <= t
        assert oracle.rel_err(got["db"][i], tb[i].grad.numpy()) <= t
    again = _device_mlp_step(x, ws, bs, y, F32)
    for key in ("dX", "logits", "loss"):
        assert np.array_equal(got[key], again[key])            # bit-deterministic across runs


# ------------------------------------------------------------------ config 3
def _square_case(n, dt, rng, slab_rows):
    """forward and both backward GEMMs at n x n x n; returns errors vs float64 (full) and the oracle (row slab)."""
    a, b, dc = (rand_storage(rng, (n, n), dt) for _ in range(3))
    d_a, d_b, d_dc = Dev(a, dt), Dev(b, dt), Dev(dc, dt)
    d_c, d_da, d_db = (Dev.empty((n, n), dt) for _ in range(3))
    rm, tr = (0, n, 1), (0, 1, n)
    _gemm(d_c, d_a, d_b, n, n, n, rm, rm, dt)
    _gemm(d_da, d_dc, d_b, n, n, n, rm, tr, dt)
    _gemm(d_db, d_a, d_dc, n, n, n, tr, rm, dt)
    c, da, db = d_c.numpy(), d_da.numpy(), d_db.numpy()
    a64, b64, dc64 = oracle.to_f64(a, dt), oracle.to_f64(b, dt), oracle.to_f64(dc, dt)
    out = {}
    out["fwd_f64"] = oracle.rel_err(oracle.to_f64(c, dt), a64 @ b64)
    out["dA_f64"] = oracle.rel_err(oracle.to_f64(da, dt), dc64 @ b64.T)
    out["dB_f64"] = oracle.rel_err(oracle.to_f64(db, dt), a64.T @ dc64)
    rows = slab_rows
    bt = np.ascontiguousarray(b.T)
    out["fwd_orc"] = oracle.rel_err(oracle.to_f64(c[rows], dt), oracle.to_f64(oracle.matmul(np.ascontiguousarray(a[rows]), b, dt), dt))
    out["dA_orc"] = oracle.rel_err(oracle.to_f64(da[rows], dt), oracle.to_f64(oracle.matmul(np.ascontiguousarray(dc[rows]), bt, dt), dt))
    out["dB_orc"] = oracle.rel_err(oracle.to_f64(db[rows], dt), oracle.to_f64(oracle.matmul(np.ascontiguousarray(a.T[rows]), dc, dt), dt))
    # checksum: row sums of C against A · (B · 1), a property that needs no second GEMM
    out["checksum"] = oracle.rel_err(oracle.to_f64(c, dt).sum(1), a64 @ b64.sum(1))
    return out


@pytest.mark.parametrize("dt", [BF16, F16], ids=lambda d: NAMES[d])
def test_config3_square_1024_full_oracle(dt):
    rng = np.random.default_rng(2)
    errs = _square_case(1024, dt, rng, slab_rows=np.arange(0, 1024, 8))
    for key, e in errs.items():
        assert e <= tol(dt, 1024), (key, e)


@pytest.mark.parametrize("n,dt,nrows", [(4096, BF16, 2), (4096, F16, 2), (4096, F32, 2), (8192, BF16, 1), (8192, F16, 1)],
                         ids=["4096-bf16", "4096-f16", "4096-f32", "8192-bf16", "8192-f16"])
def test_config3_square_large(n, dt, nrows):
    rng = np.random.default_rng(2)
    rows = np.sort(rng.choice(n, nrows, replace=False))
    errs = _square_case(n, dt, rng, slab_rows=rows)
    for key, e in errs.items():
        assert e <= tol(dt, n), (key, e)


# ------------------------------------------------------------------ config 4
@pytest.mark.parametrize("dt", [BF16, F32], ids=lambda d: NAMES[d])
def test_config4_attention_forward_backward(dt):
    rng = np.random.default_rng(3)
    B, H, S, D = 16, 12, 512, 64
    Z = B * H
    q, k, v, do = (rand_storage(rng, (Z, S, D), dt) for _ in range(4))
    d_q, d_k, d_v, d_do = Dev(q, dt), Dev(k, dt), Dev(v, dt), Dev(do, dt)
    d_s, d_ss, d_p = (Dev.empty((Z, S, S), dt) for _ in range(3))
    d_o = Dev.empty((Z, S, D), dt)
    d_dp, d_dss, d_ds = (Dev.empty((Z, S, S), dt) for _ in range(3))
    d_dq, d_dk, d_dv = (Dev.empty((Z, S, D), dt) for _ in range(3))
    sd, ss = S * D, S * S
    scale = scalar_arg(0.125, dt)
    # forward: S = Q · Kᵀ with Kᵀ the permuted view (strides (S*D, 1, D)), P = softmax(S/8), O = P · V
    _gemm(d_s, d_q, d_k, S, D, S, (sd, D, 1), (sd, 1, D), dt, batch=Z, c_bs=ss)
    capi.check(L().mul_scalar_kernel_device(d_ss.ptr, d_s.ptr, scale, Z * ss, dt), "mul_scalar")
    capi.check(L().softmax_kernel_device(d_p.ptr, d_ss.ptr, Z * S, S, 1, dt), "softmax")
    _gemm(d_o, d_p, d_v, S, S, D, (ss, S, 1), (sd, D, 1), dt, batch=Z, c_bs=sd)
    # backward: dP = dO · Vᵀ, dV = Pᵀ · dO, dS = softmax'(dP) / 8, dQ = dS · K, dK = dSᵀ · Q  (all transposes are views)
    _gemm(d_dp, d_do, d_v, S, D, S, (sd, D, 1), (sd, 1, D), dt, batch=Z, c_bs=ss)
    _gemm(d_dv, d_p, d_do, S, S, D, (ss, 1, S), (sd, D, 1), dt, batch=Z, c_bs=sd)
    capi.check(L().backwards_softmax_device(d_dp.ptr, d_p.ptr, d_dss.ptr, Z * S, S, 1, dt), "backwards_softmax")
    capi.check(L().mul_scalar_kernel_device(d_ds.ptr, d_dss.ptr, scale, Z * ss, dt), "mul_scalar")
    _gemm(d_dq, d_ds, d_k, S, S, D, (ss, S, 1), (sd, D, 1), dt, batch=Z, c_bs=sd)
    _gemm(d_dk, d_ds, d_q, S, S, D, (ss, 1, S), (sd, D, 1), dt, batch=Z, c_bs=sd)
    got = {"O": d_o.numpy(), "dQ": d_dq.numpy(), "dK": d_dk.numpy(), "dV": d_dv.numpy(), "P": d_p.numpy()}

    # Every GEMM of the chain against float64 on the operands the device itself fed it (its own rounded S, P, dS), at the
    # tolerance of a single GEMM: 2e-2 for bfloat16, 1e-5 sqrt(k) for float32.
    f64 = lambda t: oracle.to_f64(t, dt)
    q64, k64, v64, do64 = f64(q), f64(k), f64(v), f64(do)
    p_dev, ds_dev = f64(got["P"]), f64(d_ds.numpy())
    per_gemm = {
        "S=Q.Kt": (f64(d_s.numpy()), np.matmul(q64, k64.transpose(0, 2, 1)), D),
        "O=P.V": (f64(got["O"]), np.matmul(p_dev, v64), S),
        "dP=dO.Vt": (f64(d_dp.numpy()), np.matmul(do64, v64.transpose(0, 2, 1)), D),
        "dV=Pt.dO": (f64(got["dV"]), np.matmul(p_dev.transpose(0, 2, 1), do64), S),
        "dQ=dS.K": (f64(got["dQ"]), np.matmul(ds_dev, k64), S),
        "dK=dSt.Q": (f64(got["dK"]), np.matmul(ds_dev.transpose(0, 2, 1), q64), S),
    }
    for name, (have, want, kk) in per_gemm.items():
        e = oracle.rel_err(have, want)
        assert e <= tol(dt, kk), (name, e)
    del per_gemm, p_dev, ds_dev

    # and the whole chain against float64 autograd: in bfloat16 the roundings of S, S/8, P, dP and dS stack up, so the
    # end-to-end bound is that of the chain (3e-2), not of one GEMM
    import torch
    tq, tk, tv = (torch.tensor(x, requires_grad=True) for x in (q64, k64, v64))
    p64 = torch.softmax(tq @ tk.transpose(1, 2) * 0.125, -1)
    o64 = p64 @ tv
    o64.backward(torch.tensor(do64))
    t_val = 3e-2 if dt == BF16 else 1e-5 * np.sqrt(S)
    assert oracle.rel_err(oracle.to_f64(got["O"], dt), o64.detach().numpy()) <= t_val
    for name, t in (("dQ", tq), ("dK", tk), ("dV", tv)):
        assert oracle.rel_err(oracle.to_f64(got[name], dt), t.grad.numpy()) <= t_val, name
    # the CPU oracle (chain of reference ops) on three slices
    for z in (0, 77, Z - 1):
        want = oracle.attention(q[z], k[z], v[z], dt, scale=0.125, d_out=do[z])
        for name in ("O", "dQ", "dK", "dV", "P"):
            e = oracle.rel_err(oracle.to_f64(got[name][z], dt), oracle.to_f64(want[name], dt))
            assert e <= (2e-2 if dt == BF16 else 1e-5 * np.sqrt(S)), (name, z, e)


# ------------------------------------------------------------------ config 5
@pytest.mark.parametrize("m", [1, 8, 32])
def test_config5a_skinny_bf16(m):
    rng = np.random.default_rng(4)
    k = n = 8192
    a = rand_storage(rng, (m, k), BF16); w = rand_storage(rng, (k, n), BF16)
    got = device_gemm(a, w, BF16)
    assert oracle.rel_err(oracle.to_f64(got, BF16), f64_gemm(a, w, BF16)) <= tol(BF16, k)
    row = [0] if m == 1 else [m - 1]
    want = oracle.matmul(np.ascontiguousarray(a[row]), w, BF16)          # one row through the reference's loop
    assert oracle.rel_err(oracle.to_f64(got[row], BF16), oracle.to_f64(want, BF16)) <= tol(BF16, k)
    assert np.array_equal(got, device_gemm(a, w, BF16))


def test_config5b_fp64_2048():
    rng = np.random.default_rng(4)
    n = 2048
    a = rng.uniform(-1, 1, (n, n)); b = rng.uniform(-1, 1, (n, n))
    got = device_gemm(a, b, F64)
    assert oracle.rel_err(got, a @ b) <= 1e-12
    rows = np.array([0, 1023, 2047])
    want = oracle.matmul(np.ascontiguousarray(a[rows]), b, F64)
    assert oracle.rel_err(got[rows], want) <= 1e-12
    ref = oracle.load_reference()
    if ref is not None:                                                   # the reference's own kernel, where it was built
        assert oracle.rel_err(got[rows], oracle.reference_matmul(ref, np.ascontiguousarray(a[rows]), b, F64)) <= 1e-12
