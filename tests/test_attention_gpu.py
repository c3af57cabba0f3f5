"""Fused attention forward (rp_hip_attention_forward) against a float64 oracle and the reference's op chain."""
import ctypes

import numpy as np
import pytest

import oracle
from recpulse_amd import capi
from devhelp import BF16, F16, F32, NAMES, Dev, rand_storage

pytestmark = pytest.mark.gpu


def _fused(q, k, v, dt, scale, q_view=None, want_lse=False):
    """q, k, v: storage arrays [Z, S, D] (dense).  Returns O (and the log-sum-exp rows)."""
    Z, sq, d = q.shape
    sk = k.shape[1]
    dq, dk, dv = Dev(q, dt), Dev(k, dt), Dev(v, dt)
    do = Dev.empty((Z, sq, d), dt)
    lse = capi.DeviceBuffer(Z * sq * 4) if want_lse else None
    rc = capi.lib().rp_hip_attention_forward(do.ptr, dq.ptr, dk.ptr, dv.ptr, lse.ptr if lse else None, Z, sq, sk, d,
                                             sq * d, d, sk * d, d, sk * d, d, sq * d, d, float(scale), dt)
    capi.check(rc, "rp_hip_attention_forward")
    out = do.numpy()
    return (out, lse.to_numpy(np.float32, (Z, sq))) if want_lse else out


def _f64(q, k, v, dt, scale):
    q64, k64, v64 = (oracle.to_f64(x, dt) for x in (q, k, v))
    s = np.einsum("zqd,zkd->zqk", q64, k64) * scale
    m = s.max(-1, keepdims=True)
    e = np.exp(s - m)
    l = e.sum(-1, keepdims=True)
    return np.einsum("zqk,zkd->zqd", e / l, v64), (m + np.log(l))[..., 0]


FWD_TOL = {BF16: 1e-2, F16: 2e-3, F32: 2e-6}
BWD_TOL = {BF16: 2e-2, F16: 4e-3, F32: 1e-5}


@pytest.mark.parametrize("dt", [BF16, F16, F32], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("shape", [(6, 512, 512, 64), (3, 200, 333, 64), (2, 130, 65, 32), (2, 96, 160, 128), (1, 1, 1, 64), (5, 33, 31, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_fused_attention_forward(dt, shape):
    Z, sq, sk, d = shape
    rng = np.random.default_rng(60)
    q, k, v = rand_storage(rng, (Z, sq, d), dt), rand_storage(rng, (Z, sk, d), dt), rand_storage(rng, (Z, sk, d), dt)
    scale = 1.0 / np.sqrt(d)
    got, lse = _fused(q, k, v, dt, scale, want_lse=True)
    want, want_lse = _f64(q, k, v, dt, scale)
    # probabilities are rounded to the tensor dtype before the second product, as the reference's P is
    assert oracle.rel_err(oracle.to_f64(got, dt), want) <= FWD_TOL[dt]
    assert np.max(np.abs(lse - want_lse)) <= (1e-3 if dt != F32 else 1e-5) * max(1.0, np.max(np.abs(want_lse)))
    # the reference's chain (matmul, mul_scalar, softmax, matmul with a rounding after each) on one slice
    ref = oracle.attention(q[Z - 1], k[Z - 1], v[Z - 1], dt, scale=scale)["O"]
    assert oracle.rel_err(oracle.to_f64(got[Z - 1], dt), oracle.to_f64(ref, dt)) <= (2e-2 if dt != F32 else 1e-5 * np.sqrt(max(sk, d)))
    # running it again gives the same bits
    assert np.array_equal(got, _fused(q, k, v, dt, scale))


def test_fused_attention_large_scores_and_config4_size():
    """Scores far from zero (the online softmax must not overflow) at the configuration's full size."""
    rng = np.random.default_rng(61)
    Z, S, D = 16 * 12, 512, 64
    q = oracle.to_storage(rng.normal(0, 4, (Z, S, D)), BF16); k = oracle.to_storage(rng.normal(0, 4, (Z, S, D)), BF16)
    v = rand_storage(rng, (Z, S, D), BF16)
    got = _fused(q, k, v, BF16, 0.125)
    assert np.all(np.isfinite(oracle.to_f64(got, BF16)))
    sel = [0, 77, Z - 1]
    want, _ = _f64(q[sel], k[sel], v[sel], BF16, 0.125)
    assert oracle.rel_err(oracle.to_f64(got[sel], BF16), want) <= 1e-2


def test_fused_attention_rejects_bad_arguments():
    d = capi.DeviceBuffer(4096)
    L = capi.lib()
    assert L.rp_hip_attention_forward(d.ptr, d.ptr, d.ptr, d.ptr, None, 1, 4, 4, 48, 192, 48, 192, 48, 192, 48, 192, 48, 1.0, BF16) == -1
    assert b"head dimension" in L.rp_hip_last_error()
    assert L.rp_hip_attention_forward(d.ptr, d.ptr, d.ptr, d.ptr, None, 1, 4, 4, 64, 256, 64, 256, 64, 256, 64, 256, 64, 1.0, capi.F64) == -1
    assert L.rp_hip_attention_forward(d.ptr, d.ptr, d.ptr, d.ptr, None, 1, 4, 4, 96, 384, 96, 384, 96, 384, 96, 384, 96, 1.0, capi.F32) == -1
    assert L.rp_hip_attention_forward(d.ptr, d.ptr, d.ptr, d.ptr, None, 1, 4, 4, 64, 256, 66, 256, 64, 256, 64, 256, 64, 1.0, capi.F32) == -1      # row stride not a multiple of 16 bytes
    assert L.rp_hip_attention_forward(d.ptr, d.ptr, d.ptr, d.ptr, None, 1, 4, 4, 64, 256, 60, 256, 64, 256, 64, 256, 64, 1.0, BF16) == -1


def _f64_backward(q, k, v, g, dt, scale):
    """Closed-form gradients of O = softmax(scale q k^T) v in float64 (the chain rule the reference's autograd applies)."""
    q64, k64, v64, g64 = (oracle.to_f64(x, dt) for x in (q, k, v, g))
    s = np.einsum("zqd,zkd->zqk", q64, k64) * scale
    e = np.exp(s - s.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    dv = np.einsum("zqk,zqd->zkd", p, g64)
    dp = np.einsum("zqd,zkd->zqk", g64, v64)
    ds = p * (dp - (dp * p).sum(-1, keepdims=True)) * scale
    return np.einsum("zqk,zkd->zqd", ds, k64), np.einsum("zqk,zqd->zkd", ds, q64), dv


def _fused_backward(q, k, v, g, dt, scale):
    Z, sq, d = q.shape
    sk = k.shape[1]
    dq, dk, dv, dg = Dev(q, dt), Dev(k, dt), Dev(v, dt), Dev(g, dt)
    do = Dev.empty((Z, sq, d), dt)
    lse = capi.DeviceBuffer(Z * sq * 4)
    L = capi.lib()
    capi.check(L.rp_hip_attention_forward(do.ptr, dq.ptr, dk.ptr, dv.ptr, lse.ptr, Z, sq, sk, d,
                                          sq * d, d, sk * d, d, sk * d, d, sq * d, d, float(scale), dt), "rp_hip_attention_forward")
    gq, gk, gv = Dev.empty((Z, sq, d), dt), Dev.empty((Z, sk, d), dt), Dev.empty((Z, sk, d), dt)
    capi.check(L.rp_hip_attention_backward(gq.ptr, gk.ptr, gv.ptr, dq.ptr, dk.ptr, dv.ptr, do.ptr, dg.ptr, lse.ptr, Z, sq, sk, d,
                                           sq * d, d, sk * d, d, sk * d, d, sq * d, d, sq * d, d, float(scale), dt), "rp_hip_attention_backward")
    return gq.numpy(), gk.numpy(), gv.numpy()


@pytest.mark.parametrize("dt", [BF16, F16, F32], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("shape", [(6, 512, 512, 64), (3, 200, 333, 64), (2, 130, 65, 32), (2, 96, 160, 128), (1, 1, 1, 64), (5, 33, 31, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_fused_attention_backward(dt, shape):
    Z, sq, sk, d = shape
    rng = np.random.default_rng(62)
    q, k, v = rand_storage(rng, (Z, sq, d), dt), rand_storage(rng, (Z, sk, d), dt), rand_storage(rng, (Z, sk, d), dt)
    g = rand_storage(rng, (Z, sq, d), dt)
    scale = 1.0 / np.sqrt(d)
    got = _fused_backward(q, k, v, g, dt, scale)
    want = _f64_backward(q, k, v, g, dt, scale)
    # P and dS are rounded to the tensor dtype before they enter a product (as the reference's chain rounds them)
    tol = BWD_TOL[dt]
    for name, a, b in zip(("dQ", "dK", "dV"), got, want):
        assert oracle.rel_err(oracle.to_f64(a, dt), b) <= tol, name
    again = _fused_backward(q, k, v, g, dt, scale)
    assert all(np.array_equal(a, b) for a, b in zip(got, again))


def test_fused_attention_backward_large_scores():
    """Rows whose softmax is nearly one-hot: exp(scale s - lse) must reproduce the forward's probabilities."""
    rng = np.random.default_rng(63)
    Z, S, D = 4, 256, 64
    q = oracle.to_storage(rng.normal(0, 3, (Z, S, D)), BF16); k = oracle.to_storage(rng.normal(0, 3, (Z, S, D)), BF16)
    v, g = rand_storage(rng, (Z, S, D), BF16), rand_storage(rng, (Z, S, D), BF16)
    got = _fused_backward(q, k, v, g, BF16, 0.125)
    want = _f64_backward(q, k, v, g, BF16, 0.125)
    for a, b in zip(got, want):
        assert np.all(np.isfinite(oracle.to_f64(a, BF16)))
        assert oracle.rel_err(oracle.to_f64(a, BF16), b) <= 3e-2


def test_fused_attention_backward_rejects_bad_arguments():
    d = capi.DeviceBuffer(4096)
    L = capi.lib()
    p = d.ptr
    assert L.rp_hip_attention_backward(p, p, p, p, p, p, p, p, p, 1, 4, 4, 48, 192, 48, 192, 48, 192, 48, 192, 48, 192, 48, 1.0, BF16) == -1
    assert b"head dimension" in L.rp_hip_last_error()
    assert L.rp_hip_attention_backward(p, p, p, p, p, p, p, p, None, 1, 4, 4, 64, 256, 64, 256, 64, 256, 64, 256, 64, 256, 64, 1.0, BF16) == -1
    assert L.rp_hip_attention_backward(p, p, p, p, p, p, p, p, p, 1, 4, 4, 64, 256, 64, 256, 64, 256, 64, 256, 64, 256, 64, 1.0, capi.F64) == -1
    assert L.rp_hip_attention_backward(p, p, p, p, p, p, p, p, p, 1, 4, 4, 96, 384, 96, 384, 96, 384, 96, 384, 96, 384, 96, 1.0, capi.F32) == -1


def test_fused_attention_batch_longer_than_a_grid_axis():
    """70 000 heads of 8 x 8 x 32: forward and backward go in two chunks of the batch; checked on both sides of the seam."""
    rng = np.random.default_rng(64)
    Z, S, D = 70000, 8, 32
    q, k, v, g = (rand_storage(rng, (Z, S, D), BF16) for _ in range(4))
    scale = 1.0 / np.sqrt(D)
    sel = [0, 65534, 65535, 65536, Z - 1]
    out = _fused(q, k, v, BF16, scale)
    want, _ = _f64(q[sel], k[sel], v[sel], BF16, scale)
    assert oracle.rel_err(oracle.to_f64(out[sel], BF16), want) <= 1e-2
    got = _fused_backward(q, k, v, g, BF16, scale)
    wants = _f64_backward(q[sel], k[sel], v[sel], g[sel], BF16, scale)
    for a, b in zip(got, wants):
        assert oracle.rel_err(oracle.to_f64(a[sel], BF16), b) <= 2e-2
