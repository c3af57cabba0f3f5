"""GPU parity of the GEMM entry points against the CPU oracle and a float64 oracle.

Every case goes through the C ABI (rp_hip_gemm_strided_batched or
matmul_kernel_device).  Small cases are compared with the oracle's full
result; integer-valued cases must match bit for bit.
"""
import json
import os

import numpy as np
import pytest

import oracle
from recpulse_amd import capi
from devhelp import Dev, ALL, BF16, F16, F32, F64, NAMES, device_gemm, elem_strides, f64_gemm, oracle_gemm, rand_storage, tol

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


def _check(got, a, b, dtype, k, **kw):
    want = oracle_gemm(a, b, dtype, **kw)
    want64 = f64_gemm(a, b, dtype, **kw)
    e_orc = oracle.rel_err(oracle.to_f64(got, dtype), oracle.to_f64(want, dtype))
    e_64 = oracle.rel_err(oracle.to_f64(got, dtype), want64)
    assert e_orc <= tol(dtype, k), f"vs oracle {e_orc:.3e} > {tol(dtype, k):.3e}"
    assert e_64 <= tol(dtype, k), f"vs f64 {e_64:.3e} > {tol(dtype, k):.3e}"
    return e_orc, e_64


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_reference_known_answers_bit_exact(dt):
    for key in ("matmul_2x3_3x2", "matmul_identity"):
        g = GOLD[key]
        a = oracle.to_storage(np.array(g["a"], dtype=np.float64), dt)
        b = oracle.to_storage(np.array(g["b"], dtype=np.float64), dt)
        got = device_gemm(a, b, dt)
        assert np.array_equal(oracle.to_f64(got, dt), np.array(g["c"], dtype=np.float64)), key
    for key in ("backward_a", "backward_both_2x2", "backward_nonsquare_2x4_4x3"):
        g = GOLD[key]
        a = oracle.to_storage(np.array(g["a"], dtype=np.float64), dt)
        b = oracle.to_storage(np.array(g["b"], dtype=np.float64), dt)
        dc = oracle.to_storage(np.ones((a.shape[0], b.shape[1])), dt)
        da = device_gemm(dc, b.T, dt)            # dA = dC · Bᵀ, Bᵀ passed as a stride view
        db = device_gemm(a.T, dc, dt)            # dB = Aᵀ · dC
        assert np.array_equal(oracle.to_f64(da, dt), np.array(g["da"], dtype=np.float64)), key
        assert np.array_equal(oracle.to_f64(db, dt), np.array(g["db"], dtype=np.float64)), key


def test_matmul_kernel_device_seam_f64_parity_shapes():
    rng = np.random.default_rng(30)
    g = GOLD["parity_shapes"]
    for m, k, n in g["mkn"]:
        a = rng.uniform(-1, 1, (m, k)); b = rng.uniform(-1, 1, (k, n))
        da, db = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b)
        dc = capi.DeviceBuffer(m * n * 8)
        capi.check(capi.lib().matmul_kernel_device(dc.ptr, da.ptr, db.ptr, m, k, n, F64), "matmul_kernel_device")
        capi.synchronize()
        np.testing.assert_allclose(dc.to_numpy(np.float64, (m, n)), a @ b, rtol=g["rtol"], atol=g["atol"])


LAYOUTS = ["nn", "nt", "tn", "tt"]
HALF = [F16, BF16]


def _operands(rng, m, k, n, dt, layout, dist="normal"):
    a = rand_storage(rng, (m, k), dt, dist) if layout[0] == "n" else rand_storage(rng, (k, m), dt, dist).T
    b = rand_storage(rng, (k, n), dt, dist) if layout[1] == "n" else rand_storage(rng, (n, k), dt, dist).T
    return a, b


SHAPES = [
    (3, 4, 5), (1, 7, 1), (16, 32, 8), (33, 65, 17),          # generic (odd extents)
    (64, 64, 64), (64, 128, 64), (48, 80, 56),                # 64x64 tiles, full and edge
    (128, 192, 128), (256, 64, 384), (200, 136, 264),         # 128x128 tiles, full and edge
    (128, 784, 256),                                          # config 1 shape
]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_small_shapes_all_layouts(dt, layout):
    rng = np.random.default_rng(31)
    for m, k, n in SHAPES:
        a, b = _operands(rng, m, k, n, dt, layout)
        got = device_gemm(a, b, dt)
        _check(got, a, b, dt, k)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_integer_valued_inputs_are_exact(dt):
    """Small integers: every partial sum is exact in every dtype's accumulator, so any order must agree bit for bit."""
    rng = np.random.default_rng(32)
    for (m, k, n), layout in [((64, 64, 64), "nn"), ((128, 128, 128), "tn"), ((40, 24, 72), "nt"), ((130, 96, 66), "tt")]:
        a = oracle.to_storage(rng.integers(-3, 4, (m, k) if layout[0] == "n" else (k, m)).astype(np.float64), dt)
        b = oracle.to_storage(rng.integers(-3, 4, (k, n) if layout[1] == "n" else (n, k)).astype(np.float64), dt)
        a = a if layout[0] == "n" else a.T
        b = b if layout[1] == "n" else b.T
        got = device_gemm(a, b, dt)
        want = oracle_gemm(a, b, dt)
        assert np.array_equal(got, want), (m, k, n, layout)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_bias_and_accumulate_epilogue(dt):
    rng = np.random.default_rng(33)
    for m, k, n in [(5, 9, 7), (64, 64, 64), (128, 784, 256), (72, 40, 136)]:
        a, b = _operands(rng, m, k, n, dt, "nn")
        bias = rand_storage(rng, (n,), dt)
        c0 = rand_storage(rng, (m, n), dt)
        for kw in ({"bias": bias}, {"c_init": c0, "accumulate": True}, {"bias": bias, "c_init": c0, "accumulate": True}):
            got = device_gemm(a, b, dt, **kw)
            _check(got, a, b, dt, k, **kw)
    # exact epilogue: integer data makes the whole chain exact, so the three roundings of the 16-bit chain must agree
    a = oracle.to_storage(rng.integers(-2, 3, (64, 64)).astype(np.float64), dt)
    b = oracle.to_storage(rng.integers(-2, 3, (64, 64)).astype(np.float64), dt)
    bias = oracle.to_storage(rng.integers(-4, 5, (64,)).astype(np.float64), dt)
    c0 = oracle.to_storage(rng.integers(-4, 5, (64, 64)).astype(np.float64), dt)
    got = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True)
    assert np.array_equal(got, oracle_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True))


@pytest.mark.parametrize("dt", [F16, BF16], ids=lambda d: NAMES[d])
def test_16bit_rounding_is_the_references_half_away_from_zero(dt):
    """Products chosen so the fp32 sum sits exactly on a 16-bit tie: round-to-nearest-even would differ."""
    if dt == BF16:
        vals = [257.0, 259.0, -257.0]                        # 257 = 0x1.01p8: tie between 256 and 258 in bf16
    else:
        vals = [2049.0, 2051.0, -2049.0]                     # 2049: tie between 2048 and 2050 in fp16
    m = len(vals)
    a64 = np.zeros((m, 8)); b64 = np.zeros((8, 8))
    for i, v in enumerate(vals):
        a64[i, 0] = 1.0 if v > 0 else -1.0
        a64[i, 1] = 1.0 if v > 0 else -1.0
    b64[0, :] = 1.0
    got_all = []
    for i, v in enumerate(vals):
        b = b64.copy(); b[1, :] = abs(v) - 1.0              # |v|-1 is representable in both 16-bit formats for these values
        a_s = oracle.to_storage(a64[i:i + 1], dt); b_s = oracle.to_storage(b, dt)
        assert oracle.to_f64(b_s, dt)[1, 0] == abs(v) - 1.0
        got = device_gemm(a_s, b_s, dt)
        want = oracle_gemm(a_s, b_s, dt)
        assert np.array_equal(got, want), v
        got_all.append(oracle.to_f64(got, dt)[0, 0])
    assert got_all[0] == (258.0 if dt == BF16 else 2050.0)
    assert got_all[2] == (-258.0 if dt == BF16 else -2050.0)


@pytest.mark.parametrize("m,n,k", [(256, 128, 64), (512, 512, 256)])
def test_fp16_epilogue_rounding_at_the_tile_level(m, n, k):
    """The fp16 epilogue narrows a tile with two instructions per value when every value of it rounds to a normal fp16
    number and with the general rule otherwise.  C[i, j] = hi_i + lo_i * s_j is exact in fp32 and sits on, just above
    or just below a rounding tie of the reference's add-the-first-dropped-bit rule (core/half_precision.h:50-83);
    rows in the upper half of the output also hold zeros, results below the normal range, sums that overflow, and
    infinities, so their tiles take the general path.  Either way: the oracle's bits."""
    rng = np.random.default_rng(37)
    e = rng.integers(-3, 15, m)
    hi = (1.0 + rng.integers(0, 1024, m) / 1024.0) * np.exp2(e) * rng.choice([-1.0, 1.0], m)
    ulp = np.exp2(e - 10.0)
    frac = rng.choice([0.5, 0.5 * (1 + 2.0 ** -10), 0.5 * (1 - 2.0 ** -10), 0.25, 0.0, 0.75], m)
    lo = frac * ulp * np.sign(hi) * rng.choice([-1.0, 1.0], m)
    special = np.arange(m) >= m // 2
    pick = rng.integers(0, 6, m)
    hi = np.where(special & (pick == 0), 0.0, hi); lo = np.where(special & (pick == 0), 0.0, lo)                    # exact zero
    hi = np.where(special & (pick == 1), 2.0 ** -15 * 1.5, hi); lo = np.where(special & (pick == 1), 2.0 ** -24, lo)     # subnormal result
    hi = np.where(special & (pick == 2), 65504.0, hi); lo = np.where(special & (pick == 2), 16.0, lo)               # 65520: the reference's infinity
    hi = np.where(special & (pick == 3), np.inf, hi); lo = np.where(special & (pick == 3), 0.0, lo)
    hi = np.where(special & (pick == 4), 2.0 ** -14, hi); lo = np.where(special & (pick == 4), -(2.0 ** -24), lo)   # just below the smallest normal
    a64 = np.zeros((m, k)); a64[:, 0] = hi; a64[:, 1] = lo
    b64 = np.zeros((k, n)); b64[0, :] = 1.0; b64[1, :] = rng.choice([1.0, -1.0, 0.5, 0.0], n)
    a, b = oracle.to_storage(a64, F16), oracle.to_storage(b64, F16)
    assert np.array_equal(oracle.to_f64(a, F16)[:, :2], a64[:, :2])                  # the construction is representable
    with np.errstate(invalid="ignore", over="ignore"):
        want = oracle_gemm(a, b, F16)
    got = device_gemm(a, b, F16)
    assert capi.last_gemm_kernel().startswith("mfma16_")
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_batched_strided_views(dt):
    rng = np.random.default_rng(34)
    B, H, S, D = 2, 3, 64, 32
    q = rand_storage(rng, (B * H, S, D), dt); kmat = rand_storage(rng, (B * H, S, D), dt)
    kt = kmat.transpose(0, 2, 1)                       # permuted view, no copy
    s = device_gemm(q, kt, dt)
    _check(s, q, kt, dt, D)
    p = rand_storage(rng, (B * H, S, S), dt); v = rand_storage(rng, (B * H, S, D), dt)
    o = device_gemm(p, v, dt)
    _check(o, p, v, dt, S)
    # dV = Pᵀ · dO with Pᵀ a view, odd sizes (generic path with batch)
    p2 = rand_storage(rng, (4, 9, 13), dt); do = rand_storage(rng, (4, 9, 5), dt)
    dv = device_gemm(p2.transpose(0, 2, 1), do, dt)
    _check(dv, p2.transpose(0, 2, 1), do, dt, 9)


@pytest.mark.parametrize("dt", HALF, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("batch,m,k,n", [(3, 256, 128, 384), (13, 200, 96, 136), (37, 128, 192, 128), (192, 512, 128, 128)])
def test_batched_tiled_16bit_every_matrix_and_tile_once(dt, batch, m, k, n):
    """Batched products on the 16-bit tiled kernel, whose workgroups are re-dealt so that an XCD takes a contiguous
    share of the (matrix, tile) pairs: batch sizes that are no multiple of 8, ragged tiles, integer data so that a
    tile computed twice, skipped or taken from another matrix shows as a wrong value (every matrix has its own sum)."""
    rng = np.random.default_rng(36)
    assert capi.gemm_kernel_name(batch, m, k, n, (k, 1), (n, 1), (n, 1), dt).startswith("mfma16_")
    a64 = rng.integers(-2, 3, (batch, m, k)).astype(np.float64)
    b64 = rng.integers(-2, 3, (batch, k, n)).astype(np.float64)
    b64[:, 0, :] = 1.0
    a64[:, :, 0] = (np.arange(batch) % 5 - 2)[:, None]                   # a per-matrix constant added to every output
    a = oracle.to_storage(a64, dt); b = oracle.to_storage(b64, dt)
    got = device_gemm(a, b, dt)
    want = oracle.to_storage(np.einsum("zik,zkj->zij", a64, b64), dt)
    assert np.array_equal(got, want)


def test_sliced_operand_with_offset_and_padding():
    rng = np.random.default_rng(35)
    big_a = rand_storage(rng, (96, 200), F32); big_b = rand_storage(rng, (200, 160), F32)
    a = big_a[16:80, 8:136]          # 64 x 128 window, row stride 200, base offset
    b = big_b[8:136, 32:96]
    got = device_gemm(a, b, F32)
    _check(got, a, b, F32, 128)
    a2 = big_a[::2, ::2]             # no unit stride at all -> generic
    b2 = big_b[:100:1, ::2]
    got = device_gemm(a2, b2, F32)
    _check(got, a2, b2, F32, 100)


@pytest.mark.parametrize("dt", [BF16, F16, F32], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("m", [1, 2, 4, 8])
def test_skinny_rows_streaming_kernel(dt, m):
    rng = np.random.default_rng(36)
    k, n = 2048, 1024
    if m <= 4 or dt == F32:
        assert capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), dt) == "skinny"
    a, b = _operands(rng, m, k, n, dt, "nn")
    bias = rand_storage(rng, (n,), dt)
    got = device_gemm(a, b, dt, bias=bias)
    _check(got, a, b, dt, k, bias=bias)
    got2 = device_gemm(a, b, dt, bias=bias)
    assert np.array_equal(got, got2)                   # split-k partials are combined in a fixed order


@pytest.mark.parametrize("dt", [BF16, F16], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("layout", LAYOUTS)
def test_skinny_rows_mfma_split_k(dt, layout):
    rng = np.random.default_rng(38)
    for m, k, n in [(8, 4096, 1024), (5, 4160, 1032), (32, 8192, 512), (16, 4096, 1024)]:
        if layout[0] == "t" and m % 8:
            continue                                   # a transposed A needs whole 16-byte vectors along m
        a, b = _operands(rng, m, k, n, dt, layout)
        a_st = (a.strides[0] // 2, a.strides[1] // 2); b_st = (b.strides[0] // 2, b.strides[1] // 2)
        want_kernel = _stream_kernel(m, k, n) if layout == "nn" else "mfma16_skinny_32x128"
        assert capi.gemm_kernel_name(1, m, k, n, a_st, b_st, (n, 1), dt) == want_kernel
        bias = rand_storage(rng, (n,), dt); c0 = rand_storage(rng, (m, n), dt)
        got = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True)
        _check(got, a, b, dt, k, bias=bias, c_init=c0, accumulate=True)
        assert np.array_equal(got, device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True))
    # integer data: exact in fp32 whatever the split, so the split-k path must agree with the oracle bit for bit
    a = oracle.to_storage(rng.integers(-2, 3, (8, 4096)).astype(np.float64), dt)
    b = oracle.to_storage(rng.integers(-2, 3, (4096, 1024)).astype(np.float64), dt)
    assert np.array_equal(device_gemm(a, b, dt), oracle_gemm(a, b, dt))


def _stream_kernel(m, k, n):
    """Row-major A and B with at most 32 rows take the streaming kernel unless the split of k it would need makes its
    finish too long (the dispatcher's rule, restated for a device of 256 CUs): then the tiled kernel."""
    groups = -(-n // 128)
    nsplit = min(-(-256 // groups), max(1, k // 256))            # at least two passes of 128 rows per block
    takes = m <= 32 and n % 8 == 0 and k % 8 == 0 and nsplit * m <= 256 and (nsplit <= 8 or k * n >= 1 << 24)
    return "mfma16_stream_32x128" if takes else "mfma16_skinny_32x128"


@pytest.mark.parametrize("m", [1, 3, 5, 8, 11, 16, 17, 27, 32])
def test_streaming_rows_single_launch_finish(m):
    """Row-major A times row-major B with few rows: one launch, the last block of a column group to arrive adds the
    k splits.  Repeated launches must reproduce the first result bit for bit (fixed summation order, counters left
    clean), with ragged k (a partial last round, waves with unequal numbers of rounds) and n (a partial last strip, a
    number of strips that is not a multiple of 8), a bias and an accumulating epilogue."""
    rng = np.random.default_rng(39)
    for dt, k, n in [(BF16, 8192, 4096), (F16, 4104, 4104), (BF16, 1024, 4096), (F16, 1064, 8200), (BF16, 8192, 2048)]:
        a, b = _operands(rng, m, k, n, dt, "nn")
        assert capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), dt) == _stream_kernel(m, k, n)
        if (k, n) != (8192, 2048):
            assert _stream_kernel(m, k, n) == "mfma16_stream_32x128"          # (the shapes meant for the streaming kernel do take it)
        bias = rand_storage(rng, (n,), dt); c0 = rand_storage(rng, (m, n), dt)
        first = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True)
        _check(first, a, b, dt, k, bias=bias, c_init=c0, accumulate=True)
        for _ in range(20):
            assert np.array_equal(first, device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True))
    # integer data is exact in fp32 whatever the split: bit-equal to the oracle, NaN and Inf carried through
    a = oracle.to_storage(rng.integers(-2, 3, (m, 4096)).astype(np.float64), BF16)
    b = oracle.to_storage(rng.integers(-2, 3, (4096, 1024)).astype(np.float64), BF16)
    assert np.array_equal(device_gemm(a, b, BF16), oracle_gemm(a, b, BF16))


@pytest.mark.parametrize("dt", [BF16, F16], ids=lambda d: NAMES[d])
def test_streaming_rows_output_layouts(dt):
    """The streaming kernel writes its output in three ways (one 8-byte vector per four columns without and with
    bias / accumulation, value by value when C's layout has no such vectors), from two places (the k-split finish,
    and the block itself when k is too short to split).  Every layout of C must hold the bits of the dense result,
    and the elements of C's buffer that are not part of C must keep theirs."""
    rng = np.random.default_rng(41)
    for m, k, n in [(8, 2048, 4096), (5, 1024, 32776), (27, 4096, 4104)]:           # 8 splits; no split (257 strips); ragged, 8 splits
        assert capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), dt) == "mfma16_stream_32x128"
        a, b = _operands(rng, m, k, n, dt, "nn")
        bias = rand_storage(rng, (n,), dt); c0 = rand_storage(rng, (m, n), dt)
        for with_epilogue in (False, True):
            kw = dict(bias=bias, c_init=c0, accumulate=True) if with_epilogue else {}
            dense = device_gemm(a, b, dt, **kw)
            _check(dense, a, b, dt, k, **kw)
            da, db, dbias = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b), capi.DeviceBuffer.from_numpy(bias)
            for what, shape, view_of in [("padded rows, vectors", (m, n + 24), lambda buf: buf[:, :n]),
                                         ("odd row pitch", (m, n + 3), lambda buf: buf[:, :n]),
                                         ("column-major", (n, m + 2), lambda buf: buf[:, :m].T)]:
                host = np.full(shape, 0x7e31, dtype=capi.NP_STORAGE[dt])           # a pattern no result has everywhere
                guard = host.copy()
                if with_epilogue:
                    view_of(host)[...] = c0
                c_view = view_of(host)
                dc = capi.DeviceBuffer.from_numpy(host)
                capi.gemm(dc.ptr, da.ptr, db.ptr, dbias.ptr if with_epilogue else None, 1, m, k, n, (0, k, 1), (0, n, 1),
                          (0,) + tuple(elem_strides(c_view)), with_epilogue, dt)
                capi.synchronize()
                out = dc.to_numpy(capi.NP_STORAGE[dt], shape)
                dc.free()
                assert np.array_equal(view_of(out), dense), (what, m, k, n, with_epilogue)
                view_of(out)[...] = 0x7e31
                assert np.array_equal(out, guard), ("wrote outside C", what, m, k, n)
            for d in (da, db, dbias):
                d.free()


@pytest.mark.parametrize("m", [1, 8, 16, 32])
def test_streaming_rows_finish_repeats_bit_for_bit_over_hundreds_of_launches(m):
    """The finish exchanges partial sums between the workgroups of a column group while other groups still stream:
    launched back to back a few hundred times on resident operands (no synchronisation in between), every launch
    must leave the bits of the first one, and the fp64 product stays inside the tolerance."""
    rng = np.random.default_rng(41)
    k = n = 8192
    dt = BF16
    a = rand_storage(rng, (m, k), dt); b = rand_storage(rng, (k, n), dt)
    assert capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), dt) == "mfma16_stream_32x128"
    da, db = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b)
    launches = 300
    outs = [capi.DeviceBuffer(m * n * 2) for _ in range(launches)]
    for dc in outs:
        capi.gemm(dc.ptr, da.ptr, db.ptr, None, 1, m, k, n, (0, k, 1), (0, n, 1), (0, n, 1), False, dt)
    capi.synchronize()
    first = outs[0].to_numpy(np.uint16, (m, n))
    for i, dc in enumerate(outs[1:], 1):
        assert np.array_equal(first, dc.to_numpy(np.uint16, (m, n))), f"launch {i} differs from launch 0"
    want = oracle.to_f64(a, dt) @ oracle.to_f64(b, dt)
    assert oracle.rel_err(oracle.to_f64(first, dt), want) <= tol(dt, k)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_tiled_rows_split_k_ragged(layout):
    """More rows or another operand layout: the tiled kernel splits k across the grid and a second kernel adds the
    partial tiles in split order.  Ragged k (a partial last slab, splits of unequal length) and n (a partial last
    strip, a number of strips that is not a multiple of 8), several row tiles, bias and accumulation; repeated
    launches reproduce the first bit for bit."""
    rng = np.random.default_rng(43)
    for dt, m, k, n in [(BF16, 32, 8192, 2048), (F16, 24, 4104, 1288), (BF16, 17, 1032, 4096), (F16, 104, 4160, 1160), (BF16, 8, 2048, 2048)]:
        if (layout == "nn" and _stream_kernel(m, k, n) != "mfma16_skinny_32x128") or (layout[0] == "t" and m % 8):
            continue                                   # the streaming kernel's case; a transposed A needs whole 16-byte vectors along m
        a, b = _operands(rng, m, k, n, dt, layout)
        a_st = (a.strides[0] // 2, a.strides[1] // 2); b_st = (b.strides[0] // 2, b.strides[1] // 2)
        assert capi.gemm_kernel_name(1, m, k, n, a_st, b_st, (n, 1), dt) == "mfma16_skinny_32x128"
        bias = rand_storage(rng, (n,), dt); c0 = rand_storage(rng, (m, n), dt)
        first = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True)
        _check(first, a, b, dt, k, bias=bias, c_init=c0, accumulate=True)
        for _ in range(10):
            assert np.array_equal(first, device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True))
    # integer data is exact in fp32 whatever the split: bit-equal to the oracle
    a, b = _operands(rng, 40, 4096, 1024, BF16, layout)
    a[...] = oracle.to_storage(rng.integers(-2, 3, a.shape).astype(np.float64), BF16)
    b[...] = oracle.to_storage(rng.integers(-2, 3, b.shape).astype(np.float64), BF16)
    assert np.array_equal(device_gemm(a, b, BF16), oracle_gemm(a, b, BF16))


def test_tiled_rows_repeat_bit_for_bit_over_hundreds_of_launches():
    """The tiled k-split kernel and its combine kernel share one workspace from the pool across back-to-back launches:
    300 launches without synchronisation in between leave the bits of the first."""
    rng = np.random.default_rng(44)
    m, k, n, dt = 40, 8192, 8192, BF16
    a = rand_storage(rng, (m, k), dt); b = rand_storage(rng, (k, n), dt)
    assert capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), dt) == "mfma16_skinny_32x128"
    da, db = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b)
    outs = [capi.DeviceBuffer(m * n * 2) for _ in range(300)]
    for dc in outs:
        capi.gemm(dc.ptr, da.ptr, db.ptr, None, 1, m, k, n, (0, k, 1), (0, n, 1), (0, n, 1), False, dt)
    capi.synchronize()
    first = outs[0].to_numpy(np.uint16, (m, n))
    for i, dc in enumerate(outs[1:], 1):
        assert np.array_equal(first, dc.to_numpy(np.uint16, (m, n))), f"launch {i} differs from launch 0"
    want = oracle.to_f64(a, dt) @ oracle.to_f64(b, dt)
    assert oracle.rel_err(oracle.to_f64(first, dt), want) <= tol(dt, k)


def test_streaming_rows_both_exchanges_give_the_same_bits(tmp_path):
    """The k-split finish goes through the XCD's own L2 when workgroup placement was verified, and through memory at
    device scope otherwise (RP_HIP_DISABLE=l2_exchange forces that, read once per process): a child process computes
    the same products the other way, and the bits must agree (same partial sums, same order)."""
    import subprocess
    import sys
    code = (
        "import sys, numpy as np\n"
        "sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
        "from devhelp import device_gemm, rand_storage, BF16, F16\n"
        "rng = np.random.default_rng(42)\n"
        "out = {}\n"
        "for i, (dt, m, k, n) in enumerate([(BF16, 1, 8192, 8192), (BF16, 8, 8192, 8192), (F16, 16, 4104, 1288), (BF16, 11, 2048, 2048), (BF16, 32, 8192, 8192), (F16, 27, 4104, 1288)]):\n"
        "    a = rand_storage(rng, (m, k), dt); b = rand_storage(rng, (k, n), dt)\n"
        "    out[str(i)] = device_gemm(a, b, dt)\n"
        "np.savez(sys.argv[1], **out)\n"
    ) % (os.path.dirname(os.path.abspath(__file__)), os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    results = []
    for flag in ("", "l2_exchange"):
        path = str(tmp_path / f"exchange_{flag or 'on'}.npz")
        env = dict(os.environ, RP_HIP_DISABLE=flag)
        subprocess.run([sys.executable, "-c", code, path], check=True, env=env, timeout=300)
        results.append(np.load(path))
    for key in results[0].files:
        assert np.array_equal(results[0][key], results[1][key]), f"case {key}: the two exchanges disagree"


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_pair_of_separately_allocated_matrices_in_one_launch(dt):
    """Batch strides of either sign: a batch of two whose second matrices are separate allocations, addressed by their
    distances from the first (how a recurrent cell's backward issues its input-side and recurrent-side products
    together).  Every matrix must equal the oracle's product of its own operands, whichever of the two allocations
    lies higher in memory; the deep-k shape takes the k-split kernel with a batch, the short-k one the resident kernel."""
    rng = np.random.default_rng(45)
    es = np.dtype(capi.NP_STORAGE[dt]).itemsize
    cases = [(64, 4096, 1024, "nt"), (1024, 64, 4096, "tn"), (33, 70, 65, "nn"), (64, 2048, 512, "nn")]
    if dt == F64:
        cases = cases[2:]
    for m, k, n, layout in cases:
        mats = []
        for _ in range(2):
            a, b = _operands(rng, m, k, n, dt, layout)
            c0 = rand_storage(rng, (m, n), dt)
            mats.append((a, b, c0))
        for accumulate in (False, True):
            for order in ((0, 1), (1, 0)):
                # allocations in the given order, so that both signs of every distance occur
                bufs = {}
                for i in order:
                    a, b, c0 = mats[i]
                    # (an operand view starts at its buffer's first element: uploading a dense copy of the view's
                    # transpose-free form and passing the view's strides addresses the same elements)
                    bufs[i] = (capi.DeviceBuffer.from_numpy(np.ascontiguousarray(a if layout[0] == "n" else a.T)),
                               capi.DeviceBuffer.from_numpy(np.ascontiguousarray(b if layout[1] == "n" else b.T)),
                               capi.DeviceBuffer.from_numpy(c0))
                a0, b0, _ = mats[0]
                dist = [(bufs[1][j].ptr - bufs[0][j].ptr) for j in range(3)]
                assert all(d % es == 0 for d in dist)
                a_st = (dist[0] // es,) + tuple(elem_strides(a0)); b_st = (dist[1] // es,) + tuple(elem_strides(b0))
                capi.gemm(bufs[0][2].ptr, bufs[0][0].ptr, bufs[0][1].ptr, None, 2, m, k, n, a_st, b_st, (dist[2] // es, n, 1), accumulate, dt)
                capi.synchronize()
                if dt in (BF16, F16) and k >= 2048 and k * n >= 1 << 22:
                    assert capi.last_gemm_kernel() == "mfma16_skinny_32x128"
                for i in (0, 1):
                    a, b, c0 = mats[i]
                    got = bufs[i][2].to_numpy(capi.NP_STORAGE[dt], (m, n))
                    _check(got, a, b, dt, k, c_init=c0 if accumulate else None, accumulate=accumulate)
                for i in (0, 1):
                    for d in bufs[i]:
                        d.free()


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_ragged_small_outputs_deep_k(dt):
    """Outputs that no vector kernel takes (n = 10, odd strides) with a deep k.  16-bit: the generic kernel splits k
    across blocks and a scalar kernel adds the partials in split order.  fp32: the one-launch 16 x 16-tile kernel, whose
    four waves add their partial tiles in wave order.  Either way results repeat bit for bit.  fp64 does not split."""
    rng = np.random.default_rng(40)
    for m, k, n, layout in [(128, 256, 10, "tn"), (256, 128, 10, "nn"), (17, 1000, 3, "nn"), (70, 333, 65, "nt"), (10, 96, 130, "tt")]:
        a, b = _operands(rng, m, k, n, dt, layout)
        es = a.itemsize
        if dt != F64:              # 2-element vectors fit some of these shapes, which then take the fp64 MFMA kernel
            name = capi.gemm_kernel_name(1, m, k, n, (a.strides[0] // es, a.strides[1] // es), (b.strides[0] // es, b.strides[1] // es), (n, 1), dt)
            assert name == ("tiny32_16x16" if dt == F32 else "generic")
        bias = rand_storage(rng, (n,), dt); c0 = rand_storage(rng, (m, n), dt)
        got = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True)
        _check(got, a, b, dt, k, bias=bias, c_init=c0, accumulate=True)
        assert np.array_equal(got, device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True))


def test_large_tile_kernel_multi_slab():
    """4096 x 4096 outputs select the 256x256 tile; checked against float64 everywhere and the oracle on a row slab."""
    rng = np.random.default_rng(37)
    m = n = 4096; k = 320
    for dt, layout in [(BF16, "nn"), (F16, "tn"), (BF16, "nt"), (F16, "tt")]:
        assert capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), dt) == "mfma16_256x256"
        a, b = _operands(rng, m, k, n, dt, layout)
        got = device_gemm(a, b, dt)
        e64 = oracle.rel_err(oracle.to_f64(got, dt), f64_gemm(a, b, dt))
        assert e64 <= tol(dt, k), e64
        rows = np.array([0, 1, 255, 256, 1023, 2048, 4095])
        want = oracle.matmul(np.ascontiguousarray(a[rows]), np.ascontiguousarray(b), dt)
        assert oracle.rel_err(oracle.to_f64(got[rows], dt), oracle.to_f64(want, dt)) <= tol(dt, k)


def test_large_tile_kernel_with_ragged_edges():
    """The 256 x 256 tile (16 x 16 x 32 MFMAs) on extents that are whole vectors but not whole tiles or slabs: rows and
    columns past the edge, a last slab of 8, every layout, bias and accumulation.  Float64 everywhere, the oracle on
    sampled rows (first and last of tiles, the ragged last tile)."""
    rng = np.random.default_rng(43)
    m, k, n = 2856, 264, 3080
    for dt, layout, epilogue in [(BF16, "nn", True), (F16, "nt", False), (BF16, "tn", False), (F16, "tt", True)]:
        a, b = _operands(rng, m, k, n, dt, layout)
        es = a.itemsize
        assert capi.gemm_kernel_name(1, m, k, n, (a.strides[0] // es, a.strides[1] // es), (b.strides[0] // es, b.strides[1] // es), (n, 1), dt) == "mfma16_256x256"
        bias = rand_storage(rng, (n,), dt) if epilogue else None
        c0 = rand_storage(rng, (m, n), dt) if epilogue else None
        got = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=epilogue)
        assert oracle.rel_err(oracle.to_f64(got, dt), f64_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=epilogue)) <= tol(dt, k)
        rows = np.array([0, 15, 16, 255, 256, 2559, 2560, 2815, 2816, 2855])
        _check(got[rows], np.ascontiguousarray(a[rows]), b, dt, k, bias=bias, c_init=None if c0 is None else np.ascontiguousarray(c0[rows]), accumulate=epilogue)


def test_wide_tiles_for_outputs_of_at_most_64_rows():
    """Up to 64 rows and many columns: 64 x 128 tiles while k is short, 64 x 256 beyond (one row of waves, no MFMA
    spent on rows past m).  Full tiles and ragged ones, every layout, bias and accumulation; checked against float64
    everywhere and against the oracle on a slab of columns."""
    rng = np.random.default_rng(41)
    cases = [(64, 192, 32768, BF16, "nn", "mfma16_64x128", False), (33, 64, 32776, F16, "nt", "mfma16_64x128", True),
             (64, 1088, 32768, BF16, "tn", "mfma16_64x256", True), (40, 1096, 32776, F16, "nn", "mfma16_64x256", False)]
    for m, k, n, dt, layout, kernel, epilogue in cases:
        a, b = _operands(rng, m, k, n, dt, layout)
        es = a.itemsize
        assert capi.gemm_kernel_name(1, m, k, n, (a.strides[0] // es, a.strides[1] // es), (b.strides[0] // es, b.strides[1] // es), (n, 1), dt) == kernel
        bias = rand_storage(rng, (n,), dt) if epilogue else None
        c0 = rand_storage(rng, (m, n), dt) if epilogue else None
        got = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=epilogue)
        assert oracle.rel_err(oracle.to_f64(got, dt), f64_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=epilogue)) <= tol(dt, k)
        cols = np.r_[0:8, 250:262, n - 9:n]
        _check(got[:, cols], a, np.ascontiguousarray(b[:, cols]), dt, k, bias=None if bias is None else bias[cols],
               c_init=None if c0 is None else np.ascontiguousarray(c0[:, cols]), accumulate=epilogue)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_linear_backward_in_one_call(dt):
    """rp_hip_linear_backward against two GEMM calls with swapped strides and rp_hip_reduce_rows: the same bits,
    whether the three run as one launch (small float32 layers) or one after the other; outputs that are absent,
    accumulated into, and a transposed x view."""
    rng = np.random.default_rng(42)
    L = capi.lib()
    for m, k, n in ((256, 784, 256), (256, 128, 10), (37, 50, 21), (512, 1024, 512)):
        x, w, dy = rand_storage(rng, (m, k), dt), rand_storage(rng, (k, n), dt), rand_storage(rng, (m, n), dt)
        dx0, dw0, db0 = rand_storage(rng, (m, k), dt), rand_storage(rng, (k, n), dt), rand_storage(rng, (n,), dt)
        d_x, d_w, d_dy = Dev(x, dt), Dev(w, dt), Dev(dy, dt)
        for acc in (0, 1):
            want_dx, want_dw, want_db = Dev(dx0, dt), Dev(dw0, dt), Dev(db0, dt)
            capi.gemm(want_dx.ptr, d_dy.ptr, d_w.ptr, None, 1, m, n, k, (0, n, 1), (0, 1, n), (0, k, 1), bool(acc), dt)
            capi.gemm(want_dw.ptr, d_x.ptr, d_dy.ptr, None, 1, k, m, n, (0, 1, k), (0, n, 1), (0, n, 1), bool(acc), dt)
            capi.check(L.rp_hip_reduce_rows(want_db.ptr, d_dy.ptr, m, n, acc, dt), "reduce_rows")
            got_dx, got_dw, got_db = Dev(dx0, dt), Dev(dw0, dt), Dev(db0, dt)
            capi.check(L.rp_hip_linear_backward(got_dx.ptr, got_dw.ptr, got_db.ptr, d_dy.ptr, d_x.ptr, d_w.ptr, m, k, n,
                                                k, 1, n, 1, k, 1, n, 1, acc, acc, acc, dt), "linear_backward")
            assert np.array_equal(got_dx.numpy(), want_dx.numpy()) and np.array_equal(got_dw.numpy(), want_dw.numpy())
            assert np.array_equal(got_db.numpy(), want_db.numpy())
        # only some of the outputs, and x given as the transpose of a [k, m] array
        xt = Dev(np.ascontiguousarray(x.T), dt)
        only_w, only_b = Dev(dw0, dt), Dev(db0, dt)
        capi.check(L.rp_hip_linear_backward(None, only_w.ptr, None, d_dy.ptr, xt.ptr, None, m, k, n, 1, m, n, 1, k, 1, n, 1, 0, 0, 0, dt), "dw only")
        capi.check(L.rp_hip_linear_backward(None, None, only_b.ptr, d_dy.ptr, None, None, m, k, n, k, 1, n, 1, k, 1, n, 1, 0, 0, 0, dt), "db only")
        ref_w = Dev(dw0, dt)
        capi.gemm(ref_w.ptr, d_x.ptr, d_dy.ptr, None, 1, k, m, n, (0, 1, k), (0, n, 1), (0, n, 1), False, dt)
        assert oracle.rel_err(oracle.to_f64(only_w.numpy(), dt), oracle.to_f64(ref_w.numpy(), dt)) <= tol(dt, m)     # another layout may take another kernel
        ref_b = Dev(db0, dt)
        capi.check(L.rp_hip_reduce_rows(ref_b.ptr, d_dy.ptr, m, n, 0, dt), "reduce_rows")
        assert np.array_equal(only_b.numpy(), ref_b.numpy())
        _, dwant = oracle.matmul_backward(x, w, dy, dt)
        assert oracle.rel_err(oracle.to_f64(only_w.numpy(), dt), oracle.to_f64(dwant, dt)) <= tol(dt, m)
    assert L.rp_hip_linear_backward(None, None, None, None, None, None, 4, 4, 4, 4, 1, 4, 1, 4, 1, 4, 1, 0, 0, 0, dt) == -1


def test_batch_longer_than_a_grid_axis():
    """70 000 tiny matrices in one call (the batch index rides on a grid axis of at most 65 535 blocks), A shared by
    all of them through a zero batch stride."""
    rng = np.random.default_rng(41)
    Z, m, k, n = 70000, 4, 8, 4
    a = rand_storage(rng, (m, k), F32); b = rand_storage(rng, (Z, k, n), F32)
    da, db, dc = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b), capi.DeviceBuffer(Z * m * n * 4)
    capi.gemm(dc.ptr, da.ptr, db.ptr, None, Z, m, k, n, (0, k, 1), (k * n, n, 1), (m * n, n, 1), False, F32)
    got = dc.to_numpy(np.float32, (Z, m, n))
    want = np.einsum("ik,zkj->zij", a.astype(np.float64), b.astype(np.float64))
    assert oracle.rel_err(got.astype(np.float64), want) <= 1e-6
    assert oracle.rel_err(got[69999].astype(np.float64), oracle.matmul(a, np.ascontiguousarray(b[69999]), F32).astype(np.float64)) <= tol(F32, k)


def test_rejects_bad_arguments():
    lib = capi.lib()
    d = capi.DeviceBuffer(64)
    assert lib.rp_hip_gemm_strided_batched(d.ptr, d.ptr, None, None, 1, 2, 2, 2, 0, 2, 1, 0, 2, 1, 0, 2, 1, 0, F32) == -1
    assert lib.rp_hip_gemm_strided_batched(d.ptr, d.ptr, d.ptr, None, 1, 0, 2, 2, 0, 2, 1, 0, 2, 1, 0, 2, 1, 0, F32) == -1
    assert lib.rp_hip_gemm_strided_batched(d.ptr, d.ptr, d.ptr, None, 1, 2, 2, 2, 0, 2, 1, 0, 2, 1, 0, 2, 1, 0, 7) == -1
    assert lib.matmul_kernel_device(d.ptr, d.ptr, d.ptr, 2, -1, 2, F32) == -1
    assert b"extent" in lib.rp_hip_last_error()


def test_small_fp32_outputs_take_one_launch():
    """fp32 outputs of fewer than 64 tiles of 64 x 64 with k <= 2048 (the layers of the configuration-2 MLP): every layout,
    ragged extents, batches, bias and accumulation, against the oracle and float64; repeatable bit for bit."""
    rng = np.random.default_rng(43)
    cases = [(256, 784, 256, "nn"), (256, 256, 784, "nt"), (784, 256, 256, "tn"), (256, 128, 10, "nn"), (1, 5, 1, "nn"), (33, 2048, 47, "tt"),
             (100, 17, 300, "nt"), (16, 16, 16, "nn"), (250, 1, 250, "tn")]
    for m, k, n, layout in cases:
        a, b = _operands(rng, m, k, n, F32, layout)
        assert capi.gemm_kernel_name(1, m, k, n, (a.strides[0] // 4, a.strides[1] // 4), (b.strides[0] // 4, b.strides[1] // 4), (n, 1), F32) == "tiny32_16x16"
        bias = rand_storage(rng, (n,), F32); c0 = rand_storage(rng, (m, n), F32)
        for kw in ({}, {"bias": bias}, {"bias": bias, "c_init": c0, "accumulate": True}):
            got = device_gemm(a, b, F32, **kw)
            _check(got, a, b, F32, k, **kw)
            assert np.array_equal(got, device_gemm(a, b, F32, **kw))
    # beyond the limits the tiled kernels take over
    assert capi.gemm_kernel_name(1, 256, 4096, 256, (4096, 1), (256, 1), (256, 1), F32) != "tiny32_16x16"
    assert capi.gemm_kernel_name(1, 512, 512, 512, (512, 1), (512, 1), (512, 1), F32) != "tiny32_16x16"
    # a small batch of small matrices on stride views
    a3 = rand_storage(rng, (5, 40, 24), F32); b3 = rand_storage(rng, (5, 24, 56), F32)
    assert capi.gemm_kernel_name(5, 40, 24, 56, (24, 1), (56, 1), (56, 1), F32) == "tiny32_16x16"
    got = device_gemm(a3, b3, F32)
    assert oracle.rel_err(got, oracle_gemm(a3, b3, F32)) <= tol(F32, 24)
    got_t = device_gemm(a3, np.ascontiguousarray(b3.transpose(0, 2, 1)).transpose(0, 2, 1), F32)
    assert oracle.rel_err(got_t, oracle_gemm(a3, b3, F32)) <= tol(F32, 24)



# ---- fp32 products with a short reduction (k <= 64) and many tiles: the resident cross-tile kernel (every layout, ragged
# extents, k below a whole slab, bias, accumulation) and, for operands with unit stride along their free index, the
# kernel that multiplies straight out of registers
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("batch,m,k,n", [(8, 512, 64, 512), (9, 500, 64, 456), (33, 250, 44, 300), (16, 384, 36, 512), (40, 256, 20, 256)])
def test_fp32_short_reduction_batched(layout, batch, m, k, n):
    rng = np.random.default_rng(61)
    a = rand_storage(rng, (batch, m, k), F32) if layout[0] == "n" else rand_storage(rng, (batch, k, m), F32).transpose(0, 2, 1)
    b = rand_storage(rng, (batch, k, n), F32) if layout[1] == "n" else rand_storage(rng, (batch, n, k), F32).transpose(0, 2, 1)
    a_rc, b_rc = [s // 4 for s in a.strides[1:]], [s // 4 for s in b.strides[1:]]
    kernel = capi.gemm_kernel_name(batch, m, k, n, a_rc, b_rc, (n, 1), F32)
    if layout == "tn" and k > 32 and m % 4 == 0 and n % 4 == 0:
        assert kernel == "direct32_128x128"
    elif m % 4 == 0 and n % 4 == 0 and k % 4 == 0:
        assert kernel == "mfma32_128x128"
    got = device_gemm(a, b, F32)
    _check(got, a, b, F32, k)
    bias = rand_storage(rng, (n,), F32)
    c0 = rand_storage(rng, (batch, m, n), F32)
    got = device_gemm(a, b, F32, bias=bias, c_init=c0, accumulate=True)
    _check(got, a, b, F32, k, bias=bias, c_init=c0, accumulate=True)


# ---- fp32, k <= 64, both operands contiguous along k, at least one 128 x 128 tile per CU: the resident kernel whose
# fetching waves fill LDS directly and whose multiplying waves store the previous tile between the MFMAs
PIPE32_SHAPES = [(16, 512, 64, 512), (20, 500, 64, 456), (48, 250, 44, 300), (32, 384, 36, 512), (70, 256, 20, 256), (300, 130, 8, 129), (260, 128, 32, 128),
                   (1, 2048, 64, 2048), (3, 1100, 60, 1300)]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("batch,m,k,n", PIPE32_SHAPES)
def test_fp32_pipelined_kernel(batch, m, k, n, layout):
    rng = np.random.default_rng(63)
    # free-index-major operands need 16-byte aligned k rows: pad the storage, view the first m (n) entries
    mp, npad = (m + 3) // 4 * 4, (n + 3) // 4 * 4
    a = rand_storage(rng, (batch, m, k), F32) if layout[0] == "n" else rand_storage(rng, (batch, k, mp), F32)[:, :, :m].transpose(0, 2, 1)
    b = rand_storage(rng, (batch, k, npad), F32)[:, :, :n] if layout[1] == "n" else rand_storage(rng, (batch, n, k), F32).transpose(0, 2, 1)
    a_rc, b_rc = [x // 4 for x in a.strides[1:]], [x // 4 for x in b.strides[1:]]
    assert capi.gemm_kernel_name(batch, m, k, n, a_rc, b_rc, (n, 1), F32) == "pipe32_128x128"
    got = device_gemm(a, b, F32)
    _check(got, a, b, F32, k)
    assert capi.last_gemm_kernel() == "pipe32_128x128"
    # the bias per column is this kernel's too
    bias = rand_storage(rng, (n,), F32)
    got = device_gemm(a, b, F32, bias=bias)
    assert capi.last_gemm_kernel() == "pipe32_128x128"
    _check(got, a, b, F32, k, bias=bias)
    # an accumulated C is not (reading C back leaves the product bound by memory either way): the same call must still be
    # right through the kernel that takes over
    c0 = rand_storage(rng, (batch, m, n), F32)
    got = device_gemm(a, b, F32, bias=bias, c_init=c0, accumulate=True)
    assert capi.last_gemm_kernel() != "pipe32_128x128"
    _check(got, a, b, F32, k, bias=bias, c_init=c0, accumulate=True)


def test_fp32_pipelined_kernel_views_and_strided_output():
    """Rows that are slices of wider arrays (row pitch above k), a batch stride that skips entries, and C written through
    row / column strides of a transposed, padded output: nothing outside the addressed elements may change."""
    rng = np.random.default_rng(64)
    batch, m, k, n = 24, 384, 48, 512
    wide_a = rand_storage(rng, (2 * batch, m, 80), F32)
    wide_b = rand_storage(rng, (batch, n, 96), F32)
    a = wide_a[::2, :, 16:16 + k]                              # every other batch entry, columns 16..63 of 80
    b = wide_b[:, :, 32:32 + k].transpose(0, 2, 1)
    assert capi.gemm_kernel_name(batch, m, k, n, (80, 1), (1, 96), (n, 1), F32) == "pipe32_128x128"
    got = device_gemm(a, b, F32)
    _check(got, a, b, F32, k)
    # C[z] stored transposed inside a padded [n + 3, m + 5] plane
    pitch = m + 5
    plane = (n + 3) * pitch
    c0 = rand_storage(rng, (batch, n + 3, pitch), F32)
    da, db, dc = capi.DeviceBuffer.from_numpy(wide_a), capi.DeviceBuffer.from_numpy(wide_b), capi.DeviceBuffer.from_numpy(c0)
    capi.gemm(dc.ptr, da.at(16 * 4), db.at(32 * 4), None, batch, m, k, n, (2 * m * 80, 80, 1), (n * 96, 1, 96), (plane, 1, pitch), False, F32)
    capi.synchronize()
    out = dc.to_numpy(np.float32, (batch, n + 3, pitch))
    for d in (da, db, dc):
        d.free()
    assert np.array_equal(out[:, :n, :m], got.transpose(0, 2, 1))
    assert np.array_equal(out[:, n:, :], c0[:, n:, :]) and np.array_equal(out[:, :, m:], c0[:, :, m:])


# ---- the same for bf16 / fp16 (C row-major, n in whole eights): narrowing and stores between the MFMAs of the next tile
PIPE16_SHAPES = [(16, 512, 64, 512), (20, 500, 64, 456), (48, 250, 40, 296), (32, 384, 32, 512), (70, 256, 16, 256), (300, 130, 8, 136), (3, 1100, 56, 1304)]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("dt", HALF, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("batch,m,k,n", PIPE16_SHAPES)
def test_16bit_pipelined_kernel(batch, m, k, n, dt, layout):
    rng = np.random.default_rng(65)
    mp = (m + 7) // 8 * 8                                   # m-major A needs 16-byte aligned k rows: pad the storage
    a = rand_storage(rng, (batch, m, k), dt) if layout[0] == "n" else rand_storage(rng, (batch, k, mp), dt)[:, :, :m].transpose(0, 2, 1)
    b = rand_storage(rng, (batch, k, n), dt) if layout[1] == "n" else rand_storage(rng, (batch, n, k), dt).transpose(0, 2, 1)
    es = a.itemsize
    a_rc, b_rc = [x // es for x in a.strides[1:]], [x // es for x in b.strides[1:]]
    if layout[0] == "n" or m % 8 == 0:
        assert capi.gemm_kernel_name(batch, m, k, n, a_rc, b_rc, (n, 1), dt) == "pipe16_128x128"
    got = device_gemm(a, b, dt)
    _check(got, a, b, dt, k)
    resident = layout[0] == "n" or m % 8 == 0
    bias = rand_storage(rng, (n,), dt)
    got = device_gemm(a, b, dt, bias=bias)                                     # the bias per column is this kernel's too
    if resident:
        assert capi.last_gemm_kernel() == "pipe16_128x128"
    _check(got, a, b, dt, k, bias=bias)
    c0 = rand_storage(rng, (batch, m, n), dt)
    got = device_gemm(a, b, dt, bias=bias, c_init=c0, accumulate=True)          # accumulation is not: through the one that takes over
    assert capi.last_gemm_kernel() != "pipe16_128x128"
    _check(got, a, b, dt, k, bias=bias, c_init=c0, accumulate=True)


def test_16bit_pipelined_kernel_free_index_major_bit_exact():
    """The lowered convolution's dcol = W^T.dy shape (both operands with unit stride along their free index), small
    integers: every sum is exact, so the product must equal the oracle's bits."""
    rng = np.random.default_rng(73)
    batch, m, k, n = 8, 576, 64, 3136
    for dt in HALF:
        w64 = rng.integers(-2, 3, (k, m)).astype(np.float64)            # shared by the batch (batch stride 0)
        dy64 = rng.integers(-2, 3, (batch, k, n)).astype(np.float64)
        w_st, dy_st = oracle.to_storage(w64, dt), oracle.to_storage(dy64, dt)
        dw, ddy, dc = capi.DeviceBuffer.from_numpy(w_st), capi.DeviceBuffer.from_numpy(dy_st), capi.DeviceBuffer(batch * m * n * 2)
        assert capi.gemm_kernel_name(batch, m, k, n, (1, m), (n, 1), (n, 1), dt) == "pipe16_128x128"
        capi.gemm(dc.ptr, dw.ptr, ddy.ptr, None, batch, m, k, n, (0, 1, m), (k * n, n, 1), (m * n, n, 1), False, dt)
        capi.synchronize()
        out = dc.to_numpy(capi.NP_STORAGE[dt], (batch, m, n))
        for d in (dw, ddy, dc):
            d.free()
        assert np.array_equal(out, oracle.to_storage(np.matmul(w64.T[None], dy64), dt)), dt


@pytest.mark.parametrize("dt", HALF, ids=lambda d: NAMES[d])
def test_16bit_pipelined_kernel_bit_exact_and_padded_rows(dt):
    """Small integers (every sum exact, so any order gives the oracle's bits), operands that are slices of wider arrays,
    and C with a row pitch above n: nothing outside the addressed elements may change."""
    rng = np.random.default_rng(66)
    batch, m, k, n = 24, 384, 48, 504
    wide_a = oracle.to_storage(rng.integers(-3, 4, (2 * batch, m, 80)).astype(np.float64), dt)
    wide_b = oracle.to_storage(rng.integers(-3, 4, (batch, n, 96)).astype(np.float64), dt)
    a = wide_a[::2, :, 16:16 + k]
    b = wide_b[:, :, 32:32 + k].transpose(0, 2, 1)
    want = np.matmul(oracle.to_f64(np.ascontiguousarray(a), dt), oracle.to_f64(np.ascontiguousarray(b), dt))
    pitch = n + 16
    c0 = rand_storage(rng, (batch, m + 2, pitch), dt)
    da, db, dc = capi.DeviceBuffer.from_numpy(wide_a), capi.DeviceBuffer.from_numpy(wide_b), capi.DeviceBuffer.from_numpy(c0)
    assert capi.gemm_kernel_name(batch, m, k, n, (80, 1), (1, 96), (pitch, 1), dt) == "pipe16_128x128"
    capi.gemm(dc.ptr, da.at(16 * 2), db.at(32 * 2), None, batch, m, k, n, (2 * m * 80, 80, 1), (n * 96, 1, 96), ((m + 2) * pitch, pitch, 1), False, dt)
    capi.synchronize()
    out = dc.to_numpy(capi.NP_STORAGE[dt], (batch, m + 2, pitch))
    for d in (da, db, dc):
        d.free()
    assert np.array_equal(oracle.to_f64(out[:, :m, :n], dt), want)
    assert np.array_equal(out[:, m:, :], c0[:, m:, :]) and np.array_equal(out[:, :, n:], c0[:, :, n:])


# ---- bf16 / fp16 outputs of at most 64 columns with at least one 128-row tile per CU: the resident kernel that streams k
# slabs of A and B into LDS, every operand layout, ragged m, n below 64, k that ends inside a slab
PIPE16K_SHAPES = [(64, 512, 512, 64), (70, 504, 200, 40), (300, 136, 72, 64), (1, 32768, 96, 56), (130, 256, 64, 64), (33, 1000, 328, 8)]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("dt", HALF, ids=lambda d: NAMES[d])
@pytest.mark.parametrize("batch,m,k,n", PIPE16K_SHAPES)
def test_16bit_narrow_output_kernel(batch, m, k, n, dt, layout):
    rng = np.random.default_rng(67)
    a = rand_storage(rng, (batch, m, k), dt) if layout[0] == "n" else rand_storage(rng, (batch, k, m), dt).transpose(0, 2, 1)
    b = rand_storage(rng, (batch, k, n), dt) if layout[1] == "n" else rand_storage(rng, (batch, n, k), dt).transpose(0, 2, 1)
    es = a.itemsize
    a_rc, b_rc = [x // es for x in a.strides[1:]], [x // es for x in b.strides[1:]]
    assert capi.gemm_kernel_name(batch, m, k, n, a_rc, b_rc, (n, 1), dt) == "pipe16k_128x64"
    got = device_gemm(a, b, dt)
    _check(got, a, b, dt, k)
    # the bias per column and the accumulation into C (the gradient rule of ops/ops.c:6781-6788) are this kernel's too
    bias = rand_storage(rng, (n,), dt)
    c0 = rand_storage(rng, (batch, m, n), dt)
    for kw in ({"bias": bias}, {"c_init": c0, "accumulate": True}, {"bias": bias, "c_init": c0, "accumulate": True}):
        got = device_gemm(a, b, dt, **kw)
        assert capi.last_gemm_kernel() == "pipe16k_128x64", kw.keys()
        _check(got, a, b, dt, k, **kw)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_16bit_narrow_output_kernel_bit_exact(layout):
    """Small integers: every partial sum is exact in fp32, so the product must equal the oracle's bits in any summation
    order; C rows with a pitch above n must keep what lies between them."""
    rng = np.random.default_rng(68)
    batch, m, k, n, dt = 40, 1024, 448, 48, BF16
    a64 = rng.integers(-2, 3, (batch, m, k) if layout[0] == "n" else (batch, k, m)).astype(np.float64)
    b64 = rng.integers(-2, 3, (batch, k, n) if layout[1] == "n" else (batch, n, k)).astype(np.float64)
    a_st, b_st = oracle.to_storage(a64, dt), oracle.to_storage(b64, dt)
    a = a_st if layout[0] == "n" else a_st.transpose(0, 2, 1)
    b = b_st if layout[1] == "n" else b_st.transpose(0, 2, 1)
    want = np.matmul(a64 if layout[0] == "n" else a64.transpose(0, 2, 1), b64 if layout[1] == "n" else b64.transpose(0, 2, 1))
    pitch = 64
    c0 = rand_storage(rng, (batch, m, pitch), dt)
    da, db, dc = capi.DeviceBuffer.from_numpy(a_st), capi.DeviceBuffer.from_numpy(b_st), capi.DeviceBuffer.from_numpy(c0)
    es = 2
    a_str = (m * k,) + tuple(x // es for x in a.strides[1:])
    b_str = (k * n,) + tuple(x // es for x in b.strides[1:])
    assert capi.gemm_kernel_name(batch, m, k, n, a_str[1:], b_str[1:], (pitch, 1), dt) == "pipe16k_128x64"
    capi.gemm(dc.ptr, da.ptr, db.ptr, None, batch, m, k, n, a_str, b_str, (m * pitch, pitch, 1), False, dt)
    capi.synchronize()
    out = dc.to_numpy(capi.NP_STORAGE[dt], (batch, m, pitch))
    for d in (da, db, dc):
        d.free()
    assert np.array_equal(oracle.to_f64(out[:, :, :n], dt), want)
    assert np.array_equal(out[:, :, n:], c0[:, :, n:])
    # with a bias and an accumulated C every rounding of the reference's three ops is visible (sums up to 1800 need more
    # than bf16's 8 bits): the oracle's bits, from this kernel and from the tiled one that a misaligned bias falls back to
    bias = oracle.to_storage(rng.integers(-40, 41, (n + 8,)).astype(np.float64), dt)
    cacc = oracle.to_storage(rng.integers(-300, 301, (batch, m, n)).astype(np.float64), dt)
    want_bits = oracle_gemm(a, b, dt, bias=bias[:n], c_init=cacc, accumulate=True)
    got = device_gemm(a, b, dt, bias=bias[:n], c_init=cacc, accumulate=True)
    assert capi.last_gemm_kernel() == "pipe16k_128x64"
    assert np.array_equal(got, want_bits)
    dbias_all = capi.DeviceBuffer.from_numpy(bias)
    da, db, dc = capi.DeviceBuffer.from_numpy(a_st), capi.DeviceBuffer.from_numpy(b_st), capi.DeviceBuffer.from_numpy(cacc)
    capi.gemm(dc.ptr, da.ptr, db.ptr, dbias_all.at(2), batch, m, k, n, a_str, b_str, (m * n, n, 1), True, dt)      # bias at a 2-byte offset
    capi.synchronize()
    assert capi.last_gemm_kernel() != "pipe16k_128x64"
    tiled = dc.to_numpy(capi.NP_STORAGE[dt], (batch, m, n))
    assert np.array_equal(tiled, oracle_gemm(a, b, dt, bias=bias[1:n + 1], c_init=cacc, accumulate=True))
    for d in (da, db, dc, dbias_all):
        d.free()


# ---- and its fp32 twin (any n up to 64, any C strides)
PIPE32K_SHAPES = [(64, 512, 512, 64), (70, 500, 200, 40), (300, 130, 72, 64), (1, 32768, 96, 50), (130, 256, 32, 64), (33, 1000, 324, 7)]


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("batch,m,k,n", PIPE32K_SHAPES)
def test_fp32_narrow_output_kernel(batch, m, k, n, layout):
    rng = np.random.default_rng(69)
    # free-index-major operands need 16-byte aligned k rows: pad the storage, view the first m (n) entries
    mp, npad = (m + 3) // 4 * 4, (n + 3) // 4 * 4
    a = rand_storage(rng, (batch, m, k), F32) if layout[0] == "n" else rand_storage(rng, (batch, k, mp), F32)[:, :, :m].transpose(0, 2, 1)
    b = rand_storage(rng, (batch, k, npad), F32)[:, :, :n] if layout[1] == "n" else rand_storage(rng, (batch, n, k), F32).transpose(0, 2, 1)
    a_rc, b_rc = [x // 4 for x in a.strides[1:]], [x // 4 for x in b.strides[1:]]
    assert capi.gemm_kernel_name(batch, m, k, n, a_rc, b_rc, (n, 1), F32) == "pipe32k_128x64"
    got = device_gemm(a, b, F32)
    _check(got, a, b, F32, k)
    # the bias per column and the accumulation into C are this kernel's too
    bias = rand_storage(rng, (n,), F32)
    c0 = rand_storage(rng, (batch, m, n), F32)
    for kw in ({"bias": bias}, {"c_init": c0, "accumulate": True}, {"bias": bias, "c_init": c0, "accumulate": True}):
        got = device_gemm(a, b, F32, **kw)
        assert capi.last_gemm_kernel() == "pipe32k_128x64", kw.keys()
        _check(got, a, b, F32, k, **kw)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_fp32_narrow_output_kernel_bit_exact_strided_c(layout):
    """Small integers (every partial sum exact: the oracle's bits in any order) into a transposed, padded C."""
    rng = np.random.default_rng(70)
    batch, m, k, n = 40, 1024, 448, 48
    a64 = rng.integers(-3, 4, (batch, m, k) if layout[0] == "n" else (batch, k, m)).astype(np.float32)
    b64 = rng.integers(-3, 4, (batch, k, n) if layout[1] == "n" else (batch, n, k)).astype(np.float32)
    a = a64 if layout[0] == "n" else a64.transpose(0, 2, 1)
    b = b64 if layout[1] == "n" else b64.transpose(0, 2, 1)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)
    pitch = m + 3
    c0 = rand_storage(rng, (batch, n + 1, pitch), F32)
    da, db, dc = capi.DeviceBuffer.from_numpy(a64), capi.DeviceBuffer.from_numpy(b64), capi.DeviceBuffer.from_numpy(c0)
    a_str = (m * k,) + tuple(x // 4 for x in a.strides[1:])
    b_str = (k * n,) + tuple(x // 4 for x in b.strides[1:])
    assert capi.gemm_kernel_name(batch, m, k, n, a_str[1:], b_str[1:], (1, pitch), F32) == "pipe32k_128x64"
    capi.gemm(dc.ptr, da.ptr, db.ptr, None, batch, m, k, n, a_str, b_str, ((n + 1) * pitch, 1, pitch), False, F32)
    capi.synchronize()
    out = dc.to_numpy(np.float32, (batch, n + 1, pitch))
    for d in (da, db, dc):
        d.free()
    assert np.array_equal(out[:, :n, :m], want.transpose(0, 2, 1))
    assert np.array_equal(out[:, n:, :], c0[:, n:, :]) and np.array_equal(out[:, :, m:], c0[:, :, m:])
    # integers with a bias and an accumulated C: exact in fp32, so the oracle's bits
    bias = rng.integers(-40, 41, (n,)).astype(np.float32)
    cacc = rng.integers(-300, 301, (batch, m, n)).astype(np.float32)
    got = device_gemm(a, b, F32, bias=bias, c_init=cacc, accumulate=True)
    assert capi.last_gemm_kernel() == "pipe32k_128x64"
    assert np.array_equal(got, oracle_gemm(a, b, F32, bias=bias, c_init=cacc, accumulate=True))


def test_fp32_short_reduction_integers_bit_exact():
    """Small integers: every partial sum is exact, so the product must equal the oracle's bit for bit in any summation order."""
    rng = np.random.default_rng(62)
    batch, m, k, n = 16, 512, 64, 512
    for layout in LAYOUTS:
        a = rng.integers(-3, 4, (batch, m, k) if layout[0] == "n" else (batch, k, m)).astype(np.float32)
        b = rng.integers(-3, 4, (batch, k, n) if layout[1] == "n" else (batch, n, k)).astype(np.float32)
        a = a if layout[0] == "n" else a.transpose(0, 2, 1)
        b = b if layout[1] == "n" else b.transpose(0, 2, 1)
        got = device_gemm(a, b, F32)
        assert np.array_equal(got, np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)), layout
