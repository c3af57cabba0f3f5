"""GPU parity of the non-GEMM entry points against the CPU oracle."""
import ctypes

import numpy as np
import pytest

import oracle
from recpulse_amd import capi
from devhelp import ALL, BF16, F16, F32, F64, NAMES, Dev, rand_storage, scalar_arg

pytestmark = pytest.mark.gpu
L = capi.lib


def _tol(dt):
    # element-wise ops differ from the oracle only through expf/logf and summation order
    return {F32: 2e-6, F64: 1e-14, F16: 2e-3, BF16: 1.6e-2}[dt]


def _arr(*v):
    return (ctypes.c_int * len(v))(*[int(x) for x in v])


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_flat_maps_bit_exact(dt):
    rng = np.random.default_rng(40)
    for n in (1, 7, 256, 1000, 65537):
        x = rand_storage(rng, (n,), dt); y = rand_storage(rng, (n,), dt)
        dx, dy, do = Dev(x, dt), Dev(y, dt), Dev.empty((n,), dt)
        capi.check(L().add_kernel_device(do.ptr, dx.ptr, dy.ptr, n, dt), "add")
        assert np.array_equal(do.numpy(), oracle.add(x, y, dt))
        capi.check(L().mul_scalar_kernel_device(do.ptr, dx.ptr, scalar_arg(0.125, dt), n, dt), "mul_scalar")
        assert np.array_equal(do.numpy(), oracle.mul_scalar(x, 0.125, dt))
        capi.check(L().mul_scalar_kernel_device(do.ptr, dx.ptr, scalar_arg(1.0 / 3.0, dt), n, dt), "mul_scalar")
        assert np.array_equal(do.numpy(), oracle.mul_scalar(x, 1.0 / 3.0, dt))
        capi.check(L().relu_kernel_device(do.ptr, dx.ptr, n, dt), "relu")
        assert np.array_equal(do.numpy(), oracle.relu(x, dt))
        capi.check(L().backwards_relu_device(dy.ptr, dx.ptr, do.ptr, n, dt), "backwards_relu")
        assert np.array_equal(do.numpy(), oracle.backwards_relu(y, x, dt))


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_broadcasting_add_bit_exact(dt):
    rng = np.random.default_rng(41)
    y = rand_storage(rng, (37, 53), dt); b = rand_storage(rng, (53,), dt)
    dy, db, do = Dev(y, dt), Dev(b, dt), Dev.empty((37, 53), dt)
    capi.check(L().add_strided_kernel_device(do.ptr, dy.ptr, db.ptr, 2, _arr(37, 53), _arr(53, 1), _arr(0, 1), y.size, dt), "add_strided")
    assert np.array_equal(do.numpy(), oracle.bias_add(y, b, dt))
    # general case: [4,1,6] + [5,1] -> [4,5,6]
    x1 = rand_storage(rng, (4, 1, 6), dt); x2 = rand_storage(rng, (5, 1), dt)
    d1, d2, d3 = Dev(x1, dt), Dev(x2, dt), Dev.empty((4, 5, 6), dt)
    capi.check(L().add_strided_kernel_device(d3.ptr, d1.ptr, d2.ptr, 3, _arr(4, 5, 6), _arr(6, 0, 1), _arr(0, 1, 0), 120, dt), "add_strided")
    assert np.array_equal(d3.numpy(), oracle.add_strided(x1, x2, (4, 5, 6), (6, 0, 1), (0, 1, 0), dt))


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_softmax_family(dt):
    rng = np.random.default_rng(42)
    # rows of 64 .. 4096 elements take the kernels that hold a row in registers (1, 2, 4 or 8 pieces per lane, partly filled)
    for shape, dim in (((9, 10), -1), ((33, 512), -1), ((3, 17, 5), 1), ((2, 3, 64), -1), ((5, 1024), -1), ((3, 2040), -1), ((2, 4096), -1), ((2, 4104), -1)):
        x = oracle.to_storage(rng.normal(0, 2, shape), dt); g = rand_storage(rng, shape, dt)
        o, d, i = oracle._split(shape, dim)
        dx, dg, do = Dev(x, dt), Dev(g, dt), Dev.empty(shape, dt)
        capi.check(L().softmax_kernel_device(do.ptr, dx.ptr, o, d, i, dt), "softmax")
        y = do.numpy()
        want = oracle.softmax(x, dt, dim=dim)
        assert oracle.rel_err(oracle.to_f64(y, dt), oracle.to_f64(want, dt)) <= _tol(dt)
        capi.check(L().log_softmax_kernel_device(do.ptr, dx.ptr, o, d, i, dt), "log_softmax")
        assert oracle.rel_err(oracle.to_f64(do.numpy(), dt), oracle.to_f64(oracle.softmax(x, dt, dim=dim, log=True), dt)) <= _tol(dt)
        dy = Dev(want, dt)
        capi.check(L().backwards_softmax_device(dg.ptr, dy.ptr, do.ptr, o, d, i, dt), "backwards_softmax")
        wantg = oracle.backwards_softmax(g, want, dt, dim=dim)
        assert oracle.rel_err(oracle.to_f64(do.numpy(), dt), oracle.to_f64(wantg, dt)) <= 4 * _tol(dt)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_contiguous_copy_of_views(dt):
    rng = np.random.default_rng(43)
    base = rand_storage(rng, (4, 6, 10), dt)
    view = base.transpose(2, 0, 1)[2:, :, ::2]
    strides = [s // base.itemsize for s in view.strides]
    off = (view.__array_interface__["data"][0] - base.__array_interface__["data"][0])
    db, do = Dev(base, dt), Dev.empty(view.shape, dt)
    capi.check(L().contiguous_copy_kernel_device(do.ptr, db.ptr + off, view.ndim, _arr(*view.shape), _arr(*strides), view.size, dt), "contiguous_copy")
    assert np.array_equal(do.numpy(), view)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_reductions(dt):
    rng = np.random.default_rng(44)
    for n in (1, 100, 4097, 300000):
        x = rand_storage(rng, (n,), dt)
        dx, do = Dev(x, dt), Dev.empty((1,), dt)
        x64 = oracle.to_f64(x, dt)
        scale = np.abs(x64).sum()
        capi.check(L().sum_all_kernel_device(do.ptr, dx.ptr, n, dt), "sum_all")
        got = oracle.to_f64(do.numpy(), dt)[0]
        unit = {F32: 1e-6, F64: 1e-15, F16: 1e-3, BF16: 8e-3}[dt]
        assert abs(got - x64.sum()) <= unit * scale + unit * abs(x64.sum()) * 4
        capi.check(L().mean_all_kernel_device(do.ptr, dx.ptr, n, dt), "mean_all")
        got = oracle.to_f64(do.numpy(), dt)[0]
        assert abs(got - x64.mean()) <= (unit * scale + unit * abs(x64.sum()) * 4) / n
        again = Dev.empty((1,), dt)
        capi.check(L().mean_all_kernel_device(again.ptr, dx.ptr, n, dt), "mean_all")
        assert np.array_equal(again.numpy(), do.numpy())        # deterministic
    x = rand_storage(rng, (3, 50, 7), dt)
    dx, do = Dev(x, dt), Dev.empty((3, 7), dt)
    capi.check(L().sum_dim_kernel_device(do.ptr, dx.ptr, 3, 50, 7, dt), "sum_dim")
    assert oracle.rel_err(oracle.to_f64(do.numpy(), dt), oracle.to_f64(x, dt).sum(1)) <= 8 * _tol(dt)


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_reduce_rows_matches_reference_order_bit_exact(dt):
    rng = np.random.default_rng(45)
    for rows, cols in ((1, 1), (256, 10), (256, 256), (37, 131)):
        g = rand_storage(rng, (rows, cols), dt)
        dg, do = Dev(g, dt), Dev.empty((cols,), dt)
        capi.check(L().rp_hip_reduce_rows(do.ptr, dg.ptr, rows, cols, 0, dt), "reduce_rows")
        want = oracle.reduce_rows(g, dt)
        assert np.array_equal(do.numpy(), want)
        capi.check(L().rp_hip_reduce_rows(do.ptr, dg.ptr, rows, cols, 1, dt), "reduce_rows")
        assert np.array_equal(do.numpy(), oracle.add(want, want, dt))


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_fill_and_convert(dt):
    rng = np.random.default_rng(46)
    d = Dev.empty((1000,), dt)
    capi.check(L().rp_hip_fill(d.ptr, 1.0 / 3.0, 1000, dt), "fill")
    assert np.array_equal(d.numpy(), oracle.to_storage(np.full(1000, np.float32(1.0 / 3.0) if dt != F64 else 1.0 / 3.0), dt))
    x = rand_storage(rng, (777,), dt)
    dx = Dev(x, dt)
    for dst in ALL:
        do = Dev.empty((777,), dst)
        capi.check(L().rp_hip_convert(do.ptr, dst, dx.ptr, dt, 777), "convert")
        want = oracle.to_storage(oracle.to_f64(x, dt), dst)
        assert np.array_equal(do.numpy(), want), (dt, dst)
    # bases that are not 16-byte aligned: the elements before the first boundary and after the last whole vector go one by one
    es = x.itemsize
    canvas = Dev(np.zeros(1100, dtype=x.dtype), dt)
    for first, count in ((3, 1000), (1, 5), (7, 1), (5, 64)):
        capi.check(L().rp_hip_fill(canvas.ptr, 0.0, 1100, dt), "fill")
        capi.check(L().rp_hip_fill(canvas.ptr + first * es, 2.0, count, dt), "fill")
        got = oracle.to_f64(canvas.numpy(), dt)
        assert (got[first:first + count] == 2.0).all() and not got[:first].any() and not got[first + count:].any(), (first, count)
    for dst in ALL:
        do = Dev(np.zeros(800, dtype=oracle.to_storage(np.zeros(1), dst).dtype), dst)
        capi.check(L().rp_hip_convert(do.ptr + do.numpy().itemsize, dst, dx.ptr + es, dt, 776), "convert")
        want = oracle.to_storage(oracle.to_f64(x[1:], dt), dst)
        got = do.numpy()
        assert np.array_equal(got[1:777], want) and not oracle.to_f64(got[:1], dst).any() and not oracle.to_f64(got[777:], dst).any(), (dt, dst)
    buf = Dev.empty((1001,), F32)
    capi.check(L().rp_hip_fill(buf.ptr, 5.0, 1001, F32), "fill")
    capi.check(L().rp_hip_memset(buf.ptr + 4, 0, 4 * 999), "memset")
    got = buf.numpy()
    assert got[0] == 5.0 and got[-1] == 5.0 and not got[1:-1].any()


@pytest.mark.parametrize("dt", [F32, F64], ids=lambda d: NAMES[d])
def test_cross_entropy(dt):
    rng = np.random.default_rng(47)
    for batch, classes in ((256, 10), (7, 3), (1000, 33)):
        logits = oracle.to_storage(rng.normal(0, 3, (batch, classes)), dt)
        t = rng.integers(0, classes, batch).astype(np.int32)
        dl, dt_ = Dev(logits, dt), capi.DeviceBuffer.from_numpy(t)
        dloss, dgrad = Dev.empty((1,), dt), Dev.empty((batch, classes), dt)
        capi.check(L().rp_hip_cross_entropy_mean(dloss.ptr, dgrad.ptr, dl.ptr, dt_.ptr, batch, classes, 1.0, dt), "ce")
        loss, grad = oracle.cross_entropy_mean(logits, t, dt)
        tolv = 4e-6 if dt == F32 else 1e-13
        assert abs(float(dloss.numpy()[0]) - float(loss[0])) <= tolv * max(1.0, abs(float(loss[0])))
        assert oracle.rel_err(dgrad.numpy(), grad) <= tolv
    bad = capi.DeviceBuffer.from_numpy(np.array([0, 3, 1], dtype=np.int32))
    lg = Dev(oracle.to_storage(rng.normal(0, 1, (3, 3)), dt), dt)
    ls = Dev.empty((1,), dt)
    capi.check(L().rp_hip_cross_entropy_mean(ls.ptr, None, lg.ptr, bad.ptr, 3, 3, 1.0, dt), "ce")
    assert np.isnan(ls.numpy()[0])
    assert L().rp_hip_cross_entropy_mean(ls.ptr, None, lg.ptr, bad.ptr, 3, 3, 1.0, BF16) == -1


@pytest.mark.parametrize("dt", [F32, F64], ids=lambda d: NAMES[d])
def test_cross_entropy_backward_reads_the_upstream_gradient_on_the_device(dt):
    """Same gradient, bit for bit, as the entry that takes the upstream factor from the host."""
    rng = np.random.default_rng(49)
    for batch, classes, up in ((256, 10, 1.0), (7, 3, -0.375), (1000, 33, 2.5)):
        logits = oracle.to_storage(rng.normal(0, 3, (batch, classes)), dt)
        t = rng.integers(0, classes, batch).astype(np.int32)
        dl, dtg = Dev(logits, dt), capi.DeviceBuffer.from_numpy(t)
        dup = Dev(oracle.to_storage(np.array([up]), dt), dt)
        want, got = Dev.empty((batch, classes), dt), Dev.empty((batch, classes), dt)
        capi.check(L().rp_hip_cross_entropy_mean(None, want.ptr, dl.ptr, dtg.ptr, batch, classes, up, dt), "ce")
        capi.check(L().rp_hip_cross_entropy_backward(got.ptr, dl.ptr, dtg.ptr, batch, classes, dup.ptr, dt), "ce backward")
        assert np.array_equal(got.numpy(), want.numpy())
        _, grad = oracle.cross_entropy_mean(logits, t, dt)
        assert oracle.rel_err(got.numpy(), grad * up) <= (4e-6 if dt == F32 else 1e-13)
    assert L().rp_hip_cross_entropy_backward(got.ptr, dl.ptr, dtg.ptr, batch, classes, dup.ptr, BF16) == -1


@pytest.mark.parametrize("dt", [F32, F64], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("from_logits", [True, False], ids=["logits", "probabilities"])
@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_cross_entropy_every_reduction_on_logits_and_probabilities(dt, from_logits, reduction):
    """rp_hip_cross_entropy_forward / _grad against the oracle's restatement of op_cross_entropy_loss and its backward
    (reference ops/ops.c:5545-5643, 5412-5543)."""
    rng = np.random.default_rng(50)
    red = oracle.REDUCTIONS[reduction]
    tolv = 4e-6 if dt == F32 else 1e-13
    for batch, classes in ((256, 10), (7, 3), (1000, 33)):
        x = oracle.to_storage(rng.normal(0, 3, (batch, classes)), dt)
        if not from_logits:
            x = oracle.softmax(x, dt)
        t = rng.integers(0, classes, batch).astype(np.int32)
        up = oracle.to_storage(rng.normal(0, 1, batch if red == 0 else 1), dt)
        dx, dtg, dup = Dev(x, dt), capi.DeviceBuffer.from_numpy(t), Dev(up, dt)
        dloss, dgrad = Dev.empty((batch if red == 0 else 1,), dt), Dev.empty((batch, classes), dt)
        capi.check(L().rp_hip_cross_entropy_forward(dloss.ptr, dx.ptr, dtg.ptr, batch, classes, red, int(from_logits), dt), "ce forward")
        capi.check(L().rp_hip_cross_entropy_grad(dgrad.ptr, dx.ptr, dtg.ptr, batch, classes, red, int(from_logits), dup.ptr, dt), "ce grad")
        loss, grad = oracle.cross_entropy(x, t, dt, reduction, from_logits, upstream=up)
        assert oracle.rel_err(dloss.numpy(), loss) <= tolv
        assert oracle.rel_err(dgrad.numpy(), grad) <= tolv
        if reduction == "mean" and from_logits:              # the older mean-on-logits entry gives the same bits
            old = Dev.empty((1,), dt)
            capi.check(L().rp_hip_cross_entropy_mean(old.ptr, None, dx.ptr, dtg.ptr, batch, classes, 1.0, dt), "ce")
            assert np.array_equal(old.numpy(), dloss.numpy())
    assert L().rp_hip_cross_entropy_forward(dloss.ptr, dx.ptr, dtg.ptr, batch, classes, 3, 1, dt) == -1
    assert L().rp_hip_cross_entropy_forward(dloss.ptr, dx.ptr, dtg.ptr, batch, classes, red, 1, BF16) == -1


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_backwards_log_softmax(dt):
    """Gradient of log_softmax (reference ops/grad_host.c:1428-1500) over the last and over a middle axis."""
    rng = np.random.default_rng(51)
    for shape, dim in (((7, 33), -1), ((1000, 10), -1), ((3, 600), -1), ((3, 5, 4), 1), ((2, 70, 3), 1)):
        x = rand_storage(rng, shape, dt); g = rand_storage(rng, shape, dt)
        y = oracle.softmax(x, dt, dim=dim, log=True)
        o, d, i = oracle._split(shape, dim)
        dg, dy, dgx = Dev(g, dt), Dev(y, dt), Dev.empty(shape, dt)
        capi.check(L().backwards_log_softmax_device(dg.ptr, dy.ptr, dgx.ptr, o, d, i, dt), "backwards_log_softmax")
        want = oracle.backwards_log_softmax(g, y, dt, dim=dim)
        assert oracle.rel_err(oracle.to_f64(dgx.numpy(), dt), oracle.to_f64(want, dt)) <= _tol(dt), (shape, dim)
    assert L().backwards_log_softmax_device(None, dy.ptr, dgx.ptr, o, d, i, dt) == -1


@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_fill_scaled_matches_a_host_side_product(dt):
    for value, scale, n in ((1.0, 1.0 / 777, 777), (-2.5, 1.0, 5000), (0.3, 1.0 / 3, 1)):
        stored = oracle.to_storage(np.array([value]), dt)
        ds, out, want = Dev(stored, dt), Dev.empty((n,), dt), Dev.empty((n,), dt)
        capi.check(L().rp_hip_fill_scaled(out.ptr, ds.ptr, scale, n, dt), "fill scaled")
        capi.check(L().rp_hip_fill(want.ptr, float(oracle.to_f64(stored, dt)[0]) * scale, n, dt), "fill")
        assert np.array_equal(out.numpy(), want.numpy())


def test_allocator_reuses_blocks_and_reports_errors():
    a = capi.DeviceBuffer(1000); p = a.ptr
    a.free()
    b = capi.DeviceBuffer(900)
    assert b.ptr == p                       # same 512-byte size class, handed out again
    assert L().rp_hip_free(ctypes.c_void_p(12345)) == -1
    assert b"not allocated" in L().rp_hip_last_error()
    assert capi.device_count() >= 1
    e0, e1 = capi.Event(), capi.Event()
    e0.record(); e1.record(); e1.synchronize()
    assert e0.elapsed_ms(e1) >= 0.0


def test_graph_replay_matches_eager():
    """A recorded GEMM + bias-gradient + relu sequence replays to the eager result every time (no memset nodes inside)."""
    rng = np.random.default_rng(48)
    m, k, n = 64, 96, 128
    a = rand_storage(rng, (m, k), F32); b = rand_storage(rng, (k, n), F32); bias = rand_storage(rng, (n,), F32)
    da, db, dbias = Dev(a, F32), Dev(b, F32), Dev(bias, F32)
    dy, dr, dg = Dev.empty((m, n), F32), Dev.empty((m, n), F32), Dev.empty((n,), F32)
    w = rand_storage(rng, (1, 2048), BF16); x = rand_storage(rng, (2048, 1024), BF16)
    dw, dxx, dz = Dev(w, BF16), Dev(x, BF16), Dev.empty((1, 1024), BF16)

    def seq():
        capi.gemm(dy.ptr, da.ptr, db.ptr, dbias.ptr, 1, m, k, n, (0, k, 1), (0, n, 1), (0, n, 1), False, F32)
        capi.check(L().relu_kernel_device(dr.ptr, dy.ptr, m * n, F32), "relu")
        capi.check(L().rp_hip_reduce_rows(dg.ptr, dr.ptr, m, n, 0, F32), "reduce_rows")
        capi.check(L().rp_hip_memset(dy.ptr, 0, 64), "memset")
        capi.gemm(dz.ptr, dw.ptr, dxx.ptr, None, 1, 1, 2048, 1024, (0, 2048, 1), (0, 1024, 1), (0, 1024, 1), False, BF16)   # skinny: split-k workspace

    seq()
    want = (dr.numpy().copy(), dg.numpy().copy(), dy.numpy().copy(), dz.numpy().copy())
    stream = capi.Stream()
    with stream:
        with capi.Graph.capture() as graph:
            seq()
        for _ in range(4):
            capi.check(L().rp_hip_fill(dr.ptr, -1.0, m * n, F32), "fill")      # eager work between replays
            capi.check(L().rp_hip_fill(dz.ptr, -1.0, 1024, BF16), "fill")
            graph.launch()
            capi.check(L().rp_hip_stream_synchronize(), "sync")
            got = (dr.numpy(), dg.numpy(), dy.numpy(), dz.numpy())
            for g_, w_ in zip(got, want):
                assert np.array_equal(g_, w_)


def test_workspace_recorded_into_a_graph_is_not_handed_out_while_the_graph_lives():
    """A split-k GEMM recorded into a graph keeps writing its partial sums to the workspace it was recorded with.
    Until the graph is destroyed that block must not be given to anyone else: buffers allocated after the recording,
    of every size the workspace could have, keep their contents across replays."""
    rng = np.random.default_rng(52)
    w = rand_storage(rng, (1, 2048), BF16); x = rand_storage(rng, (2048, 1024), BF16)
    dw, dxx, dz = Dev(w, BF16), Dev(x, BF16), Dev.empty((1, 1024), BF16)

    def skinny():
        capi.gemm(dz.ptr, dw.ptr, dxx.ptr, None, 1, 1, 2048, 1024, (0, 2048, 1), (0, 1024, 1), (0, 1024, 1), False, BF16)

    skinny()                                        # eager once: the workspace block now sits in the pool
    capi.synchronize()
    want = dz.numpy().copy()
    stream = capi.Stream()
    with stream:
        with capi.Graph.capture() as graph:
            skinny()
        # whatever size the workspace had (nsplit x 1 x 1024 floats, rounded to 512 bytes), one of these would get its block
        guards = [capi.DeviceBuffer(nsplit * 1024 * 4) for nsplit in range(1, 33)]
        for gbuf in guards:
            capi.check(L().rp_hip_memset(gbuf.ptr, 0x5A, gbuf.nbytes), "memset")
        for _ in range(3):
            capi.check(L().rp_hip_fill(dz.ptr, -1.0, 1024, BF16), "fill")
            graph.launch()
            capi.check(L().rp_hip_stream_synchronize(), "sync")
            assert np.array_equal(dz.numpy(), want)
            for gbuf in guards:
                assert np.all(gbuf.to_numpy(np.uint8, (gbuf.nbytes,)) == 0x5A)
        for gbuf in guards:
            gbuf.free()


def test_narrowing_to_fp16_every_exponent_and_rounding_case():
    """fp32 -> fp16 on the device against the oracle, bit for bit: every sign and exponent with mantissas that sit
    on, just below and just above every rounding boundary (ties, carries into the next binade, the subnormal range,
    the overflow threshold), random mantissas and infinities; NaNs must stay NaNs."""
    rng = np.random.default_rng(48)
    exps = np.arange(256, dtype=np.uint32)
    edge = []
    for sh in range(0, 24):                       # a dropped-bit position for every subnormal shift and the normal one
        bit = np.uint32(1) << np.uint32(sh)
        for m in (bit - 1, bit, bit + 1, (bit << 1) - 1 if sh < 23 else bit, 0x7FFFFF & ~(bit - 1), 0x7FFFFF, 0x7FFFFF - bit + 1):
            edge.append(np.uint32(m) & np.uint32(0x7FFFFF))
    mant = np.unique(np.concatenate([np.array(edge, dtype=np.uint32), np.array([0, 1, 0x1000, 0x0FFF, 0x1001, 0x1FFF, 0x2000, 0x3000, 0x7FE000, 0x7FF000, 0x7FEFFF], dtype=np.uint32),
                                     rng.integers(0, 1 << 23, 3000, dtype=np.uint32)]))
    w = (exps[:, None] << np.uint32(23)) | mant[None, :]
    w = np.concatenate([w.ravel(), w.ravel() | np.uint32(0x80000000)])
    x = w.view(np.float32)
    dx, do = Dev(x, F32), Dev.empty(x.shape, F16)
    capi.check(L().rp_hip_convert(do.ptr, F16, dx.ptr, F32, x.size), "convert")
    got, want = do.numpy(), oracle.narrow(x, F16)
    nan = np.isnan(x)                      # a NaN must stay a NaN of the same sign; its payload bits are not compared
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x03FF) != 0) and np.all((got[nan] & 0x8000) == (want[nan] & 0x8000))
    got, want, w = got[~nan], want[~nan], w[~nan]
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(int(w[i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:8]]


# ---- softmax(x * scalar) and its gradient in one pass; a scalar multiply whose launch is postponed
@pytest.mark.parametrize("dt", ALL, ids=lambda d: NAMES[d])
def test_scaled_softmax_is_the_two_ops_bit_for_bit(dt):
    """rp_hip_scaled_softmax / rp_hip_backwards_scaled_softmax against mul_scalar_kernel_device + softmax_kernel_device and
    backwards_softmax_device + mul_scalar_kernel_device (reference ops/ops.c:6022-6086, 5721-5788, grad_host.c:1387-1398):
    rows the one-pass kernels take (whole 16-byte vectors, up to 4096 elements) and rows they hand to the two launches."""
    rng = np.random.default_rng(47)
    for shape, dim in (((33, 512), -1), ((5, 1024), -1), ((7, 64), -1), ((3, 2040), -1), ((9, 10), -1), ((3, 17, 5), 1), ((2, 4104), -1)):
        x = rand_storage(rng, shape, dt, dist="normal")
        g = rand_storage(rng, shape, dt)
        d = dim % len(shape)
        outer = int(np.prod(shape[:d])); n = shape[d]; inner = int(np.prod(shape[d + 1:]))
        for scalar in (0.125, 1.0 / 3.0):
            dx, dg = Dev(x, dt), Dev(g, dt)
            t, y, y1, gt, g2, g1 = (Dev.empty(shape, dt) for _ in range(6))
            capi.check(L().mul_scalar_kernel_device(t.ptr, dx.ptr, scalar_arg(scalar, dt), x.size, dt), "mul_scalar")
            capi.check(L().softmax_kernel_device(y.ptr, t.ptr, outer, n, inner, dt), "softmax")
            capi.check(L().rp_hip_scaled_softmax(y1.ptr, dx.ptr, scalar_arg(scalar, dt), outer, n, inner, dt), "scaled_softmax")
            assert np.array_equal(y.numpy(), y1.numpy()), (shape, scalar)
            capi.check(L().backwards_softmax_device(dg.ptr, y.ptr, gt.ptr, outer, n, inner, dt), "backwards_softmax")
            capi.check(L().mul_scalar_kernel_device(g2.ptr, gt.ptr, scalar_arg(scalar, dt), x.size, dt), "mul_scalar")
            capi.check(L().rp_hip_backwards_scaled_softmax(dg.ptr, y.ptr, g1.ptr, scalar_arg(scalar, dt), outer, n, inner, dt), "backwards_scaled_softmax")
            assert np.array_equal(g2.numpy(), g1.numpy()), (shape, scalar)


@pytest.mark.parametrize("dt", [BF16, F32], ids=lambda d: NAMES[d])
def test_postponed_scalar_multiply_runs_before_whatever_follows(dt):
    """rp_hip_mul_scalar_deferred leaves its launch to the thread's next call into the library.  Whatever that call is
    (a copy to the host, another kernel reading the product, freeing the source, a second postponed multiply, a
    synchronisation) the product is there as if launched at once; only rp_hip_take_deferred keeps it from being written."""
    rng = np.random.default_rng(48)
    n = 4096
    x = rand_storage(rng, (n,), dt)
    want = oracle.mul_scalar(x, 0.125, dt)
    sentinel = rand_storage(rng, (n,), dt)

    def fresh():
        return Dev(x, dt), Dev(sentinel, dt)

    # a copy to the host
    dx, do = fresh()
    capi.check(L().rp_hip_mul_scalar_deferred(do.ptr, dx.ptr, scalar_arg(0.125, dt), n, dt), "deferred")
    assert np.array_equal(do.buf.to_numpy(capi.NP_STORAGE[dt], (n,)), want)
    # a kernel that reads the product
    dx, do = fresh()
    d2 = Dev.empty((n,), dt)
    capi.check(L().rp_hip_mul_scalar_deferred(do.ptr, dx.ptr, scalar_arg(0.125, dt), n, dt), "deferred")
    capi.check(L().relu_kernel_device(d2.ptr, do.ptr, n, dt), "relu")
    assert np.array_equal(d2.numpy(), oracle.relu(want, dt))
    # freeing the source
    dx, do = fresh()
    capi.check(L().rp_hip_mul_scalar_deferred(do.ptr, dx.ptr, scalar_arg(0.125, dt), n, dt), "deferred")
    dx.buf.free()
    assert np.array_equal(do.numpy(), want)
    # a second postponed multiply, then a synchronisation
    dx, do = fresh()
    do2 = Dev(sentinel, dt)
    capi.check(L().rp_hip_mul_scalar_deferred(do.ptr, dx.ptr, scalar_arg(0.125, dt), n, dt), "deferred")
    capi.check(L().rp_hip_mul_scalar_deferred(do2.ptr, dx.ptr, scalar_arg(2.0, dt), n, dt), "deferred")
    capi.synchronize()
    assert np.array_equal(do.numpy(), want) and np.array_equal(do2.numpy(), oracle.mul_scalar(x, 2.0, dt))
    # taken back: never written, and the source and scalar come back for the one-pass softmax
    dx, do = fresh()
    capi.check(L().rp_hip_mul_scalar_deferred(do.ptr, dx.ptr, scalar_arg(0.125, dt), n, dt), "deferred")
    src, s = ctypes.c_void_p(), ctypes.c_double()
    assert L().rp_hip_take_deferred(do.ptr, ctypes.byref(src), ctypes.byref(s)) == 1
    assert src.value == dx.ptr and s.value == 0.125
    assert L().rp_hip_take_deferred(do.ptr, ctypes.byref(src), ctypes.byref(s)) == 0
    capi.synchronize()
    assert np.array_equal(do.numpy(), sentinel)
