"""The entry point that allocates nothing, rp_hip_gemm_strided_batched_noalloc, against rp_hip_gemm_strided_batched.

Both are called through the C ABI on the same device buffers; the results must agree bit for bit (they run the
same kernels, the split-k partial sums and arrival counters of the one living in a fixed device array).  Each case
makes two calls in a row, the second on a smaller input, so that what the first call leaves in the array (partial
sums, counters) is in place when the second runs.
"""
import numpy as np
import pytest

from recpulse_amd import capi
from devhelp import BF16, F16, F32, rand_storage

import ctypes

pytestmark = pytest.mark.gpu
WORKSPACE = 16 << 20            # RP_HIP_NOALLOC_WORKSPACE_BYTES


def _alloc_counters():
    """(calls to rp_hip_malloc, calls that reached hipMalloc, live blocks, cached blocks) of the process so far."""
    v = [ctypes.c_longlong(0) for _ in range(4)]
    capi.check(capi.lib().rp_hip_memory_stats(*[ctypes.byref(x) for x in v]), "rp_hip_memory_stats")
    return tuple(x.value for x in v)


def _both(rng, m, k, n, dtype, bias=False, accumulate=False, b_transposed=False):
    """One problem through both entry points; returns (result of the allocating one, result of the other)."""
    a = rand_storage(rng, (m, k), dtype)
    b = rand_storage(rng, (n, k) if b_transposed else (k, n), dtype)
    c0 = rand_storage(rng, (m, n), dtype)
    bv = rand_storage(rng, (n,), dtype) if bias else None
    da, db = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b)
    dbias = capi.DeviceBuffer.from_numpy(bv) if bias else None
    b_st = (0, 1, k) if b_transposed else (0, n, 1)
    outs = []
    for entry in ("rp_hip_gemm_strided_batched", "rp_hip_gemm_strided_batched_noalloc"):
        dc = capi.DeviceBuffer.from_numpy(c0)
        fn = getattr(capi.lib(), entry)
        before = _alloc_counters()
        capi.check(fn(dc.ptr, da.ptr, db.ptr, dbias.ptr if dbias else None, 1, m, k, n, 0, k, 1, *b_st, 0, n, 1, int(accumulate), dtype), entry)
        if entry.endswith("_noalloc"):              # the contract itself: no request to the pool, no hipMalloc, nothing held or parked
            assert _alloc_counters() == before, (entry, before, _alloc_counters())
        capi.synchronize()
        outs.append(dc.to_numpy(capi.NP_STORAGE[dtype], (m, n)).copy())
        dc.free()
    return outs


# (kernel the dispatcher picks, first shape, second smaller shape): every split-k launcher that takes a workspace
CASES = [
    ("mfma16_stream_32x128", BF16, (4, 4096, 4096), (2, 2048, 4096), {}),                 # partial sums + arrival counters, single launch
    ("mfma16_stream_32x128", F16, (16, 8192, 2048), (8, 4096, 4096), {"bias": True}),
    ("mfma16_stream_32x128", BF16, (32, 4096, 4096), (20, 2048, 8192), {"accumulate": True}),
    ("mfma16_skinny_32x128", BF16, (40, 4096, 4096), (33, 2048, 2048), {"accumulate": True}),      # tiled split-k + combine launch
    ("mfma16_skinny_32x128", BF16, (8, 4096, 2048), (8, 2048, 2048), {"b_transposed": True}),
    ("skinny", F32, (4, 4096, 4096), (2, 2048, 1024), {}),                                # VALU streaming kernel
    ("mfma32_64x64", F32, (128, 4096, 256), (64, 4096, 128), {"bias": True}),             # fp32 MFMA split-k
    ("generic", BF16, (30, 1000, 50), (7, 500, 9), {}),                                   # any-stride kernel, split-k for a small output
]


@pytest.mark.parametrize("kernel,dtype,first,second,opts", CASES)
def test_noalloc_matches_allocating_entry_point_on_two_calls_in_a_row(kernel, dtype, first, second, opts):
    rng = np.random.default_rng(71)
    for step, (m, k, n) in enumerate((first, second)):
        b_rc = (1, k) if opts.get("b_transposed") else (n, 1)
        assert capi.gemm_kernel_name(1, m, k, n, (k, 1), b_rc, (n, 1), dtype) == kernel, (m, k, n)
        want, got = _both(rng, m, k, n, dtype, **opts)
        assert np.array_equal(want, got), f"call {step} ({m}x{k}x{n})"


def test_noalloc_without_workspace_and_batched():
    """Shapes whose kernels need no workspace go straight through (the 256 x 256 tile, a batched short-k product)."""
    rng = np.random.default_rng(72)
    want, got = _both(rng, 512, 512, 512, BF16, bias=True)
    assert np.array_equal(want, got)
    want, got = _both(rng, 96, 64, 200, F32)
    assert np.array_equal(want, got)


def test_noalloc_rejects_a_workspace_beyond_the_fixed_array():
    """A few-row GEMM whose split-k partial sums exceed the array fails with a message naming both sizes, and the next call still works."""
    m, k, n = 96, 4096, 16256                       # tiled split-k: 3 splits x 96 x 16256 floats > 16 MiB
    assert capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), BF16) == "mfma16_skinny_32x128"
    rng = np.random.default_rng(73)
    a, b = rand_storage(rng, (m, k), BF16), rand_storage(rng, (k, n), BF16)
    da, db, dc = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b), capi.DeviceBuffer(m * n * 2)
    L = capi.lib()
    before = _alloc_counters()
    rc = L.rp_hip_gemm_strided_batched_noalloc(dc.ptr, da.ptr, db.ptr, None, 1, m, k, n, 0, k, 1, 0, n, 1, 0, n, 1, 0, BF16)
    assert rc == -1
    assert _alloc_counters() == before              # the refusal allocates nothing either
    msg = L.rp_hip_last_error().decode()
    assert "workspace" in msg and str(WORKSPACE) in msg, msg
    capi.synchronize()
    want, got = _both(rng, 8, 2048, 1024, BF16)
    assert np.array_equal(want, got)


@pytest.mark.parametrize("m,k,n", [(4, 4096, 4096), (8, 4096, 4096), (40, 4096, 4096)])
def test_noalloc_recorded_into_a_graph_replays_like_the_eager_call(m, k, n):
    """The callers the entry point is for include code under HIP graph capture.  After a warm eager call the entry is
    recorded on a created stream (single-launch k-split finish at 4 and 8 rows, partial sums + combine launch at 40), the
    graph is replayed three times with other work and a synchronisation in between, and every replay must leave the
    eager result; neither the recording nor the replays may touch the allocator."""
    rng = np.random.default_rng(74)
    a, b = rand_storage(rng, (m, k), BF16), rand_storage(rng, (k, n), BF16)
    da, db = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b)
    d_eager, d_graph, d_other = (capi.DeviceBuffer(m * n * 2) for _ in range(3))
    L = capi.lib()

    def call(dst):
        capi.check(L.rp_hip_gemm_strided_batched_noalloc(dst.ptr, da.ptr, db.ptr, None, 1, m, k, n, 0, k, 1, 0, n, 1, 0, n, 1, 0, BF16), "noalloc")

    call(d_eager)                                   # warm: resolves the fixed array's address, measures workgroup placement
    capi.synchronize()
    want = d_eager.to_numpy(np.uint16, (m, n)).copy()
    stream = capi.Stream()
    with stream:
        before = _alloc_counters()
        with capi.Graph.capture() as graph:
            call(d_graph)
        assert _alloc_counters() == before
        for replay in range(3):
            capi.check(L.rp_hip_memset(d_graph.ptr, 0xff, m * n * 2), "memset")
            graph.launch()
            capi.check(L.rp_hip_stream_synchronize(), "sync")
            assert np.array_equal(d_graph.to_numpy(np.uint16, (m, n)), want), f"replay {replay}"
            # the program's own eager work between replays: another product through the allocating entry, on this stream
            capi.gemm(d_other.ptr, da.ptr, db.ptr, None, 1, m, k, n, (0, k, 1), (0, n, 1), (0, n, 1), False, BF16)
            capi.check(L.rp_hip_stream_synchronize(), "sync")
        assert _alloc_counters()[2] == before[2]    # no block of the recording stays handed out
