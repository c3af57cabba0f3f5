"""The C-ABI library loads and exports every symbol include/rp_hip.h declares (no GPU needed)."""
import os
import re

from recpulse_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "rp_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{}]*\)\s*;", text)


def test_header_declares_the_expected_entry_points():
    names = _declared()
    assert len(names) == len(set(names))
    for must in ("matmul_kernel_device", "rp_hip_gemm_strided_batched", "rp_hip_malloc", "add_strided_kernel_device",
                 "softmax_kernel_device", "backwards_softmax_device", "rp_hip_reduce_rows"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = capi.lib()
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in rp_hip.h but not exported by librp_hip.so"


def test_python_binding_covers_every_declared_symbol():
    assert set(_declared()) == set(capi.SIGNATURES)


def test_argument_errors_are_reported_without_a_gpu():
    lib = capi.lib()
    assert lib.rp_hip_gemm_strided_batched(None, None, None, None, 1, 1, 1, 1, 0, 1, 1, 0, 1, 1, 0, 1, 1, 0, 0) == -1
    assert b"null operand" in lib.rp_hip_last_error()
    assert lib.matmul_kernel_device(None, None, None, 2, 2, 2, 0) == -1
    assert lib.add_kernel_device(None, None, None, 4, 0) == -1
    assert lib.rp_hip_free(None) == 0


def test_kernel_selection_names():
    name = capi.gemm_kernel_name
    assert name(1, 8192, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), capi.BF16) == "mfma16_256x256"
    assert name(1, 8192, 8192, 8192, (1, 8192), (8192, 1), (8192, 1), capi.F16) == "mfma16_256x256"       # A^T view
    assert name(1, 1, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), capi.BF16) == "mfma16_stream_32x128"
    assert name(1, 8, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), capi.BF16) == "mfma16_stream_32x128"
    assert name(1, 16, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), capi.F16) == "mfma16_stream_32x128"
    assert name(1, 32, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), capi.F16) == "mfma16_stream_32x128"
    assert name(1, 33, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), capi.F16) == "mfma16_skinny_32x128"
    assert name(1, 32, 8192, 2048, (8192, 1), (2048, 1), (2048, 1), capi.F16) == "mfma16_skinny_32x128"      # 16 splits x 32 rows: its finish would be too long
    assert name(1, 16, 4096, 2048, (4096, 1), (2048, 1), (2048, 1), capi.F16) == "mfma16_skinny_32x128"      # a small B that would need 16 splits
    assert name(1, 8, 8192, 8192, (8192, 1), (1, 8192), (8192, 1), capi.BF16) == "mfma16_skinny_32x128"
    assert name(1, 8, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), capi.F32) == "skinny"
    assert name(1, 128, 784, 256, (784, 1), (256, 1), (256, 1), capi.F32) == "tiny32_16x16"          # a small fp32 output: one launch of 16 x 16 tiles
    assert name(1, 128, 4096, 256, (4096, 1), (256, 1), (256, 1), capi.F32) == "mfma32_64x64"        # deeper k: small tile + split-k over workgroups
    assert name(1, 4096, 4096, 4096, (4096, 1), (4096, 1), (4096, 1), capi.F32) == "mfma32_128x128"
    assert name(1, 2048, 2048, 2048, (2048, 1), (2048, 1), (2048, 1), capi.F64) == "mfma64_128x128"
    assert name(64, 64, 576, 3136, (576, 1), (3136, 1), (3136, 1), capi.BF16) == "mfma16_64x128"           # at most 64 rows, short k (a lowered convolution)
    assert name(64, 64, 3136, 576, (3136, 1), (1, 3136), (576, 1), capi.F16) == "mfma16_64x256"            # at most 64 rows, long k (its weight gradient)
    assert name(1, 64, 1024, 4096, (1024, 1), (4096, 1), (4096, 1), capi.BF16) == "mfma16_64x64"           # too few column tiles for the wide ones
    # configuration 4 per head, and shapes like it: the resident kernels
    Z, S, D = 192, 512, 64
    for dt, short_k, narrow in ((capi.BF16, "pipe16_128x128", "pipe16k_128x64"), (capi.F16, "pipe16_128x128", "pipe16k_128x64"), (capi.F32, "pipe32_128x128", "pipe32k_128x64")):
        assert name(Z, S, D, S, (D, 1), (1, D), (S, 1), dt) == short_k                 # S = Q.K^T, K^T a stride view
        assert name(Z, S, S, D, (S, 1), (D, 1), (D, 1), dt) == narrow                  # O = P.V
        assert name(Z, S, S, D, (1, S), (D, 1), (D, 1), dt) == narrow                  # dV = P^T.dO
        assert name(64, 576, D, 3136, (1, 576), (3136, 1), (3136, 1), dt) == short_k   # the lowered convolution's dcol = W^T.dy
    assert name(8, S, D, S, (D, 1), (1, D), (S, 1), capi.BF16) == "mfma16_128x128"       # fewer tiles than CUs: the tiled kernels
    assert name(8, S, D, S, (D, 1), (1, D), (S, 1), capi.F32) == "mfma32_128x128"
    assert name(Z, S, 128, S, (128, 1), (1, 128), (S, 1), capi.BF16) == "mfma16_128x128"  # k above 64
    assert name(Z, S, S, 128, (S, 1), (128, 1), (128, 1), capi.F32) == "mfma32_128x128"   # more than 64 columns
    assert name(Z, S, D, S, (D, 1), (1, D), (1, S), capi.BF16) == "mfma16_128x128"        # 16-bit C not row-major
    assert name(1, 5, 7, 3, (7, 1), (3, 1), (3, 1), capi.BF16) == "generic"                                # odd extents
    assert name(1, 64, 64, 64, (128, 2), (64, 1), (64, 1), capi.F64) == "generic"                          # no unit stride
