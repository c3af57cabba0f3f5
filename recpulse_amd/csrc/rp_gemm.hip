// GEMM kernels for gfx950 and their dispatcher.
//
//   C_z[m,n] = A_z[m,k] · B_z[k,n] (+ bias[n]) (+ C_z)      z in [0, batch)
//
// Operands are described by (batch, row, column) strides in elements, so
// transposed and permuted views are read in place.  Each operand is in one of
// two fast layouts, chosen from its strides:
//   KC  the reduction (k) axis is the unit-stride one      (A row-major, or Bᵀ stored)
//   MC  the free (m or n) axis is the unit-stride one       (B row-major, or Aᵀ stored)
// Anything else (both strides > 1, misaligned bases, odd extents) takes the
// generic strided kernel.
//
// Kernel families:
//   mfma16   bf16 / fp16 inputs, fp32 accumulate, v_mfma_f32_32x32x16_{bf16,f16};
//            KC tiles are read from LDS with ds_read_b128, MC tiles with the
//            transposing ds_read_b64_tr_b16, so no layout needs a copy.
//   mfmaw    fp32 (v_mfma_f32_32x32x2_f32) and fp64 (v_mfma_f64_16x16x4_f64).
//   skinny   m <= 8 against a row-major B: a split-k streaming kernel bound by HBM.
//   tiny     fp32 outputs of a few hundred 16 x 16 tiles: one launch, k split over the waves of a workgroup.
//   generic  any strides, any shape; LDS-tiled scalar FMA.
#include "rp_gemm.h"

#include <mutex>

namespace rp {

// ============================================================================
// dispatch
// ============================================================================
static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// rows up to which a deep 16-bit GEMM with few output tiles splits k
constexpr int SKINNY_MAX_ROWS = 128;

// Tile counts that decide between kernels stand for "one tile per CU" and "half of the CUs": they follow the device
// (whole rounds of the 8 XCDs, as the launchers size their grids); 256 where no device can be asked.
static int cu_tiles() {
    const int n = device_cu_count() / 8 * 8;
    return n >= 8 ? n : 256;
}

// Tile of the 16-bit MFMA kernel for an output of batch x m x n with reduction length k.
static void choose_tile16(Plan& p, int batch, int m, int k, int n) {
    p.fam = FAM_MFMA16;
    const long long tiles256 = (long long)((m + 255) / 256) * ((n + 255) / 256) * batch;
    const long long tiles128 = (long long)((m + 127) / 128) * ((n + 127) / 128) * batch;
    // the 256 x 256 tile runs one block per CU, so it needs a k loop long enough to hide its prologue and
    // epilogue; with fewer than four slabs the smaller tile (two blocks per CU) overlaps them instead
    if (m >= 256 && n >= 256 && tiles256 >= cu_tiles() / 2 && k >= 4 * M16_BK) { p.bm = 256; p.bn = 256; p.name = "mfma16_256x256"; }
    // fewer than 128 tiles of 128 x 128 would leave over half the CUs idle: the 64 x 64 tile quadruples the workgroups
    // (1024^3: 10.9 -> 7.3 us)
    // at most 64 rows: a 64 x 256 tile (the same 64 x 64 patch per wave as the 128 x 128 tile, none of it past the last row)
    // (64 x 128 while k is short: two blocks share a CU and one's loads and stores overlap the other's few slabs)
    else if (m <= 64 && n >= 256 && !path_disabled("wide64") && (long long)((n + 255) / 256) * batch >= cu_tiles() / 2) {
        p.bm = 64; p.bn = k <= 1024 ? 128 : 256; p.name = k <= 1024 ? "mfma16_64x128" : "mfma16_64x256";
    }
    else if ((m > 64 || n > 64) && tiles128 >= cu_tiles() / 2) { p.bm = 128; p.bn = 128; p.name = "mfma16_128x128"; }
    else { p.bm = 64; p.bn = 64; p.name = "mfma16_64x64"; }
    p.edge = (m % p.bm) || (n % p.bn) || (k % M16_BK);
}

// Decide the kernel family and tile from shapes and strides alone (pointer
// alignment is checked by the caller, which may still fall back to generic).
static Plan make_plan(int batch, int m, int k, int n, long long a_rs, long long a_cs, long long b_rs, long long b_cs,
                      long long c_rs, long long c_cs, long long a_bs, long long b_bs, int dtype, bool allow_direct = true) {
    Plan p{FAM_GENERIC, 64, 64, false, false, true, "generic"};
    if (path_disabled("mfma")) return p;
    const int vec = 16 / (int)dtype_size(dtype);                // elements per 16-byte vector
    // operand layouts: KC = unit stride along k, MC = unit stride along the free axis.
    // Extent-1 axes make the other stride irrelevant, but vector loads still need alignment of the non-unit stride.
    bool a_kc = (a_cs == 1) && (a_rs % vec == 0) && (k % vec == 0);
    bool a_mc = (a_rs == 1) && (a_cs % vec == 0) && (m % vec == 0);
    bool b_mc = (b_cs == 1) && (b_rs % vec == 0) && (n % vec == 0);
    bool b_kc = (b_rs == 1) && (b_cs % vec == 0) && (k % vec == 0);
    bool batch_ok = (batch == 1) || ((a_bs % vec == 0) && (b_bs % vec == 0));

    // the MFMA kernels address a tile with 32-bit byte offsets from a 64-bit tile pointer
    const long long max_stride = 1ll << 22;
    const bool strides_ok = a_rs < max_stride && a_cs < max_stride && b_rs < max_stride && b_cs < max_stride;
    const bool mfma_ok = (a_kc || a_mc) && (b_kc || b_mc) && batch_ok && strides_ok;
    const bool is16 = dtype == RP_DTYPE_FLOAT16 || dtype == RP_DTYPE_BFLOAT16;

    // 16-bit, few rows, deep k: split k over many blocks so that B streams at HBM speed (output columns in whole 8s).
    // Up to 32 rows always; up to SKINNY_MAX_ROWS when the 128 x 128 tiles of the output would occupy under half the
    // CUs and k is deep enough to be worth a second launch for the partial sums (64 x 1024 x 4096: 6.6 us on 64 x 64 tiles
    // in one launch against 9.4 us split; 64 x 4096 x 1024: 16.4 against 9.1).  A short batch of such products is
    // split the same way while its tiles together stay under half the CUs.
    const long long tiles128_16 = (long long)((m + 127) / 128) * ((n + 127) / 128) * batch;
    const bool few_rows = batch == 1 ? (m <= 32 || (m <= SKINNY_MAX_ROWS && tiles128_16 < cu_tiles() / 2 && k >= 2048))
                                     : (m <= SKINNY_MAX_ROWS && tiles128_16 < cu_tiles() / 2 && k >= 2048);
    if (is16 && mfma_ok && few_rows && n % 8 == 0 && n >= 256 && k >= 1024 &&
        (long long)k * n >= (1ll << 22)) {
        p.fam = FAM_MFMA16_SKINNY; p.bm = 32; p.bn = 128; p.edge = true; p.a_mc = !a_kc; p.b_mc = b_mc;
        // row-major A and B with at most 32 rows: the streaming kernel, for the shapes it is the right one for
        p.name = (batch == 1 && !p.a_mc && p.b_mc && stream128_shape(batch, m, k, n)) ? "mfma16_stream_32x128" : "mfma16_skinny_32x128";
        return p;
    }
    // VALU skinny: few rows, row-major B, enough columns and depth to be worth streaming
    const int valu_rows = (dtype == RP_DTYPE_FLOAT32) ? SK_MAX_M : 4;
    if (batch == 1 && dtype != RP_DTYPE_FLOAT64 && m <= valu_rows && b_mc && n >= 64 * vec && (long long)k * n >= (1ll << 20) &&
        (n + 64 * vec - 1) / (64 * vec) <= SK_MAX_GROUPS) {
        p.fam = FAM_SKINNY; p.name = "skinny"; p.b_mc = true;
        return p;
    }
    // fp32, an output of fewer than 64 tiles of 64 x 64 and a k that one workgroup walks in a few microseconds: one launch
    // of 16 x 16 tiles with k split over the four waves of a workgroup, any strides (no split over workgroups, no second launch)
    if (dtype == RP_DTYPE_FLOAT32 && k <= 2048 && (long long)((m + 63) / 64) * ((n + 63) / 64) * batch < 64 && !path_disabled("tiny")) {
        p.fam = FAM_TINY; p.bm = 16; p.bn = 16; p.name = "tiny32_16x16";
        return p;
    }
    // fp32 with k <= 64, any operand layout with a unit stride and at least one 128 x 128 tile per CU: one resident workgroup per
    // CU whose fetching waves fill LDS directly and whose multiplying waves store the previous tile between the MFMAs
    if (dtype == RP_DTYPE_FLOAT32 && allow_direct && !path_disabled("pipe32") && k <= 64 && k % 4 == 0 && ((a_cs == 1 && a_rs % 4 == 0) || (a_rs == 1 && a_cs % 4 == 0)) &&
        ((b_rs == 1 && b_cs % 4 == 0) || (b_cs == 1 && b_rs % 4 == 0)) &&
        batch_ok && m > 64 && n > 64 && (long long)((m + 127) / 128) * ((n + 127) / 128) * batch >= cu_tiles()) {
        p.fam = FAM_PIPE32; p.bm = 128; p.bn = 128; p.a_mc = !(a_cs == 1 && a_rs % 4 == 0); p.b_mc = !(b_rs == 1 && b_cs % 4 == 0); p.edge = (m % 128) || (n % 128); p.name = "pipe32_128x128";
        return p;
    }
    // fp32 with 32 < k <= 64, both operands with unit stride along their free index and an output of at least 128 tiles of
    // 128 x 128: no k loop to pipeline, so every wave multiplies a 64 x 64 patch straight out of registers (no LDS, no
    // barrier).  (With unit stride along k a lane's loads touch 64 cache lines per instruction and the vector cache's
    // tag lookups take longer than the MFMAs: those layouts keep LDS.)
    if (dtype == RP_DTYPE_FLOAT32 && allow_direct && !path_disabled("direct32") && k > 32 && k <= 64 && a_rs == 1 && a_cs != 1 && b_cs == 1 && b_rs != 1 &&
        (a_cs != 1 || (k % 4 == 0 && a_rs % 4 == 0 && a_bs % 4 == 0)) && (b_rs != 1 || (k % 4 == 0 && b_cs % 4 == 0 && b_bs % 4 == 0)) &&
        m >= 64 && n >= 64 && (long long)((m + 127) / 128) * ((n + 127) / 128) * batch >= cu_tiles() / 2) {
        p.fam = FAM_DIRECT32; p.bm = 128; p.bn = 128; p.a_mc = a_cs != 1; p.b_mc = b_rs != 1; p.name = "direct32_128x128";
        return p;
    }
    // the same for bf16 / fp16 (C row-major): there the stores and the narrowing are what takes time
    if (is16 && allow_direct && !path_disabled("pipe16") && k <= 64 && k % 8 == 0 && (a_kc || a_mc) && (b_kc || b_mc) && batch_ok &&
        c_cs == 1 && c_rs % 8 == 0 && n % 8 == 0 && m > 64 && n > 64 && (long long)((m + 127) / 128) * ((n + 127) / 128) * batch >= cu_tiles()) {
        p.fam = FAM_PIPE16; p.bm = 128; p.bn = 128; p.a_mc = !a_kc; p.b_mc = !b_kc; p.edge = (m % 128) || (n % 128); p.name = "pipe16_128x128";
        return p;
    }
    // bf16 / fp16, at most 64 output columns, at least one 128-row tile per CU (O = P.V per head, a tall matrix times a narrow
    // one): bound by reading A; the resident kernel whose fetching waves keep three k slabs in flight into LDS
    if (is16 && allow_direct && !path_disabled("pipe16k") && n <= 64 && n % 8 == 0 && k % 8 == 0 && k >= 64 && (a_kc || a_mc) && (b_kc || b_mc) && batch_ok &&
        c_cs == 1 && c_rs % 8 == 0 && m > 64 && (long long)((m + 127) / 128) * batch >= cu_tiles()) {
        p.fam = FAM_PIPE16K; p.bm = 128; p.bn = 64; p.a_mc = !a_kc; p.b_mc = !b_kc; p.edge = (m % 128) || n != 64; p.name = "pipe16k_128x64";
        return p;
    }
    // the same in fp32 (any C strides): bound by the MFMAs, which the resident kernel keeps fed without a wait per slab
    if (dtype == RP_DTYPE_FLOAT32 && allow_direct && !path_disabled("pipe32k") && n <= 64 && k % 4 == 0 && k >= 32 && (a_kc || (a_rs == 1 && a_cs % 4 == 0)) &&
        (b_kc || (b_cs == 1 && b_rs % 4 == 0)) && batch_ok && m > 64 && (long long)((m + 127) / 128) * batch >= cu_tiles()) {
        p.fam = FAM_PIPE32K; p.bm = 128; p.bn = 64; p.a_mc = !a_kc; p.b_mc = !b_kc; p.edge = (m % 128) || n != 64; p.name = "pipe32k_128x64";
        return p;
    }
    if (!mfma_ok) return p;
    p.a_mc = !a_kc;             // when both qualify (extent-1 corner cases) keep the row-major reading
    p.b_mc = b_mc;

    if (is16) {
        choose_tile16(p, batch, m, k, n);
    } else {
        p.fam = FAM_MFMAW;
        long long tiles128 = (long long)((m + 127) / 128) * ((n + 127) / 128) * batch;
        // a 128 x 128 tile over a 64-wide output would compute and fetch half of it for nothing
        if (m > 64 && n > 64 && tiles128 >= cu_tiles() / 2) { p.bm = 128; p.bn = 128; p.name = (dtype == RP_DTYPE_FLOAT32) ? "mfma32_128x128" : "mfma64_128x128"; }
        else { p.bm = 64; p.bn = 64; p.name = (dtype == RP_DTYPE_FLOAT32) ? "mfma32_64x64" : "mfma64_64x64"; }
        p.edge = (m % p.bm) || (n % p.bn) || (k % (dtype == RP_DTYPE_FLOAT32 ? 32 : 16));
    }
    return p;
}

static thread_local const char* g_last_kernel = "none";      // what rp_hip_last_gemm_kernel reports

static int run_gemm(const GemmArgs& g, int dtype) {
    Plan p = make_plan(g.batch, g.m, g.k, g.n, g.a_rs, g.a_cs, g.b_rs, g.b_cs, g.c_rs, g.c_cs, g.a_bs, g.b_bs, dtype);
    if (p.fam == FAM_PIPE32) {
        if (pipe32_takes(g)) { g_last_kernel = p.name; return launch_pipe32(g); }
        p = make_plan(g.batch, g.m, g.k, g.n, g.a_rs, g.a_cs, g.b_rs, g.b_cs, g.c_rs, g.c_cs, g.a_bs, g.b_bs, dtype, false);     // options, base pointers or spans it does not take
    }
    if (p.fam == FAM_PIPE16) {
        if (pipe16_takes(g)) { g_last_kernel = p.name; return launch_pipe16(g, dtype); }
        p = make_plan(g.batch, g.m, g.k, g.n, g.a_rs, g.a_cs, g.b_rs, g.b_cs, g.c_rs, g.c_cs, g.a_bs, g.b_bs, dtype, false);
    }
    if (p.fam == FAM_PIPE16K) {
        if (pipe16k_takes(g)) { g_last_kernel = p.name; return launch_pipe16k(g, dtype); }
        p = make_plan(g.batch, g.m, g.k, g.n, g.a_rs, g.a_cs, g.b_rs, g.b_cs, g.c_rs, g.c_cs, g.a_bs, g.b_bs, dtype, false);
    }
    if (p.fam == FAM_PIPE32K) {
        if (pipe32k_takes(g)) { g_last_kernel = p.name; return launch_pipe32k(g); }
        p = make_plan(g.batch, g.m, g.k, g.n, g.a_rs, g.a_cs, g.b_rs, g.b_cs, g.c_rs, g.c_cs, g.a_bs, g.b_bs, dtype, false);
    }
    if (p.fam == FAM_DIRECT32) {
        if (direct32_takes(g)) { g_last_kernel = p.name; return launch_direct32(g); }
        p = make_plan(g.batch, g.m, g.k, g.n, g.a_rs, g.a_cs, g.b_rs, g.b_cs, g.c_rs, g.c_cs, g.a_bs, g.b_bs, dtype, false);     // base pointers or spans it cannot address
    }
    if (p.fam != FAM_GENERIC && p.fam != FAM_TINY && !(aligned16(g.A) && aligned16(g.B))) { p.fam = FAM_GENERIC; p.name = "generic"; }
    g_last_kernel = p.name;
    switch (p.fam) {
        case FAM_MFMA16:
        case FAM_MFMA16_SKINNY: return launch_mfma16(g, p, dtype);
        case FAM_MFMAW:  return launch_mfmaw(g, p, dtype);
        case FAM_SKINNY: return launch_skinny(g, dtype);
        case FAM_TINY:   return launch_tiny(g, dtype);
        default:         return launch_generic(g, dtype);
    }
}

// C_z = A_z . B_z with B's k axis or its n axis given as segments (GemmArgs::seg_*): the MFMA kernels read every
// segment in place, at any alignment of whole elements.  For callers inside the library (the convolution), which
// guarantee: A with unit stride along k or m, B with unit stride along n and k a whole number of segments of whole
// slabs, or B with unit stride along k and n a whole number of segments.
int launch_gemm_segmented_b(const GemmArgs& g, int dtype) {
    const bool is16 = dtype == RP_DTYPE_FLOAT16 || dtype == RP_DTYPE_BFLOAT16;
    const int vec = 16 / (int)dtype_size(dtype);
    const int bk = is16 ? M16_BK : (dtype == RP_DTYPE_FLOAT32 ? 32 : 16);           // k slab of the kernel that will run
    const bool a_kc = g.a_cs == 1, a_mc = g.a_rs == 1 && g.m % vec == 0;
    const long long max_stride = 1ll << 22;
    bool ok = dtype_size(dtype) && (a_kc || a_mc) && g.seg_w > 0 && g.a_rs < max_stride && g.a_cs < max_stride && g.b_rs < max_stride && g.b_cs < max_stride &&
              g.batch <= 65535 && g.b_extent > 0 && g.b_extent < (1ll << 30);
    if (!is16) ok = ok && (a_kc ? g.a_rs % vec == 0 && g.k % vec == 0 : g.a_cs % vec == 0) && g.a_bs % vec == 0;     // the fp32 / fp64 kernel loads A with plain vector loads
    if (g.seg_k > 0) ok = ok && g.seg_n == 0 && g.b_cs == 1 && g.n % vec == 0 && g.seg_k % bk == 0 && g.k % g.seg_k == 0;    // segments along k
    else ok = ok && g.seg_n > 0 && g.b_rs == 1 && g.k % vec == 0 && g.n % g.seg_n == 0;                                     // segments along n
    // the folded store and the per-row bias exist on the vector path of the epilogue only
    if (g.c_fold_from > 0)
        ok = ok && g.c_cs == 1 && g.c_rs % vec == 0 && g.c_bs % vec == 0 && aligned16(g.C) && g.c_fold_from % vec == 0 && g.c_fold_to % vec == 0 &&
             g.c_fold_to <= g.c_fold_from && g.n % g.c_fold_from == 0;
    if (!ok) {
        set_error("segmented GEMM: operands outside what the MFMA kernels read in place");
        return -1;
    }
    if (is16) {
        Plan p{FAM_MFMA16, 64, 64, !a_kc, g.seg_k > 0, true, "mfma16"};
        choose_tile16(p, g.batch, g.m, g.k, g.n);
        return launch_mfma16(g, p, dtype);
    }
    Plan p{FAM_MFMAW, 64, 64, !a_kc, g.seg_k > 0, true, "mfmaw"};
    const long long tiles128 = (long long)((g.m + 127) / 128) * ((g.n + 127) / 128) * g.batch;
    if (g.m > 64 && g.n > 64 && tiles128 >= cu_tiles() / 2) { p.bm = 128; p.bn = 128; }
    p.edge = (g.m % p.bm) || (g.n % p.bn) || (g.k % bk);
    return launch_mfmaw(g, p, dtype);
}

// ============================================================================
// The entry point that allocates nothing (rp_hip_gemm_strided_batched_noalloc).
// Its split-k launchers take their workspace and arrival counters from one fixed
// device array instead of the pool.  Every GPU the library runs on holds its own
// copy of the array at its own address for the life of the process; host code
// never uses the array's name as an address, only the pointer that
// hipGetSymbolAddress returned for the device that was current.
// ============================================================================
constexpr size_t NOALLOC_COUNTER_BYTES = (size_t)SPLITK_MAX_TILES * sizeof(int);      // arrival counters, then the partial sums
constexpr size_t NOALLOC_WORKSPACE_BYTES = (size_t)RP_HIP_NOALLOC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[NOALLOC_COUNTER_BYTES + NOALLOC_WORKSPACE_BYTES];

constexpr int NOALLOC_MAX_DEVICES = 64;
static std::mutex g_scratch_mu;
static unsigned char* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};      // per device: where that device's copy of `scratch` lives
static thread_local unsigned char* g_noalloc_base = nullptr;        // non-null while the calling thread is inside the entry point
static thread_local bool g_noalloc_busy = false;                    // its workspace is handed out (one launcher at a time)
static thread_local bool g_noalloc_cleared = false;                 // this call has cleared the arrival counters

// Address of the current device's copy of the array, resolved once per device.
static unsigned char* noalloc_scratch_of_current_device() {
    int dev = 0;
    if (!check_hip(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) { set_error("rp_hip_gemm_strided_batched_noalloc: device ordinal %d is beyond the %d this entry point tracks", dev, NOALLOC_MAX_DEVICES); return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (!check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
        g_scratch_ptr[dev] = (unsigned char*)p;
    }
    return g_scratch_ptr[dev];
}

int gemm_workspace(void** ws, size_t bytes) {
    if (!g_noalloc_base) return rp_hip_malloc(ws, bytes);
    *ws = nullptr;
    if (bytes > NOALLOC_WORKSPACE_BYTES) {
        set_error("rp_hip_gemm_strided_batched_noalloc: this shape needs %zu bytes of split-k workspace, the fixed array holds %zu", bytes, NOALLOC_WORKSPACE_BYTES);
        return -1;
    }
    if (g_noalloc_busy) { set_error("rp_hip_gemm_strided_batched_noalloc: workspace requested twice"); return -1; }
    g_noalloc_busy = true;
    *ws = g_noalloc_base + NOALLOC_COUNTER_BYTES;
    return 0;
}

void gemm_workspace_release(void* ws) {
    if (!ws) return;
    if (g_noalloc_base && ws == g_noalloc_base + NOALLOC_COUNTER_BYTES) { g_noalloc_busy = false; return; }
    rp_hip_free(ws);
}

__global__ void __launch_bounds__(256) clear_counters_kernel(int* counters, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) counters[i] = 0;
}

bool noalloc_active() { return g_noalloc_base != nullptr; }

// The array keeps what the last call left.  The partial sums are fully overwritten before they are read; the arrival
// counters must read zero, and a launch that was cut short could have left some standing: the first launcher of a call
// that wants them has them cleared by a kernel (stream-ordered before the GEMM; not a memset node, so the call can be
// recorded into a graph).  Calls whose kernels use no counters launch nothing extra.
int* noalloc_arrival_counters() {
    if (!g_noalloc_base) return nullptr;
    if (!g_noalloc_cleared) {
        hipLaunchKernelGGL(clear_counters_kernel, dim3((SPLITK_MAX_TILES + 255) / 256), dim3(256), 0, current_stream(), (int*)g_noalloc_base, SPLITK_MAX_TILES);
        if (!check_launch("clear_counters_kernel")) return nullptr;
        g_noalloc_cleared = true;
    }
    return (int*)g_noalloc_base;
}

}  // namespace rp

using namespace rp;

extern "C" {

int rp_hip_gemm_strided_batched(void* C, const void* A, const void* B, const void* bias,
                                int batch, int m, int k, int n,
                                long long a_bs, long long a_rs, long long a_cs,
                                long long b_bs, long long b_rs, long long b_cs,
                                long long c_bs, long long c_rs, long long c_cs,
                                int accumulate, int dtype) {
    if (!C || !A || !B || batch <= 0 || m <= 0 || k <= 0 || n <= 0) {
        set_error("rp_hip_gemm_strided_batched: null operand or non-positive extent (batch=%d m=%d k=%d n=%d)", batch, m, k, n);
        return -1;
    }
    if (!dtype_size(dtype)) { set_error("rp_hip_gemm_strided_batched: unsupported dtype %d", dtype); return -1; }
    // (Batch strides may have any sign: matrix z of an operand starts z strides from matrix 0, which lets one launch
    // cover separately allocated matrices of equal shape.  Row and column strides address inside a matrix.)
    if (a_rs < 0 || a_cs < 0 || b_rs < 0 || b_cs < 0 || c_rs < 0 || c_cs < 0) {
        set_error("rp_hip_gemm_strided_batched: negative row or column stride");
        return -1;
    }
    // the batch rides on a grid axis that holds at most 65535 blocks: longer batches go in chunks
    constexpr int MAX_BATCH = 65535;
    const long long esz = (long long)dtype_size(dtype);
    for (int b0 = 0; b0 < batch; b0 += MAX_BATCH) {
        const int nb = batch - b0 < MAX_BATCH ? batch - b0 : MAX_BATCH;
        GemmArgs g{(char*)C + b0 * c_bs * esz, (const char*)A + b0 * a_bs * esz, (const char*)B + b0 * b_bs * esz, bias,
                   nb, m, k, n, a_bs, a_rs, a_cs, b_bs, b_rs, b_cs, c_bs, c_rs, c_cs, accumulate};
        if (run_gemm(g, dtype) != 0) return -1;
    }
    return 0;
}

int rp_hip_gemm_strided_batched_noalloc(void* C, const void* A, const void* B, const void* bias,
                                        int batch, int m, int k, int n,
                                        long long a_bs, long long a_rs, long long a_cs,
                                        long long b_bs, long long b_rs, long long b_cs,
                                        long long c_bs, long long c_rs, long long c_cs,
                                        int accumulate, int dtype) {
    if (g_noalloc_base) { set_error("rp_hip_gemm_strided_batched_noalloc: re-entered"); return -1; }
    unsigned char* base = noalloc_scratch_of_current_device();
    if (!base) return -1;
    g_noalloc_base = base;
    g_noalloc_busy = false;
    g_noalloc_cleared = false;
    const int rc = rp_hip_gemm_strided_batched(C, A, B, bias, batch, m, k, n, a_bs, a_rs, a_cs, b_bs, b_rs, b_cs, c_bs, c_rs, c_cs, accumulate, dtype);
    g_noalloc_base = nullptr;
    g_noalloc_busy = false;
    return rc;
}

int matmul_kernel_device(void* C, const void* A, const void* B, int m, int k, int n, int dtype) {
    return rp_hip_gemm_strided_batched(C, A, B, nullptr, 1, m, k, n, 0, k, 1, 0, n, 1, 0, n, 1, 0, dtype);
}

int rp_hip_linear_backward(void* dx, void* dw, void* db, const void* dy, const void* x, const void* w, int m, int k, int n,
                           long long x_rs, long long x_cs, long long w_rs, long long w_cs,
                           long long dx_rs, long long dx_cs, long long dw_rs, long long dw_cs,
                           int accumulate_dx, int accumulate_dw, int accumulate_db, int dtype) {
    if (!dy || (dx && !w) || (dw && !x) || m <= 0 || k <= 0 || n <= 0 || !dtype_size(dtype)) {
        set_error("rp_hip_linear_backward: null operand, non-positive extent or unsupported dtype (m=%d k=%d n=%d)", m, k, n);
        return -1;
    }
    if (x_rs < 0 || x_cs < 0 || w_rs < 0 || w_cs < 0 || dx_rs < 0 || dx_cs < 0 || dw_rs < 0 || dw_cs < 0) { set_error("rp_hip_linear_backward: negative stride"); return -1; }
    // dx[m, k] = dy[m, n] . w^T (w [k, n] read with its strides swapped); dw[k, n] = x^T . dy (x [m, k] likewise)
    GemmArgs gx{dx, dy, w, nullptr, 1, m, n, k, 0, n, 1, 0, w_cs, w_rs, 0, dx_rs, dx_cs, accumulate_dx};
    GemmArgs gw{dw, x, dy, nullptr, 1, k, m, n, 0, x_cs, x_rs, 0, n, 1, 0, dw_rs, dw_cs, accumulate_dw};
    bool fused = dtype == RP_DTYPE_FLOAT32 && (dx || dw);
    if (fused && dx) fused = make_plan(1, gx.m, gx.k, gx.n, gx.a_rs, gx.a_cs, gx.b_rs, gx.b_cs, gx.c_rs, gx.c_cs, 0, 0, dtype).fam == FAM_TINY;
    if (fused && dw) fused = make_plan(1, gw.m, gw.k, gw.n, gw.a_rs, gw.a_cs, gw.b_rs, gw.b_cs, gw.c_rs, gw.c_cs, 0, 0, dtype).fam == FAM_TINY;
    if (fused) {
        // small layer: one launch does all three, block for block what the separate launches would do
        if (!dx) gx.m = 0;
        if (!dw) gw.m = 0;
        return launch_linear_backward_tiny(gx, gw, db, dy, m, n, accumulate_db);
    }
    if (dx && run_gemm(gx, dtype) != 0) return -1;
    if (dw && run_gemm(gw, dtype) != 0) return -1;
    if (db && rp_hip_reduce_rows(db, dy, m, n, accumulate_db, dtype) != 0) return -1;
    return 0;
}

const char* rp_hip_last_gemm_kernel(void) { return g_last_kernel; }

const char* rp_hip_gemm_kernel_name(int batch, int m, int k, int n, long long a_rs, long long a_cs,
                                    long long b_rs, long long b_cs, long long c_rs, long long c_cs, int dtype) {
    if (batch <= 0 || m <= 0 || k <= 0 || n <= 0 || !dtype_size(dtype)) return "invalid";
    Plan p = make_plan(batch, m, k, n, a_rs, a_cs, b_rs, b_cs, c_rs, c_cs, 0, 0, dtype);
    return p.name;
}

}  // extern "C"
