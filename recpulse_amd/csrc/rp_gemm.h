// Shared declarations of the GEMM translation units: the problem descriptor,
// the dispatcher's plan, the XCD-aware tile schedule and the per-family launchers.
#pragma once
#include "rp_common.h"

#include <type_traits>

#include <cstdlib>
#include <cstring>

namespace rp {

struct GemmArgs {
    void* C;
    const void* A;
    const void* B;
    const void* bias;
    int batch, m, k, n;
    long long a_bs, a_rs, a_cs;
    long long b_bs, b_rs, b_cs;
    long long c_bs, c_rs, c_cs;
    int accumulate;
    // B's k axis in segments (MFMA kernels only; all zero = one plain matrix).  k is cut into segments of seg_k
    // elements (whole k slabs of the kernel); segment s = (sh, sw), sw = s % seg_w, starts at element offset sh * seg_sh + sw * seg_sw
    // from B and runs with B's strides from there.  This is how a convolution reads its taps from one zero-bordered
    // copy of the image instead of from a lowered matrix.  b_extent: elements of one batch entry of B that may be read.
    int seg_k, seg_w;
    long long seg_sh, seg_sw, b_extent;
    // Or B's n axis in segments of seg_n columns (B with unit stride along k): column j = (s, c) sits at the
    // segment's offset (same formula) plus c * b_cs.  This is the weight gradient: the reduction runs over positions
    // and every (tap, channel) column is a shifted plane of the padded image.
    int seg_n;
    // Epilogue options of the MFMA kernels (non-split path, C with unit column stride in whole 16-byte vectors).
    // bias_by_row: bias[m] is added to row m instead of bias[n] to column n.  c_fold_from / c_fold_to: output column
    // f = r * c_fold_from + c is stored at column r * c_fold_to + c when c < c_fold_to and dropped otherwise (both
    // whole 16-byte vectors): a product computed in the pitch of zero-bordered planes lands in dense planes.
    int bias_by_row, c_fold_from, c_fold_to;
};

enum Family { FAM_GENERIC = 0, FAM_SKINNY, FAM_MFMA16, FAM_MFMA16_SKINNY, FAM_MFMAW, FAM_TINY, FAM_DIRECT32, FAM_PIPE32, FAM_PIPE16, FAM_PIPE16K, FAM_PIPE32K };

struct Plan {
    Family fam;
    int bm, bn;
    bool a_mc, b_mc, edge;
    const char* name;
};

constexpr int SK_MAX_M = 8;           // rows the skinny kernel takes
constexpr int SK_MAX_GROUPS = 4096;   // column groups it can track
constexpr int M16_BK = 64;            // k slab of the 16-bit MFMA kernels

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) double f64x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2_t;

// ---- small helpers shared by the kernels ----
// compile-time loop: f(integral_constant<int, I>) for I in [I0, N)
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Raw buffer descriptor over [base, base + bytes): loads past the end return zero, stores past it are dropped.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_rsrc(const void* base, long long bytes) {
    const int n = bytes <= 0 ? 0 : (bytes > 0x7fffffffll ? 0x7fffffff : (int)bytes);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, n, 0x00020000);
}
constexpr uint32_t BUFFER_OOB = 0x80000000u;     // an offset no descriptor covers

// Tile `id` of a batch walked matrix by matrix, row-major inside a matrix: matrix and origin of its BM x BN tile.
struct TileOrigin { int z, m0, n0; };
template <int BM, int BN>
__device__ __forceinline__ TileOrigin tile_origin(unsigned id, unsigned per_matrix, unsigned tiles_n) {
    TileOrigin t;
    const unsigned z = id / per_matrix, tile = id - z * per_matrix, tm = tile / tiles_n;
    t.z = (int)z;
    t.m0 = (int)tm * BM;
    t.n0 = (int)(tile - tm * tiles_n) * BN;
    return t;
}

// Tile scheduling shared by the MFMA kernels.
// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so a
// linear block id is first split into (xcd, slot); every XCD then walks its
// own sequence of 4x8-tile super-tiles, which keeps the 32 tiles resident on an
// XCD at one time inside a compact window of the output (4 A row panels and
// 8 B column panels shared through that XCD's L2).
// ----------------------------------------------------------------------------
struct TileCoord { int tm, tn; bool valid; };

// The XCD-aware order launches whole rounds of 8 super-tiles (one per XCD): a super-tile count that is neither a
// multiple of 8 nor large leaves XCDs idle in the last round (with 2 super-tiles only 2 of the 8 XCDs would work,
// for every matrix of a batch), and super-tiles that hang over the edge of the output give their XCD less work
// than the others (5 x 25 tiles make 8 super-tiles holding 32, 32, 32, 4, 8, 8, 8 and 1 tiles).  Unless at least
// nine tenths of the launched slots hold a tile, plain row-major order is used, which deals tiles evenly.
__host__ __device__ __forceinline__ bool schedule_by_xcd(int tiles_m, int tiles_n) {
    constexpr int XCDS = 8, GM = 4, GN = 8;
    const int sup = ((tiles_m + GM - 1) / GM) * ((tiles_n + GN - 1) / GN);
    if (!(sup % XCDS == 0 || sup >= 4 * XCDS)) return false;
    const long long slots = (long long)((sup + XCDS - 1) / XCDS) * XCDS * GM * GN;
    return (long long)tiles_m * tiles_n * 10 >= slots * 9;
}

__device__ __forceinline__ TileCoord schedule_tile(int bid, int tiles_m, int tiles_n) {
    constexpr int XCDS = 8, GM = 4, GN = 8, PER = GM * GN;
    if (!schedule_by_xcd(tiles_m, tiles_n)) {
        TileCoord lin;
        lin.tm = bid / tiles_n; lin.tn = bid % tiles_n; lin.valid = bid < tiles_m * tiles_n;
        return lin;
    }
    int sup_m = (tiles_m + GM - 1) / GM, sup_n = (tiles_n + GN - 1) / GN;
    int xcd = bid % XCDS, slot = bid / XCDS;
    int sup = (slot / PER) * XCDS + xcd;
    int within = slot % PER;
    TileCoord tc;
    int sm = sup / sup_n, sn = sup % sup_n;
    tc.tm = sm * GM + within / GN;
    tc.tn = sn * GN + within % GN;
    tc.valid = (sm < sup_m) && (tc.tm < tiles_m) && (tc.tn < tiles_n);
    return tc;
}

static inline int scheduled_grid(int tiles_m, int tiles_n) {
    constexpr int XCDS = 8, GM = 4, GN = 8, PER = GM * GN;
    if (!schedule_by_xcd(tiles_m, tiles_n)) return tiles_m * tiles_n;
    int sup = ((tiles_m + GM - 1) / GM) * ((tiles_n + GN - 1) / GN);
    int rounds = (sup + XCDS - 1) / XCDS;
    return rounds * XCDS * PER;
}


// ----------------------------------------------------------------------------
// Single-launch finish of a k split.
// The blocks that share an output tile write fp32 partial tiles [split][m][n] with device-scope stores (cache
// policy sc1: written through the per-XCD L2s, which are not coherent with each other), wait until their own
// stores are acknowledged, and count themselves in with a device-scope atomic.  The block that arrives last
// re-reads every split's tile with device-scope loads, adds them in split order (so the result does not depend
// on which block that is), runs the epilogue and leaves the counter at zero for the next launch.  No cache-wide
// write-back or invalidate is involved.  The finish is a chain of three device-scope round trips (store
// acknowledge, atomic, partial loads), about 3 us: it beats a second launch for the long streaming kernel, whose
// blocks all end together, and loses to it for the few-microsecond split-k GEMMs of small layers, which
// therefore keep the separate combine kernel.
// ----------------------------------------------------------------------------
constexpr int SPLITK_DEVICE_SCOPE = 16;      // buffer cache-policy bit sc1
constexpr int SPLITK_MAX_TILES = 1024;       // arrival counters per device

__device__ __forceinline__ __amdgpu_buffer_rsrc_t splitk_rsrc(const float* partials, long long bytes) {
    int n = bytes <= 0 ? 0 : (bytes > 0x7fffffffll ? 0x7fffffff : (int)bytes);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(partials), 0, n, 0x00020000);
}

// The device's block of SPLITK_MAX_TILES zeroed arrival counters (created on first use, kept for the life of the
// process), or nullptr when the single-launch finish cannot be used: more tiles than counters, partials of 2 GiB
// or more, "one_launch_splitk" in RP_HIP_DISABLE, or an allocation failure (then last_error is set and *failed is true).
// Like the workspace pool the block is not stream-aware: launches that may run at the same time on different
// streams of one device must be serialised by the caller.
int* splitk_arrival_counters(long long tiles, size_t partial_bytes, bool* failed);

// Workspace of a GEMM launcher (split-k partial sums): a pool block, or, inside the entry point that allocates
// nothing, a piece of that entry point's fixed device array (then -1 with an error when it is too small).
int gemm_workspace(void** ws, size_t bytes);
void gemm_workspace_release(void* ws);
// Inside the entry point that allocates nothing: its arrival counters, cleared by a kernel on the current stream the
// first time a call asks for them (nullptr with an error when that launch fails).
bool noalloc_active();
int* noalloc_arrival_counters();

// per-family launchers (dtype is one of the RP_DTYPE_* codes the family supports)
int launch_generic(const GemmArgs& g, int dtype);
int launch_skinny(const GemmArgs& g, int dtype);
int launch_mfma16(const GemmArgs& g, const Plan& p, int dtype);
bool stream128_shape(int batch, int m, int k, int n);      // shapes the streaming kernel on 128-column strips is chosen for (row-major A and B)
bool stream128_takes(const GemmArgs& g);
int launch_stream128(const GemmArgs& g, int dtype);
int launch_mfmaw(const GemmArgs& g, const Plan& p, int dtype);
int launch_tiny(const GemmArgs& g, int dtype);
// The tiles of this workgroup in a grid of resident workgroups (one per CU): first, first + stride, ... below last.
// Workgroups go to the XCDs round robin, so workgroup b sits on XCD b % 8.  Every XCD gets a contiguous eighth of the
// tiles, and its workgroups walk that range side by side: at any time the CUs of an XCD work on neighbouring tiles,
// and what those share (the rows of Q and K of a batch entry, the whole of V) is fetched into that XCD's L2 once, while
// it is still needed.  (A contiguous run per workgroup shares as much in total, but at different times: by the time
// the second tile of a batch entry comes up on another CU, the first one's operands have left the L2.)
__device__ __forceinline__ void resident_tile_walk(unsigned total, unsigned& first, unsigned& last, unsigned& stride) {
    const unsigned grid = gridDim.x, b = blockIdx.x;
    if (grid % 8 != 0) { first = b; last = total; stride = grid; return; }
    const unsigned xcd = b % 8, slot = b / 8, per_xcd = (total + 7) / 8;
    const unsigned begin = xcd * per_xcd < total ? xcd * per_xcd : total;
    last = begin + per_xcd < total ? begin + per_xcd : total;
    first = begin + slot < last ? begin + slot : last;
    stride = grid / 8;
}

// A batched launch is a grid of (schedule slots, matrices), and its workgroups go to the XCDs round robin in launch
// order, so the tiles of one small matrix would land on all 8 L2s and each would fetch that matrix's operands.  Unless a
// matrix has enough tiles to be scheduled by XCD itself (or k is split over the grid's third axis), every XCD takes a
// contiguous eighth of the (matrix, slot) pairs instead, side by side: the tiles that share operands run at the same
// time on one L2.  (Used by the 16-bit tiled kernel, whose batched products are bound by memory traffic: 192 products of
// 512 x 128 x 512 in bf16 take 42 us instead of 50, 512 x 512 x 128 28 us instead of 37.  The fp32 kernel's are bound by
// the MFMAs and lose 3 % to it.)
__device__ __forceinline__ void batched_block(int tiles_m, int tiles_n, int& slot, int& z) {
    slot = (int)blockIdx.x;
    z = (int)blockIdx.y;
    if (gridDim.y == 1 || gridDim.z != 1 || schedule_by_xcd(tiles_m, tiles_n)) return;
    const unsigned per = gridDim.x, total = per * gridDim.y, b = blockIdx.y * per + blockIdx.x;
    const unsigned xcd = b % 8, q = total / 8, r = total % 8;
    const unsigned idx = xcd * q + (xcd < r ? xcd : r) + b / 8;          // XCD x owns q (+ 1 if x < r) consecutive pairs
    z = (int)(idx / per);
    slot = (int)(idx - (unsigned)z * per);
}

bool direct32_takes(const GemmArgs& g);          // pointer alignment and spans the short-k fp32 kernel can address
int launch_direct32(const GemmArgs& g);
bool pipe32_takes(const GemmArgs& g);          // options, alignment and spans the k-contiguous short-k fp32 kernel can address
int launch_pipe32(const GemmArgs& g);
bool pipe16_takes(const GemmArgs& g);          // the same for the 16-bit kernel (C row-major in whole 8-byte quads)
int launch_pipe16(const GemmArgs& g, int dtype);
bool pipe16k_takes(const GemmArgs& g);         // the 16-bit kernel for outputs of at most 64 columns and any k
int launch_pipe16k(const GemmArgs& g, int dtype);
bool pipe32k_takes(const GemmArgs& g);         // and its fp32 twin
int launch_pipe32k(const GemmArgs& g);
int launch_gemm_segmented_b(const GemmArgs& g, int dtype);
int launch_linear_backward_tiny(const GemmArgs& gx, const GemmArgs& gw, void* db, const void* dy, int rows, int cols, int accumulate_db);
// adds k-split partials [g.batch][nsplit][part_rows][n] (fp32, rows beyond g.m unused) in split order and runs the epilogue into C
int launch_splitk_combine(const GemmArgs& g, const float* partials, int nsplit, int part_rows, int dtype);

}  // namespace rp
