// bf16 / fp16 GEMMs with few rows and deep k: the cost is streaming B once from HBM.
//
// Row-major A times row-major B takes a streaming kernel, in which B never touches LDS and the k splits are added
// inside the same launch by the last block to arrive: the one below on 256-column strips up to 4 rows, the one in
// rp_gemm_mfma16_stream128.hip on 128-column strips up to 32 rows (this one again, up to 16 rows, when that one is
// switched off).  Other operand layouts and more rows take the tiled kernel with a 32 x 128 block tile, whose fp32
// partials a second kernel combines.  All split k across the grid so that enough waves stream B to saturate HBM,
// and all add the splits in split order.
#include "rp_gemm_mfma16_kernel.h"


namespace rp {

// ============================================================================
// Streaming kernel.  One wave owns 256 adjacent columns of B and a set of
// 16-row "rounds" of k.  In a round, lane (h, j) = (lane / 32, lane % 32)
// loads 16 bytes (columns 8j .. 8j+7) of the 8 k rows 8h .. 8h+7: every load
// instruction reads two 512-byte row segments.  The 8 x 8 block of 16-bit
// values a lane now holds is transposed in registers (byte permutes) into 8
// MFMA B-operands, one per column residue c: operand c carries column 8j + c
// at k = 8h .. 8h+7, which is exactly the 32x32x16 layout (lane % 32 selects
// the column, lane / 32 the k half).  The A operand is a 16-byte load of row
// lane % 32 (zero beyond m).  MFMA c therefore accumulates the 32 x 32 tile of
// output columns {8j + c}; 8 accumulators cover the wave's 256 columns.
// Loads for two rounds are always in flight per wave (deeper queues only add
// waiting: four rounds in flight cost 0.6 us per launch, one round 3.5 us) and are issued
// unconditionally (out-of-range rounds get an empty buffer descriptor and read
// zeros), so the waits the compiler inserts count loads exactly.
//
// Rounds are dealt cyclically: round q of k belongs to split q % nsplit, and
// inside a block to wave (q / nsplit) % 4.  At any moment the grid as a whole
// therefore reads one contiguous window of B (nsplit * 4 rounds of whole rows),
// which the memory system serves 5 - 8 % faster than the same blocks each
// walking a range of k of its own (the ranges lie a power of two apart).
//
// The block's 4 waves add their tiles through LDS in wave order, 8 rows at a
// time, and the block writes one fp32 partial (or, without a k split, the
// finished output).  With `arrivals` the block then counts itself in, and the
// last block of its column group to do so adds the group's partials in split
// order and writes the output (otherwise a second kernel does).
//
// Placement.  The grid is one-dimensional and block b stands for (XCD x = b % 8,
// slot b / 8): workgroups are dealt to the XCDs round robin, so all splits of
// column group 8i + x are given slots of XCD x.  When the host has verified that
// rule on the device (`local`), the partials and the arrival count never leave
// that XCD's L2: plain stores (complete when the L2 has them), an atomic that the
// L2 executes, and plain loads (the finishing CU's vector cache holds none of them yet).
// Otherwise they are exchanged at device scope (written through to memory and
// read back from there), which costs about 1.5 us more per launch.
// ============================================================================
constexpr int SS_WAVES = 4, SS_COLS = 256, SS_ROUND = 16, SS_RED_PITCH = SS_COLS + 8;
constexpr int SS_MAX_M = 16;
constexpr int SS_DEPTH = 2;            // rounds a wave keeps in flight (register slots): 16 KB per wave, 16 MB over the chip

template <typename T, int MT>          // MT: rows the epilogue keeps (8 or 16; m <= MT)
__global__ void __launch_bounds__(256) gemm_stream16_kernel(GemmArgs g, float* partials, int groups, int nsplit, int* arrivals, int local) {
    extern __shared__ __attribute__((aligned(16))) float red[];          // [SS_WAVES][MT][SS_RED_PITCH]
    __shared__ bool arrived_last;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);       // scalar, so that buffer descriptors built from it are too
    const int h = lane >> 5, j = lane & 31;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int group = (slot / nsplit) * 8 + xcd, split = slot % nsplit;
    if (group >= groups) return;                                           // (whole blocks, before any barrier)
    const int n0 = group * SS_COLS;
    const int total_rounds = (g.k + SS_ROUND - 1) / SS_ROUND;
    const int mine = total_rounds > split ? (total_rounds - split + nsplit - 1) / nsplit : 0;      // rounds of this block
    const int my_rounds = mine > wave ? (mine - wave + SS_WAVES - 1) / SS_WAVES : 0;               // and of this wave

    const uint16_t* Bm = (const uint16_t*)g.B;
    const uint16_t* Am = (const uint16_t*)g.A;
    const long long b_rs = g.b_rs, a_rs = g.a_rs;
    const char* b_end = (const char*)(Bm + ((long long)(g.k - 1) * b_rs + g.n));
    const char* a_end = (const char*)(Am + ((long long)(g.m - 1) * a_rs + g.k));

    uint32_t b_off[8];
#pragma unroll
    for (int e = 0; e < 8; e++)
        b_off[e] = (n0 + 8 * j < g.n) ? (uint32_t)(((long long)(8 * h + e) * b_rs + 8 * j) * 2) : BUFFER_OOB;
    const uint32_t a_off = (j < g.m) ? (uint32_t)(((long long)j * a_rs + 8 * h) * 2) : BUFFER_OOB;

    u32x4_t raw[SS_DEPTH][8], araw[SS_DEPTH];
    // request round r of this wave into register slot SLOT (r beyond the wave's share reads zeros)
    auto request = [&](auto slotc, int r) {
        constexpr int SLOT = decltype(slotc)::value;
        const int kr = ((r * SS_WAVES + wave) * nsplit + split) * SS_ROUND;
        const bool live = r < my_rounds;
        const char* bb = (const char*)(Bm + (long long)kr * b_rs + n0);
        const char* ab = (const char*)(Am + kr);
        __amdgpu_buffer_rsrc_t b_rsrc = buffer_rsrc(bb, live ? (long long)(b_end - bb) : 0);
        __amdgpu_buffer_rsrc_t a_rsrc = buffer_rsrc(ab, live ? (long long)(a_end - ab) : 0);
#pragma unroll
        for (int e = 0; e < 8; e++) raw[SLOT][e] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)b_off[e], 0, 2);
        araw[SLOT] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)((kr + 8 * h < g.k) ? a_off : BUFFER_OOB), 0, 0);
    };

    f32x16_t acc[8];
#pragma unroll
    for (int c = 0; c < 8; c++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[c][v] = 0.f;

    // consume slot SLOT (round r), then refill it with round r + SS_DEPTH
    auto consume = [&](auto slotc, int r) {
        constexpr int SLOT = decltype(slotc)::value;
        // in-register 8 x 8 transpose of 16-bit values: operand c, dword d = (k row 2d, k row 2d+1) of column c
        u32x4_t opb[8];
#pragma unroll
        for (int c = 0; c < 8; c++)
#pragma unroll
            for (int d = 0; d < 4; d++)
                opb[c][d] = __builtin_amdgcn_perm(raw[SLOT][2 * d + 1][c / 2], raw[SLOT][2 * d][c / 2], (c & 1) ? 0x07060302u : 0x05040100u);
        // (A's fragment is moved to registers of its own for the same reason.)
        u32x4_t acopy;
#pragma unroll
        for (int d = 0; d < 4; d++) asm volatile("v_mov_b32 %0, %1" : "=v"(acopy[d]) : "v"(araw[SLOT][d]));
        s16x8_t opa = __builtin_bit_cast(s16x8_t, acopy);
        // The transposed operands must exist before the slot is refilled: then the refill can land in the very
        // registers the slot occupies and nothing has to be copied (behind a full wait) at the loop's back edge.
#pragma unroll
        for (int c = 0; c < 8; c++) asm volatile("" : "+v"(opb[c]) : : "memory");
        __builtin_amdgcn_sched_barrier(0);
        request(slotc, r + SS_DEPTH);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 8; c++) acc[c] = mfma16_ops<T>::mma(opa, __builtin_bit_cast(s16x8_t, opb[c]), acc[c]);
        __builtin_amdgcn_sched_barrier(0);
    };

    // (requests stay in slot order: the wait for a slot counts the loads issued after it)
    static_for<0, SS_DEPTH>([&](auto sc) { request(sc, decltype(sc)::value); __builtin_amdgcn_sched_barrier(0); });
    for (int r = 0; r < my_rounds; r += SS_DEPTH)
        static_for<0, SS_DEPTH>([&](auto sc) { consume(sc, r + decltype(sc)::value); });
    // ---- the block's waves add their tiles through LDS ----
    // accumulator register v of a 32x32 tile holds row 8*(v/4) + 4*h + v%4 at column j (of residue c)
    T* C = (T*)g.C;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    const bool c_vec = g.c_cs == 1 && g.c_rs % 4 == 0 && ((uintptr_t)C & 7) == 0;       // a quad of outputs is one aligned 8-byte store
    const __amdgpu_buffer_rsrc_t part_rsrc = buffer_rsrc(partials, partials ? (long long)nsplit * g.m * g.n * 4 : 0);
    // four outputs of one row: the epilogue of each, stored as one vector where the layout allows
    auto store_quad = [&](int row, int col, f32x4_t sum) {
        T y[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            T* pc = C + (long long)row * g.c_rs + (long long)(col + e) * g.c_cs;
            T old = accum ? *pc : T{};
            y[e] = finish<T>(sum[e], has_bias, has_bias ? bias[col + e] : T{}, accum, old);
        }
        if (c_vec) {
            u32x2_t w = {(uint32_t)y[0].bits | ((uint32_t)y[1].bits << 16), (uint32_t)y[2].bits | ((uint32_t)y[3].bits << 16)};
            *(u32x2_t*)(C + (long long)row * g.c_rs + col) = w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) C[(long long)row * g.c_rs + (long long)(col + e) * g.c_cs] = y[e];
        }
    };
    // A lane holds columns 8j .. 8j+7 of its rows.  In LDS a row is two planes of 128 floats, columns 8j .. 8j+3 at
    // float 4j of the first and columns 8j+4 .. 8j+7 at float 4j of the second, so that both the waves' stores and
    // the block's reads below are 16 bytes per lane at consecutive addresses.
#pragma unroll
    for (int p = 0; p < MT / 8; p++)
#pragma unroll
        for (int vv = 0; vv < 4; vv++) {
            const int r = 8 * p + 4 * h + vv;
            if (r >= g.m) continue;
            float* dst = red + (wave * MT + r) * SS_RED_PITCH + 4 * j;
            *(f32x4_t*)dst = f32x4_t{acc[0][4 * p + vv], acc[1][4 * p + vv], acc[2][4 * p + vv], acc[3][4 * p + vv]};
            *(f32x4_t*)(dst + 128) = f32x4_t{acc[4][4 * p + vv], acc[5][4 * p + vv], acc[6][4 * p + vv], acc[7][4 * p + vv]};
        }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MT / 4; i++) {
        const int idx = threadIdx.x + 256 * i, r = idx / 64, plane = (idx % 64) / 32, jj = idx % 32;
        const int at_lds = r * SS_RED_PITCH + 128 * plane + 4 * jj;
        const int gn = n0 + 8 * jj + 4 * plane;
        if (r >= g.m || gn >= g.n) continue;                             // n is a multiple of 4, so a quad is wholly in or out
        f32x4_t sum = *(const f32x4_t*)(red + at_lds);
#pragma unroll
        for (int w = 1; w < SS_WAVES; w++) sum += *(const f32x4_t*)(red + w * MT * SS_RED_PITCH + at_lds);
        if (nsplit > 1) {
            const long long at = ((long long)split * g.m + r) * g.n + gn;
            if (!arrivals) *(f32x4_t*)(partials + at) = sum;
            else if (local) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sum), part_rsrc, (int)(at * 4), 0, 0);
            else __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sum), part_rsrc, (int)(at * 4), 0, SPLITK_DEVICE_SCOPE);
        } else store_quad(r, gn, sum);
    }
    if (nsplit == 1 || !arrivals) return;

    // ---- single-launch finish: the last block of this column group to arrive adds all splits ----
    // Every thread waits until its own partial stores are acknowledged (by the XCD's L2, or by memory for
    // device-scope stores) before the block's arrival is counted.  No cache-wide write-back is needed.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        int before;
        if (local) before = __hip_atomic_fetch_add(arrivals + group, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);    // executed by this XCD's L2
        else before = __hip_atomic_fetch_add(arrivals + group, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        arrived_last = before == nsplit - 1;
    }
    __syncthreads();
    if (!arrived_last) return;
    // (Loads of the partials miss this CU's vector cache, which fills on the CU's own loads only and starts every
    // launch empty: the one block of a launch that reads a group's partials reads them here for the first time.)
    const long long split_stride = (long long)g.m * g.n;
    constexpr int QPR = SS_COLS / 4;                     // quads per row of the block's columns
    constexpr int QN = MT >= 16 ? 4 : 2;                 // quads per thread and pass: a pass covers 4 * QN rows
    // the loads of eight splits of all of a thread's quads are in flight together
    for (int r0 = 0; r0 < g.m; r0 += 4 * QN) {
        long long at[QN];
        bool live[QN];
        int row[QN], col[QN];
#pragma unroll
        for (int q = 0; q < QN; q++) {
            const int idx = threadIdx.x + 256 * q;
            row[q] = r0 + idx / QPR; col[q] = n0 + (idx % QPR) * 4;
            live[q] = row[q] < g.m && col[q] < g.n;
            at[q] = live[q] ? ((long long)row[q] * g.n + col[q]) * 4 : (long long)BUFFER_OOB;      // bytes; dead quads read zeros
        }
        f32x4_t sum[QN];
#pragma unroll
        for (int q = 0; q < QN; q++) sum[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < nsplit; sp += 8) {
            u32x4_t v[QN][8];
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int q = 0; q < QN; q++) {
                    const bool in = live[q] && sp + u < nsplit;
                    const int off = in ? (int)(at[q] + (sp + u) * split_stride * 4) : (int)BUFFER_OOB;
                    if (local) v[q][u] = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, off, 0, 0);
                    else v[q][u] = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, off, 0, SPLITK_DEVICE_SCOPE);
                }
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int q = 0; q < QN; q++) sum[q] += __builtin_bit_cast(f32x4_t, v[q][u]);       // split order; absent splits add +0
        }
#pragma unroll
        for (int q = 0; q < QN; q++)
            if (live[q]) store_quad(row[q], col[q], sum[q]);
    }
    if (threadIdx.x == 0) {                                          // ready for the next launch
        if (local) __hip_atomic_store(arrivals + group, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else __hip_atomic_store(arrivals + group, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename T, int MT>
static int launch_stream16_mt(const GemmArgs& g, float* partials, int groups, int nsplit, int* arrivals, int local) {
    constexpr size_t smem = (size_t)SS_WAVES * MT * SS_RED_PITCH * sizeof(float);
    auto kern = gemm_stream16_kernel<T, MT>;
    if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
    hipLaunchKernelGGL(kern, dim3(8 * ((groups + 7) / 8) * nsplit), dim3(256), smem, current_stream(), g, partials, groups, nsplit, arrivals, local);
    return check_launch("gemm_stream16_kernel") ? 0 : -1;
}

template <typename T>
static int launch_stream16_t(const GemmArgs& g, float* partials, int groups, int nsplit, int* arrivals, int local) {
    if (g.m <= 8) return launch_stream16_mt<T, 8>(g, partials, groups, nsplit, arrivals, local);
    return launch_stream16_mt<T, 16>(g, partials, groups, nsplit, arrivals, local);
}

static int launch_stream16(const GemmArgs& g, int dtype) {
    const int groups = (g.n + SS_COLS - 1) / SS_COLS;
    constexpr int QUANTUM = SS_WAVES * SS_ROUND;             // k rows one pass of a block's waves covers
    // one block per CU (a wave per SIMD, its registers holding the rounds in flight), each at least four passes deep
    int nsplit = (256 + groups - 1) / groups;
    int max_split = g.k / (4 * QUANTUM) > 0 ? g.k / (4 * QUANTUM) : 1;
    if (nsplit > max_split) nsplit = max_split;
    const size_t part_bytes = (size_t)nsplit * g.m * g.n * sizeof(float);
    void* ws = nullptr;
    if (nsplit > 1 && gemm_workspace(&ws, part_bytes) != 0) return -1;
    int* arrivals = nullptr;
    if (nsplit > 1) {
        bool failed = false;
        arrivals = splitk_arrival_counters(groups, part_bytes, &failed);
        if (failed) { gemm_workspace_release(ws); return -1; }
    }
    // The arrival counters of a device serve launches of both kinds of exchange.  That is safe because launches
    // on one stream follow each other and every launch leaves its counters at zero: whatever copy of a counter an
    // L2 still holds from an earlier launch reads zero, like memory.
    const int local = arrivals && workgroups_share_xcd_by_residue() ? 1 : 0;
    int rc;
    if (dtype == RP_DTYPE_BFLOAT16) rc = launch_stream16_t<bf16_t>(g, (float*)ws, groups, nsplit, arrivals, local);
    else rc = launch_stream16_t<f16_t>(g, (float*)ws, groups, nsplit, arrivals, local);
    if (rc == 0 && nsplit > 1 && !arrivals) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, dtype);
    if (ws) gemm_workspace_release(ws);          // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

// ---- tiled kernel for the other operand layouts ----
template <typename T>
static int launch_skinny16_t(const GemmArgs& g, const Plan& p, float* partials, int nsplit, int k_per_split) {
    constexpr int BM = 32, BN = 128, WGM = 1;
    if (!p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, false, true, true, true>(g, partials, nsplit, k_per_split);
    if (!p.a_mc && !p.b_mc) return m16_launch<T, BM, BN, WGM, false, false, true, true>(g, partials, nsplit, k_per_split);
    if (p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, true, true, true, true>(g, partials, nsplit, k_per_split);
    return m16_launch<T, BM, BN, WGM, true, false, true, true>(g, partials, nsplit, k_per_split);
}

int launch_mfma16_skinny(const GemmArgs& g, const Plan& p, int dtype) {
    if (dtype != RP_DTYPE_BFLOAT16 && dtype != RP_DTYPE_FLOAT16) { set_error("mfma16 skinny GEMM: unsupported dtype %d", dtype); return -1; }
    // row-major A and B: 256-column strips up to 4 rows (0.2 us faster there), 128-column strips up to 32 rows
    const bool wide = g.batch == 1 && !p.a_mc && p.b_mc && g.m <= SS_MAX_M && !path_disabled("stream16");
    const bool narrow = !p.a_mc && p.b_mc && stream128_takes(g);
    if (wide && (g.m <= 4 || !narrow)) return launch_stream16(g, dtype);
    if (narrow) return launch_stream128(g, dtype);
    constexpr int BN = 128;
    const int tiles = ((g.n + BN - 1) / BN) * ((g.m + 31) / 32) * g.batch;
    // about three blocks per CU in flight, each split at least four slabs deep
    int nsplit = (768 + tiles - 1) / tiles;
    int max_split = g.k / (4 * M16_BK) > 0 ? g.k / (4 * M16_BK) : 1;
    if (nsplit > max_split) nsplit = max_split;
    int k_per_split = ((g.k + nsplit - 1) / nsplit + M16_BK - 1) / M16_BK * M16_BK;
    nsplit = (g.k + k_per_split - 1) / k_per_split;
    void* ws = nullptr;
    if (gemm_workspace(&ws, (size_t)g.batch * nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
    int rc;
    if (dtype == RP_DTYPE_BFLOAT16) rc = launch_skinny16_t<bf16_t>(g, p, (float*)ws, nsplit, k_per_split);
    else rc = launch_skinny16_t<f16_t>(g, p, (float*)ws, nsplit, k_per_split);
    if (rc == 0) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, dtype);
    gemm_workspace_release(ws);          // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

}  // namespace rp
