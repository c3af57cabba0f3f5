// bf16 / fp16 GEMMs with few rows (m <= 32) and deep k: the cost is streaming B once from HBM.
//
// Row-major A (m <= 16) times row-major B takes the streaming kernel below: B never touches LDS, and the k
// splits are added inside the same launch by the last block to arrive.  Other operand layouts and 17..32 rows
// take the tiled kernel with a 32 x 128 block tile, whose fp32 partials a second kernel combines.  Both split k
// across the grid so that enough waves stream B to saturate HBM, and both add the splits in split order.
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
// Loads for four rounds are always in flight per wave and are issued
// unconditionally (out-of-range rounds get an empty buffer descriptor and read
// zeros), so the waits the compiler inserts count loads exactly.
// The block's 4 waves take interleaved rounds; they add their tiles through
// LDS in wave order, 8 rows at a time, and the block writes one fp32 partial
// (or, without a k split, the finished output).  With `arrivals` the block
// then counts itself in, and the last block of its column group to do so adds
// the group's partials and writes the output (otherwise a second kernel does).
// ============================================================================
constexpr int SS_WAVES = 4, SS_COLS = 256, SS_ROUND = 16, SS_RED_PITCH = SS_COLS + 8;
constexpr int SS_MAX_M = 16;
constexpr int SS_DEPTH = 4;            // rounds a wave keeps in flight (register slots)

template <typename T, int MT>          // MT: rows the epilogue keeps (8 or 16; m <= MT)
__global__ void __launch_bounds__(256) gemm_stream16_kernel(GemmArgs g, float* partials, int k_per_split, int* arrivals) {
    __shared__ __attribute__((aligned(16))) float red[SS_WAVES * 8 * SS_RED_PITCH];
    __shared__ bool arrived_last;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);       // scalar, so that buffer descriptors built from it are too
    const int h = lane >> 5, j = lane & 31;
    const int n0 = blockIdx.x * SS_COLS;
    const int split = blockIdx.y, nsplit = gridDim.y;
    const int kb = split * k_per_split;                                   // a multiple of SS_WAVES * SS_ROUND
    const int ke = kb + k_per_split < g.k ? kb + k_per_split : g.k;
    const int rounds = (ke - kb + SS_ROUND - 1) / SS_ROUND;               // in this block
    const int my_rounds = rounds > wave ? (rounds - wave + SS_WAVES - 1) / SS_WAVES : 0;

    const uint16_t* Bm = (const uint16_t*)g.B;
    const uint16_t* Am = (const uint16_t*)g.A;
    const long long b_rs = g.b_rs, a_rs = g.a_rs;
    const char* b_end = (const char*)(Bm + ((long long)(g.k - 1) * b_rs + g.n));
    const char* a_end = (const char*)(Am + ((long long)(g.m - 1) * a_rs + g.k));

    uint32_t b_off[8];
#pragma unroll
    for (int e = 0; e < 8; e++)
        b_off[e] = (n0 + 8 * j < g.n) ? (uint32_t)(((long long)(8 * h + e) * b_rs + 8 * j) * 2) : M16_OOB;
    const uint32_t a_off = (j < g.m) ? (uint32_t)(((long long)j * a_rs + 8 * h) * 2) : M16_OOB;

    u32x4_t raw[SS_DEPTH][8], araw[SS_DEPTH];
    // request round r of this wave into register slot SLOT (r beyond the wave's share reads zeros)
    auto request = [&](auto slotc, int r) {
        constexpr int SLOT = decltype(slotc)::value;
        const int kr = kb + (wave + SS_WAVES * r) * SS_ROUND;
        const bool live = r < my_rounds;
        const char* bb = (const char*)(Bm + (long long)kr * b_rs + n0);
        const char* ab = (const char*)(Am + kr);
        __amdgpu_buffer_rsrc_t b_rsrc = m16_rsrc(bb, live ? (long long)(b_end - bb) : 0);
        __amdgpu_buffer_rsrc_t a_rsrc = m16_rsrc(ab, live ? (long long)(a_end - ab) : 0);
#pragma unroll
        for (int e = 0; e < 8; e++) raw[SLOT][e] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)b_off[e], 0, 2);
        araw[SLOT] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)((kr + 8 * h < g.k) ? a_off : M16_OOB), 0, 0);
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

    // ---- the block's waves add their tiles through LDS, 8 rows per pass ----
    // accumulator register v of a 32x32 tile holds row 8*(v/4) + 4*h + v%4 at column j (of residue c)
    T* C = (T*)g.C;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    const __amdgpu_buffer_rsrc_t part_rsrc = m16_rsrc(partials, partials ? (long long)nsplit * g.m * g.n * 4 : 0);
#pragma unroll
    for (int p = 0; p < MT / 8; p++) {
        if (8 * p >= g.m) break;
        __syncthreads();
#pragma unroll
        for (int vv = 0; vv < 4; vv++) {
            float* dst = red + (wave * 8 + 4 * h + vv) * SS_RED_PITCH + 8 * j;
            *(f32x4_t*)dst = f32x4_t{acc[0][4 * p + vv], acc[1][4 * p + vv], acc[2][4 * p + vv], acc[3][4 * p + vv]};
            *(f32x4_t*)(dst + 4) = f32x4_t{acc[4][4 * p + vv], acc[5][4 * p + vv], acc[6][4 * p + vv], acc[7][4 * p + vv]};
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int idx = threadIdx.x + 256 * i, r = idx / 64, c4 = (idx % 64) * 4;
            const int gm = 8 * p + r, gn = n0 + c4;
            if (gm >= g.m || gn >= g.n) continue;                        // n is a multiple of 4, so a quad is wholly in or out
            f32x4_t sum = *(const f32x4_t*)(red + r * SS_RED_PITCH + c4);
#pragma unroll
            for (int w = 1; w < SS_WAVES; w++) sum += *(const f32x4_t*)(red + (w * 8 + r) * SS_RED_PITCH + c4);
            if (nsplit > 1) {
                const long long at = ((long long)split * g.m + gm) * g.n + gn;
                if (arrivals) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sum), part_rsrc, (int)(at * 4), 0, SPLITK_DEVICE_SCOPE);
                else *(f32x4_t*)(partials + at) = sum;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    T* pc = C + (long long)gm * g.c_rs + (long long)(gn + e) * g.c_cs;
                    T old = accum ? *pc : T{};
                    *pc = finish<T>(sum[e], has_bias, has_bias ? bias[gn + e] : T{}, accum, old);
                }
            }
        }
    }
    if (nsplit == 1 || !arrivals) return;

    // ---- single-launch finish: the last block of this column group to arrive adds all splits ----
    // Partials are written and read at device scope (they bypass the per-XCD L2s, which are not coherent
    // with each other), every thread waits for its own stores to be acknowledged before the block's arrival
    // is counted, and the count is a device-scope atomic.  No cache-wide write-back or invalidate is needed.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        int before = __hip_atomic_fetch_add(arrivals + blockIdx.x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        arrived_last = before == nsplit - 1;
    }
    __syncthreads();
    if (!arrived_last) return;
    const long long split_stride = (long long)g.m * g.n;
    constexpr int QPR = SS_COLS / 4;                     // quads per row of the block's columns
    // two quads per thread and pass (one pass covers 8 rows), the loads of eight splits of both in flight together
    for (int r0 = 0; r0 < g.m; r0 += 8) {
        long long at[2];
        bool live[2];
        int row[2], col[2];
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int idx = threadIdx.x + 256 * q;
            row[q] = r0 + idx / QPR; col[q] = n0 + (idx % QPR) * 4;
            live[q] = row[q] < g.m && col[q] < g.n;
            at[q] = live[q] ? ((long long)row[q] * g.n + col[q]) * 4 : (long long)M16_OOB;      // bytes; dead quads read zeros
        }
        f32x4_t sum[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        for (int sp = 0; sp < nsplit; sp += 8) {
            u32x4_t v[2][8];
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    const bool in = live[q] && sp + u < nsplit;
                    v[q][u] = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, in ? (int)(at[q] + (sp + u) * split_stride * 4) : (int)M16_OOB, 0, SPLITK_DEVICE_SCOPE);
                }
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int q = 0; q < 2; q++) sum[q] += __builtin_bit_cast(f32x4_t, v[q][u]);       // split order; absent splits add +0
        }
#pragma unroll
        for (int q = 0; q < 2; q++) {
            if (!live[q]) continue;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                T* pc = C + (long long)row[q] * g.c_rs + (long long)(col[q] + e) * g.c_cs;
                T old = accum ? *pc : T{};
                *pc = finish<T>(sum[q][e], has_bias, has_bias ? bias[col[q] + e] : T{}, accum, old);
            }
        }
    }
    if (threadIdx.x == 0) __hip_atomic_store(arrivals + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
}

template <typename T>
static int launch_stream16_t(const GemmArgs& g, float* partials, int nsplit, int k_per_split, int* arrivals) {
    dim3 grid((g.n + SS_COLS - 1) / SS_COLS, nsplit);
    if (g.m <= 8) hipLaunchKernelGGL((gemm_stream16_kernel<T, 8>), grid, dim3(256), 0, current_stream(), g, partials, k_per_split, arrivals);
    else          hipLaunchKernelGGL((gemm_stream16_kernel<T, 16>), grid, dim3(256), 0, current_stream(), g, partials, k_per_split, arrivals);
    return check_launch("gemm_stream16_kernel") ? 0 : -1;
}

static int launch_stream16(const GemmArgs& g, int dtype) {
    const int groups = (g.n + SS_COLS - 1) / SS_COLS;
    constexpr int QUANTUM = SS_WAVES * SS_ROUND;             // k rows one pass of a block's waves covers
    // one block per CU (a wave per SIMD, its registers holding the rounds in flight), each at least four passes deep
    int nsplit = (256 + groups - 1) / groups;
    int max_split = g.k / (4 * QUANTUM) > 0 ? g.k / (4 * QUANTUM) : 1;
    if (nsplit > max_split) nsplit = max_split;
    int k_per_split = ((g.k + nsplit - 1) / nsplit + QUANTUM - 1) / QUANTUM * QUANTUM;
    nsplit = (g.k + k_per_split - 1) / k_per_split;
    const size_t part_bytes = (size_t)nsplit * g.m * g.n * sizeof(float);
    void* ws = nullptr;
    if (nsplit > 1 && gemm_workspace(&ws, part_bytes) != 0) return -1;
    int* arrivals = nullptr;
    if (nsplit > 1) {
        bool failed = false;
        arrivals = splitk_arrival_counters(groups, part_bytes, &failed);
        if (failed) { gemm_workspace_release(ws); return -1; }
    }
    int rc;
    if (dtype == RP_DTYPE_BFLOAT16) rc = launch_stream16_t<bf16_t>(g, (float*)ws, nsplit, k_per_split, arrivals);
    else rc = launch_stream16_t<f16_t>(g, (float*)ws, nsplit, k_per_split, arrivals);
    if (rc == 0 && nsplit > 1 && !arrivals) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, dtype);
    if (ws) gemm_workspace_release(ws);          // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

static bool tiled_skinny_forced() {          // RP_HIP_SKINNY_TILED=1: measure the tiled kernel on shapes the streaming one takes
    static int v = -1;
    if (v < 0) { const char* e = getenv("RP_HIP_SKINNY_TILED"); v = (e && e[0] == '1') ? 1 : 0; }
    return v == 1;
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
    // beyond 16 rows the partial tiles the streaming kernel exchanges outweigh what it saves
    if (!p.a_mc && p.b_mc && g.m <= SS_MAX_M && !tiled_skinny_forced()) return launch_stream16(g, dtype);
    constexpr int BN = 128;
    const int tiles = ((g.n + BN - 1) / BN) * ((g.m + 31) / 32);
    // about three blocks per CU in flight, each split at least four slabs deep
    int nsplit = (768 + tiles - 1) / tiles;
    int max_split = g.k / (4 * M16_BK) > 0 ? g.k / (4 * M16_BK) : 1;
    if (nsplit > max_split) nsplit = max_split;
    int k_per_split = ((g.k + nsplit - 1) / nsplit + M16_BK - 1) / M16_BK * M16_BK;
    nsplit = (g.k + k_per_split - 1) / k_per_split;
    void* ws = nullptr;
    if (gemm_workspace(&ws, (size_t)nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
    int rc;
    if (dtype == RP_DTYPE_BFLOAT16) rc = launch_skinny16_t<bf16_t>(g, p, (float*)ws, nsplit, k_per_split);
    else rc = launch_skinny16_t<f16_t>(g, p, (float*)ws, nsplit, k_per_split);
    if (rc == 0) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, dtype);
    gemm_workspace_release(ws);          // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

}  // namespace rp
