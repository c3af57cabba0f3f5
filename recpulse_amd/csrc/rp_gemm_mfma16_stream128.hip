// bf16 / fp16 GEMMs with at most 32 rows, row-major A and B, deep k: the streaming kernel (128-column strips).
#include "rp_gemm_mfma16_kernel.h"
#include "rp_gemm_splitk_finish.h"

namespace rp {

// ============================================================================
// B goes from memory to registers to the MFMAs without touching LDS.  One wave
// owns 128 adjacent columns of B (256 bytes of a row) and a set of "rounds" of
// k; the four waves of a workgroup share the columns and split k, and so do the
// workgroups of a column group, so that one workgroup per CU streams B.
//
// Rounds are dealt cyclically: round r of k belongs to split r % nsplit, and
// inside a block to wave (r / nsplit) % 4.  At any moment the grid as a whole
// therefore reads one contiguous window of B (nsplit * 4 rounds of whole rows),
// which the memory system serves 5 - 8 % faster than the same blocks each
// walking a range of k of its own (the ranges lie a power of two apart).  Loads
// are issued unconditionally (out-of-range rounds get an empty buffer
// descriptor and read zeros), so the waits the compiler inserts count loads
// exactly.
//
// The block's 4 waves add their tiles through LDS in wave order and the block
// writes one fp32 partial (or, without a k split, the finished output).  With
// `arrivals` the block then counts itself in, and the last block of its column
// group to do so adds the group's partials in split order and writes the output
// (otherwise a second kernel does).  Strips of 128 columns rather than wider
// ones keep that finish small: with one workgroup per CU an 8192-column output
// takes 4 splits, and the finishing block reads 4 x m rows of 512 bytes.
//
// Placement.  The grid is one-dimensional and block b stands for (XCD x = b % 8,
// slot b / 8): workgroups are dealt to the XCDs round robin, so all splits of
// column group 8i + x are given slots of XCD x.  When the host has verified that
// rule on the device (`local`), the partials and the arrival count never leave
// that XCD's L2: plain stores (complete when the L2 has them), an atomic that the
// L2 executes, and plain loads (the finishing CU's vector cache holds none of
// them yet).  Otherwise they are exchanged at device scope (written through to
// memory and read back from there), which costs about 1.5 us more per launch.
//
// A round is 32 rows of k, loaded in two steps of 16 and multiplied by one
// v_mfma_f32_16x16x32 per 16 x 16 output tile.  In that instruction lane
// (q, j) = (lane / 16, lane % 16) supplies the eight k values 8q .. 8q+7 of row j
// (A) or column j (B).  For A that is one 16-byte load per lane and round: the
// four q lanes of a row read 64 contiguous bytes of the row's cache line.  (With
// 16-row rounds and v_mfma_f32_16x16x16, lane (q, j) fetches 8 bytes out of each
// row's line per step; these are L2 hits, but at 16 rows they cost 1.3 us per
// launch.  64-row rounds read A in whole lines but deal k to the waves in
// coarser pieces, which B's stream likes less: 0.3 us longer at every m.  Two
// 16x16x16 per tile and round instead of one 16x16x32 cost 0.1 - 0.2 us.)
// For B, step t reads rows 8q + 4t + e (e = 0 .. 3): lane (q, j) loads 16 bytes
// (columns 8j .. 8j+7) of each, a load instruction covers four 256-byte row
// segments 8 rows apart, and the 4 x 8 block of 16-bit values a lane holds is
// transposed in registers (byte permutes) into 8 half operands, one per column
// residue c: residue c carries column 8j + c.  The first step's halves wait in
// registers for the second's; MFMA (f, c) accumulates the 16 x 16 tile of rows
// 16f .. 16f+15 and columns {8j + c}.
//
// 256-byte strips stream at the full rate only with about 8 KB of loads in
// flight per wave (a read-only probe: 19.5 - 20.2 us for 134 MB with two steps
// in flight, 23.6 with one, 21.6 with three), so a wave keeps two steps of 4 KB
// in flight, across round boundaries.  A's registers alternate between two sets
// by round; a set is refilled for the round after next as soon as its last step
// has copied its operands out.  The loop body is a pair of rounds, so that
// register sets and slots are compile-time choices and nothing is copied at the
// back edge.
// ============================================================================
constexpr int S8_WAVES = 4, S8_COLS = 128, S8_STEP = 16, S8_PITCH = S8_COLS + 8;
constexpr int S8_MAX_M = 32;
constexpr int S8_RS = 2;                // steps per round: 32 rows of k, one v_mfma_f32_16x16x32 per tile

template <typename T> struct s8_ops;
template <> struct s8_ops<bf16_t> {
    static __device__ __forceinline__ f32x4_t mma32(u32x4_t a, u32x4_t b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};
template <> struct s8_ops<f16_t> {
    static __device__ __forceinline__ f32x4_t mma32(u32x4_t a, u32x4_t b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};

template <typename T, int MR>
__global__ void __launch_bounds__(256) gemm_stream128_kernel(GemmArgs g, float* partials, int groups, int nsplit, int* arrivals, int local) {
    constexpr int NF = MR / 16;                                           // A fragments (16 rows each)
    constexpr int RS = S8_RS, S8_ROUND = S8_STEP * RS;                    // steps and k rows of a round
    extern __shared__ __attribute__((aligned(16))) float red[];          // [S8_WAVES][MR][S8_PITCH]
    __shared__ bool arrived_last;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);       // scalar, so that buffer descriptors built from it are too
    const int q = lane >> 4, j = lane & 15;
    // block b stands for (XCD b % 8, slot b / 8): all splits of column group 8i + x run on XCD x
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int group = (slot / nsplit) * 8 + xcd, split = slot % nsplit;
    if (group >= groups) return;                                           // (whole blocks, before any barrier)
    const int n0 = group * S8_COLS;
    // rounds are dealt cyclically: round r of k belongs to split r % nsplit and, inside the block, to wave (r / nsplit) % 4
    const int total_rounds = (g.k + S8_ROUND - 1) / S8_ROUND;
    const int mine = total_rounds > split ? (total_rounds - split + nsplit - 1) / nsplit : 0;      // rounds of this block
    const int my_rounds = mine > wave ? (mine - wave + S8_WAVES - 1) / S8_WAVES : 0;               // and of this wave

    const uint16_t* Bm = (const uint16_t*)g.B;
    const uint16_t* Am = (const uint16_t*)g.A;
    const long long b_rs = g.b_rs, a_rs = g.a_rs;
    const char* b_end = (const char*)(Bm + ((long long)(g.k - 1) * b_rs + g.n));
    const char* a_end = (const char*)(Am + ((long long)(g.m - 1) * a_rs + g.k));
    const int b_step = (int)(4 * b_rs * 2);                               // bytes from a step's rows to the next step's

    uint32_t b_off[4], a_off[NF];
#pragma unroll
    for (int e = 0; e < 4; e++)
        b_off[e] = (n0 + 8 * j < g.n) ? (uint32_t)(((long long)(4 * RS * q + e) * b_rs + 8 * j) * 2) : BUFFER_OOB;      // (n is a multiple of 8)
#pragma unroll
    for (int f = 0; f < NF; f++)
        a_off[f] = (16 * f + j < g.m) ? (uint32_t)(((long long)(16 * f + j) * a_rs + 4 * RS * q) * 2) : BUFFER_OOB;
    auto round_k = [&](int r) { return ((r * S8_WAVES + wave) * nsplit + split) * S8_ROUND; };

    u32x4_t raw[2][4];                 // two steps of B in flight
    uint32_t a_buf[2][NF][2 * RS];     // a lane's 4 * RS k values of a round, per fragment; rounds alternate between the two sets
    // request step t of round r of this wave into register slot SLOT (rounds beyond the wave's share read zeros)
    auto request_b = [&](auto slotc, int r, int t) {
        constexpr int SLOT = decltype(slotc)::value;
        const int kr = round_k(r);
        const char* bb = (const char*)(Bm + (long long)kr * b_rs + n0);
        __amdgpu_buffer_rsrc_t b_rsrc = buffer_rsrc(bb, r < my_rounds ? (long long)(b_end - bb) : 0);
#pragma unroll
        for (int e = 0; e < 4; e++) raw[SLOT][e] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)b_off[e], t * b_step, 2);       // (streamed: read once)
    };
    auto request_a = [&](auto parc, int r) {
        uint32_t (&dst)[NF][2 * RS] = a_buf[decltype(parc)::value];
        const int kr = round_k(r);
        const char* ab = (const char*)(Am + kr);
        __amdgpu_buffer_rsrc_t a_rsrc = buffer_rsrc(ab, r < my_rounds ? (long long)(a_end - ab) : 0);
#pragma unroll
        for (int f = 0; f < NF; f++) {
            // (k is a multiple of 8 and the lane's piece starts at a multiple of 8: wholly in or out)
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)((kr + 8 * q < g.k) ? a_off[f] : BUFFER_OOB), 0, 0);
            dst[f][0] = v[0]; dst[f][1] = v[1]; dst[f][2] = v[2]; dst[f][3] = v[3];
        }
    };

    f32x4_t acc[NF][8];
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int c = 0; c < 8; c++) acc[f][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Step S of a pair of rounds (S = 0 .. 3: round r0 + S / 2, its step S % 2): transpose it out of slot S % 2, refill
    // the slot with the step two ahead and, at a round's second step, multiply the round and refill its A registers
    // with the round two ahead.
    u32x2_t held[8];                   // the first step's halves of the B operands of the round being multiplied
    auto consume = [&](auto sc, int r0) {
        constexpr int S = decltype(sc)::value, SLOT = S & 1, PAR = S / RS, T_ = S % RS;
        // in-register 4 x 8 transpose of 16-bit values: operand c, dword d = (k row 2d, k row 2d+1) of column c
        u32x2_t opb[8];
#pragma unroll
        for (int c = 0; c < 8; c++)
#pragma unroll
            for (int d = 0; d < 2; d++)
                opb[c][d] = __builtin_amdgcn_perm(raw[SLOT][2 * d + 1][c / 2], raw[SLOT][2 * d][c / 2], (c & 1) ? 0x07060302u : 0x05040100u);
        // A round of 32 k is one v_mfma_f32_16x16x32 per tile: lane (q, j) supplies k = 8q .. 8q+7, which is its A load as
        // it stands and, for B, the first step's half followed by the second's.  The first step only transposes (its
        // halves wait in `held`), the second multiplies.  Either way the operands must exist before the slot is
        // refilled: then the refill can land in the very registers the slot occupies and nothing has to be copied
        // (behind a full wait) at the loop's back edge.
        if constexpr (T_ == 0) {
#pragma unroll
            for (int c = 0; c < 8; c++) { held[c] = opb[c]; asm volatile("" : "+v"(held[c]) : : "memory"); }
            __builtin_amdgcn_sched_barrier(0);
            request_b(std::integral_constant<int, SLOT>{}, r0 + (S + 2) / RS, (S + 2) % RS);
            __builtin_amdgcn_sched_barrier(0);
        } else {
            // (A's operand is moved to registers of its own, so that the refill below can land in the registers it came from)
            u32x4_t opa[NF];
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int d = 0; d < 4; d++) asm volatile("v_mov_b32 %0, %1" : "=v"(opa[f][d]) : "v"(a_buf[PAR][f][d]));
#pragma unroll
            for (int c = 0; c < 8; c++) asm volatile("" : "+v"(opb[c]) : : "memory");
            __builtin_amdgcn_sched_barrier(0);
            request_b(std::integral_constant<int, SLOT>{}, r0 + (S + 2) / RS, (S + 2) % RS);
            request_a(std::integral_constant<int, PAR>{}, r0 + PAR + 2);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int c = 0; c < 8; c++) acc[f][c] = s8_ops<T>::mma32(opa[f], u32x4_t{held[c][0], held[c][1], opb[c][0], opb[c][1]}, acc[f][c]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // (requests stay in program order: the wait for a register counts the loads issued after its own)
    request_a(std::integral_constant<int, 0>{}, 0);
    request_a(std::integral_constant<int, 1>{}, 1);
    request_b(std::integral_constant<int, 0>{}, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    request_b(std::integral_constant<int, 1>{}, 1 / RS, 1 % RS);
    __builtin_amdgcn_sched_barrier(0);
    for (int r0 = 0; r0 < my_rounds; r0 += 2)
        static_for<0, 2 * RS>([&](auto sc) { consume(sc, r0); });

    // ---- the block's waves add their tiles through LDS ----
    // accumulator register v of tile (f, c) holds row 16f + 4q + v at column 8j + c: a lane's 8 residues of one row are
    // 8 adjacent columns, two 16-byte stores at consecutive addresses across the lanes of a row
    const SplitkOutput<T> out(g);
    const __amdgpu_buffer_rsrc_t part_rsrc = buffer_rsrc(partials, partials ? (long long)nsplit * g.m * g.n * 4 : 0);
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int r = 16 * f + 4 * q + v;
            if (r >= g.m) continue;
            float* dst = red + (wave * MR + r) * S8_PITCH + 8 * j;
            *(f32x4_t*)dst = f32x4_t{acc[f][0][v], acc[f][1][v], acc[f][2][v], acc[f][3][v]};
            *(f32x4_t*)(dst + 4) = f32x4_t{acc[f][4][v], acc[f][5][v], acc[f][6][v], acc[f][7][v]};
        }
    __syncthreads();
    // (all sums first, then the stores back to back with the kind of store chosen once: with the choice inside the loop
    // the compiler waits for each store's acknowledgement before the next quad's LDS reads)
    constexpr int QPR = S8_COLS / 4, NQ = MR / 8;        // quads per row of the block's columns, quads per thread
    f32x4_t sum[NQ];
    int qrow[NQ], qcol[NQ];
    bool qlive[NQ];
#pragma unroll
    for (int i = 0; i < NQ; i++) {
        const int idx = threadIdx.x + 256 * i;
        qrow[i] = idx / QPR; qcol[i] = n0 + (idx % QPR) * 4;
        qlive[i] = qrow[i] < g.m && qcol[i] < g.n;                       // n is a multiple of 4, so a quad is wholly in or out
        const int at_lds = qrow[i] * S8_PITCH + (idx % QPR) * 4;        // (rows from m to MR hold nothing and are not stored)
        sum[i] = *(const f32x4_t*)(red + at_lds);
#pragma unroll
        for (int w = 1; w < S8_WAVES; w++) sum[i] += *(const f32x4_t*)(red + w * MR * S8_PITCH + at_lds);
    }
    if (nsplit == 1) { out.store_quads(qrow, qcol, qlive, sum); return; }
    if (!arrivals) {
#pragma unroll
        for (int i = 0; i < NQ; i++)
            if (qlive[i]) *(f32x4_t*)(partials + ((long long)split * g.m + qrow[i]) * g.n + qcol[i]) = sum[i];
        return;
    }
    int part_off[NQ];                                    // (dead quads: an offset beyond the buffer, the store is dropped)
#pragma unroll
    for (int i = 0; i < NQ; i++) part_off[i] = qlive[i] ? (int)((((long long)split * g.m + qrow[i]) * g.n + qcol[i]) * 4) : (int)BUFFER_OOB;
    if (local) {
#pragma unroll
        for (int i = 0; i < NQ; i++) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sum[i]), part_rsrc, part_off[i], 0, 0);
    } else {
#pragma unroll
        for (int i = 0; i < NQ; i++) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, sum[i]), part_rsrc, part_off[i], 0, SPLITK_DEVICE_SCOPE);
    }

    // ---- single-launch finish: the last block of this column group to arrive adds all splits ----
    if (!splitk_arrive(arrivals + group, nsplit, local != 0, &arrived_last)) return;
    splitk_finish_window<T, S8_COLS, MR / 8, 4>(g, out, part_rsrc, nsplit, 0, g.m, n0, local != 0, arrivals + group);
}

template <typename T, int MR>
static int launch_stream128_mr(const GemmArgs& g, float* partials, int groups, int nsplit, int* arrivals, int local) {
    constexpr size_t smem = (size_t)S8_WAVES * MR * S8_PITCH * sizeof(float);
    auto kern = gemm_stream128_kernel<T, MR>;
    if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
    hipLaunchKernelGGL(kern, dim3(8 * ((groups + 7) / 8) * nsplit), dim3(256), smem, current_stream(), g, partials, groups, nsplit, arrivals, local);
    return check_launch("gemm_stream128_kernel") ? 0 : -1;
}

template <typename T>
static int launch_stream128_t(const GemmArgs& g, float* partials, int groups, int nsplit, int* arrivals, int local) {
    if (g.m <= 16) return launch_stream128_mr<T, 16>(g, partials, groups, nsplit, arrivals, local);
    return launch_stream128_mr<T, 32>(g, partials, groups, nsplit, arrivals, local);
}

// k splits for an output of n columns: one block per CU (a wave per SIMD), each at least two passes of its waves deep
static int stream128_nsplit(int k, int n) {
    const int groups = (n + S8_COLS - 1) / S8_COLS;
    constexpr int QUANTUM = S8_WAVES * S8_STEP * S8_RS;      // k rows one pass of a block's waves covers
    const int cus = device_cu_count() >= 8 ? device_cu_count() / 8 * 8 : 256;
    const int nsplit = (cus + groups - 1) / groups;
    const int max_split = k / (2 * QUANTUM) > 0 ? k / (2 * QUANTUM) : 1;
    return nsplit < max_split ? nsplit : max_split;
}

// Shapes the kernel is the right one for.  A narrow output with a deep k would need many splits, and the one block
// that finishes a column group reads nsplit x m rows of 512 bytes: beyond 256 such rows the tiled kernel with its
// separate combine launch is faster (32 x 8192 x 2048: 16.1 us here against 14.1).  So it is for a B under 32 MB that
// needs more than 8 splits, where two short launches beat one launch with a finish chain (16 x 4096 x 2048: 10.4 us
// here against 8.5; 2 x 8192 x 1024: 10.9 against 8.4).
bool stream128_shape(int batch, int m, int k, int n) {
    if (batch != 1 || m > S8_MAX_M || n % 8 || k % 8 || path_disabled("stream128")) return false;
    const int nsplit = stream128_nsplit(k, n);
    return (long long)nsplit * m <= 256 && (nsplit <= 8 || (long long)k * n >= (1ll << 24));
}

bool stream128_takes(const GemmArgs& g) { return g.a_cs == 1 && g.b_cs == 1 && stream128_shape(g.batch, g.m, g.k, g.n); }

int launch_stream128(const GemmArgs& g, int dtype) {
    const int groups = (g.n + S8_COLS - 1) / S8_COLS;
    const int nsplit = stream128_nsplit(g.k, g.n);
    const size_t part_bytes = (size_t)nsplit * g.m * g.n * sizeof(float);
    void* ws = nullptr;
    if (nsplit > 1 && gemm_workspace(&ws, part_bytes) != 0) return -1;
    int* arrivals = nullptr;
    if (nsplit > 1) {
        bool failed = false;
        arrivals = splitk_arrival_counters(groups, part_bytes, &failed);
        if (failed) { gemm_workspace_release(ws); return -1; }
    }
    const int local = arrivals && workgroups_share_xcd_by_residue() ? 1 : 0;
    int rc;
    if (dtype == RP_DTYPE_BFLOAT16) rc = launch_stream128_t<bf16_t>(g, (float*)ws, groups, nsplit, arrivals, local);
    else rc = launch_stream128_t<f16_t>(g, (float*)ws, groups, nsplit, arrivals, local);
    if (rc == 0 && nsplit > 1 && !arrivals) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, dtype);
    if (ws) gemm_workspace_release(ws);          // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

}  // namespace rp
