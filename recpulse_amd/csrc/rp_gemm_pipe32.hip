// fp32 GEMM with a short reduction (k <= 64), e.g. S = Q.K^T per head (both operands contiguous along k); operands with
// unit stride along their free index are taken as well.
//
// Such a product writes far more than it reads (512 x 512 outputs from 2 x 512 x 64 inputs), and per 128 x 128
// tile the 64 KB of stores take about as long as the 128 MFMAs of a wave.  A block that multiplies, then stores,
// then loads leaves the matrix pipe idle for more than half of the time, and a second block on the CU only fills
// part of that.  Here one block of eight waves stays on each CU and walks its tiles with every phase overlapped:
//
//  - waves 4..7 only fetch.  A tile's rows of A and B (256 bytes each, zero-filled past k) go from memory straight
//    into LDS (buffer loads with the LDS bit: no registers, 1 KB per instruction), two tiles of LDS in rotation, so
//    tile t + 1 lands while tile t is multiplied.  A wave instruction fills four consecutive LDS rows; which 16-byte
//    piece of the global row a lane fetches is the piece index XOR the row's low four bits, so that the 16 lanes
//    that later read one piece index of 16 consecutive rows hit 16 different bank groups.
//  - waves 0..3 only multiply and store.  Each owns a 64 x 64 patch (2 x 2 MFMA tiles of v_mfma_f32_32x32x2_f32)
//    and two sets of accumulators: while tile t is accumulated into one set, the other set, tile t - 1, is stored,
//    one store behind every second MFMA.  Lane (r, h) = (lane % 32, lane / 32) reads 16 bytes of its row from LDS
//    for four MFMA steps: step (u, e) pairs k = 8u + e from the lanes with h = 0 and k = 8u + 4 + e from h = 1; A and
//    B use the same pairing, and a sum over k does not care about the order.
//
// The two roles never wait for each other's memory operations: the fetching waves wait for loads only, the
// multiplying waves issue stores only and never wait for them (a wave's loads and stores share one counter, and a
// wait for a load would also wait for every younger store).  One block-wide barrier per tile hands a filled LDS tile
// to the multipliers and an emptied one back.
#include "rp_gemm.h"

#include <type_traits>

namespace rp {

constexpr int P32_BM = 128, P32_BN = 128, P32_MAXK = 64;
constexpr int P32_ROW_BYTES = 256;                                   // one LDS row: 64 floats
constexpr int P32_TILE_BYTES = (P32_BM + P32_BN) * P32_ROW_BYTES;    // 64 KB: A rows, then B rows

typedef __attribute__((address_space(3))) void* p32_lds_t;

// (a bit cast applied directly to one element of a vector reads the wrong element with this compiler: pass the element by value)
__device__ __forceinline__ uint32_t p32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// KCH: 16-byte pieces of k per lane pair that are multiplied (8 for k <= 64, 4 for k <= 32); EDGE: m or n not whole tiles.
// A_MC / B_MC: the operand has unit stride along its free index (m, n) instead of along k: it lies in LDS as 64 k rows of
// 128 free indices (512 bytes) whose 128-byte pieces are XORed with (k row / 4) % 4, so that the two halves of a wave, which
// read k rows four apart, use different banks; its values are read one at a time.
// BIAS: g.bias[n] is added to every row (the lane's two bias values of a tile are loaded while that tile is multiplied,
// one tile before its stores).
template <int KCH, bool A_MC, bool B_MC, bool EDGE, bool BIAS>
__global__ void __launch_bounds__(512) gemm_pipe32_kernel(GemmArgs g, int tiles_m, int tiles_n, unsigned total) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char p32_smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const unsigned per_matrix = (unsigned)(tiles_m * tiles_n);
    unsigned first, walk_end, stride;
    resident_tile_walk(total, first, walk_end, stride);
    total = walk_end;                                               // this workgroup's tiles: first, first + stride, ... below total
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;      // strides of the free index and of k
    const long long a_span = (A_MC ? ((long long)(g.k - 1) * a_ks + g.m) : ((long long)(g.m - 1) * a_fs + g.k)) * 4;
    const long long b_span = (B_MC ? ((long long)(g.k - 1) * b_ks + g.n) : ((long long)(g.n - 1) * b_fs + g.k)) * 4;

    if (wave >= 4) {
        // ---- fetch: this wave brings rows [32p, 32p + 32) (k-contiguous operand) or k rows [16p, 16p + 16) (the other
        // layout) of A and of B for every tile; a wave instruction fills 1 KB of LDS: 4 rows, or 2 k rows ----
        const int p = wave - 4;
        uint32_t a_off[8], b_off[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int row = 4 * q + (lane >> 4);                        // row within the wave's 32
            const int piece = (lane & 15) ^ (row & 15);                 // which 16 bytes of the global row land in this lane's LDS slot
            const int krow = 2 * q + (lane >> 5);                       // k row within the wave's 16
            const int c128 = ((lane & 31) >> 3) ^ ((krow >> 2) & 3);    // which 128 bytes of the global k row (its 16-byte piece: lane & 7)
            const int free = c128 * 32 + (lane & 7) * 4;
            a_off[q] = A_MC ? (16 * p + krow < g.k ? (uint32_t)(((long long)krow * a_ks + free) * 4) : BUFFER_OOB)
                            : (piece * 4 < g.k ? (uint32_t)(((long long)row * a_fs + piece * 4) * 4) : BUFFER_OOB);
            b_off[q] = B_MC ? (16 * p + krow < g.k ? (uint32_t)(((long long)krow * b_ks + free) * 4) : BUFFER_OOB)
                            : (piece * 4 < g.k ? (uint32_t)(((long long)row * b_fs + piece * 4) * 4) : BUFFER_OOB);
        }
        auto fetch = [&](unsigned id, int buf) {
            const TileOrigin t = tile_origin<P32_BM, P32_BN>(id, per_matrix, tiles_n);
            const __amdgpu_buffer_rsrc_t ra = buffer_rsrc((const float*)g.A + (long long)t.z * g.a_bs, a_span);
            const __amdgpu_buffer_rsrc_t rb = buffer_rsrc((const float*)g.B + (long long)t.z * g.b_bs, b_span);
            const int sa = A_MC ? (int)(((long long)(16 * p) * a_ks + t.m0) * 4) : (int)((long long)(t.m0 + 32 * p) * a_fs * 4);
            const int sb = B_MC ? (int)(((long long)(16 * p) * b_ks + t.n0) * 4) : (int)((long long)(t.n0 + 32 * p) * b_fs * 4);
            // (both layouts put the wave's share at the same place: 32 rows of 256 bytes = 16 k rows of 512 bytes = 8 KB)
            unsigned char* dst = p32_smem + buf * P32_TILE_BYTES + 32 * p * P32_ROW_BYTES;
#pragma unroll
            for (int q = 0; q < 8; q++) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (p32_lds_t)(dst + q * 1024), 16, (int)a_off[q], sa, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (p32_lds_t)(dst + P32_BM * P32_ROW_BYTES + q * 1024), 16, (int)b_off[q], sb, 0, 0);
            }
        };
        if (first < total) fetch(first, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        int buf = 0;
        for (unsigned id = first; id < total; id += stride) {
            if (id + stride < total) fetch(id + stride, buf ^ 1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            buf ^= 1;
        }
        return;
    }

    // ---- multiply and store ----
    const int r = lane & 31, h = lane >> 5;
    const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
    // k-contiguous operand: the LDS byte address of piece 2u + h of this lane's row is lane_x ^ (32 u) (rows are 256-byte
    // aligned, so the XOR only touches the piece bits).  Other layout: the value of step (u, e), k row 8u + 4h + e, free
    // index w0 + 32 i + r, is at mc_x + (8u + e) k rows, in the 128-byte piece (w0 / 32 + i) ^ ((2u + h) % 4).
    const uint32_t lane_a = (uint32_t)((wm0 + r) * P32_ROW_BYTES + ((h ^ (r & 15)) * 16));
    const uint32_t lane_b = (uint32_t)(P32_BM * P32_ROW_BYTES + (wn0 + r) * P32_ROW_BYTES + ((h ^ (r & 15)) * 16));
    const uint32_t mc_a = (uint32_t)(4 * h * 512 + r * 4), mc_b = (uint32_t)(P32_BM * P32_ROW_BYTES + 4 * h * 512 + r * 4);
    const uint32_t c_lane = (uint32_t)(((long long)(4 * h) * g.c_rs + (long long)r * g.c_cs) * 4);
    const long long c_span = ((long long)(g.m - 1) * g.c_rs + (long long)(g.n - 1) * g.c_cs + 1) * 4;

    f32x16_t acc[2][2][2];              // [set][i][j]
    f32x4_t af[2][2], bf[2][2];         // [slot][i or j]: four k values of the lane's row
    float bias_prev[2] = {0.f, 0.f}, bias_cur[2] = {0.f, 0.f};      // BIAS: of columns n0 + wn0 + 32 j + r of the tile being stored / multiplied
    auto load_bias = [&](const TileOrigin& t) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int gn = t.n0 + wn0 + 32 * j + r;
            bias_cur[j] = gn < g.n ? ((const float*)g.bias)[gn] : 0.f;
        }
    };

    // store number n (0..63) of accumulator set SET: register v of MFMA tile (i, j), i.e. columns 32j + r of rows 32i + 8(v / 4) + 4h + v % 4
    auto store_one = [&](auto set_c, auto n_c, const TileOrigin& t, const __amdgpu_buffer_rsrc_t& rc) {
        constexpr int SET = decltype(set_c)::value, n = decltype(n_c)::value;
        constexpr int sj = n >> 5, si = (n >> 4) & 1, v = n & 15;
        constexpr int row = 32 * si + 8 * (v / 4) + (v % 4);
        const int gm = t.m0 + wm0 + row, gn = t.n0 + wn0 + 32 * sj;
        const int soff = (int)(((long long)gm * g.c_rs + (long long)gn * g.c_cs) * 4);
        uint32_t voff = c_lane;
        if constexpr (EDGE) voff = (gm + 4 * h < g.m && gn + r < g.n) ? c_lane : BUFFER_OOB;
        float val = acc[SET][si][sj][v];
        if constexpr (BIAS) val = val + bias_prev[sj];
        __builtin_amdgcn_raw_buffer_store_b32(p32_bits(val), rc, (int)voff, soff, 2);          // (streaming store: the output is not read again by this kernel)
    };

    auto read_frags = [&](const unsigned char* base, int u, int slot) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if constexpr (!A_MC) {
                af[slot][i] = *(const f32x4_t*)(base + ((lane_a ^ (uint32_t)(32 * u)) + i * 32 * P32_ROW_BYTES));
            } else {
                const uint32_t at = mc_a + (uint32_t)(8 * u * 512) + ((((uint32_t)(wm0 >> 5) + i) ^ (uint32_t)((2 * u + h) & 3)) * 128);
#pragma unroll
                for (int e = 0; e < 4; e++) af[slot][i][e] = *(const float*)(base + at + e * 512);
            }
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if constexpr (!B_MC) {
                bf[slot][j] = *(const f32x4_t*)(base + ((lane_b ^ (uint32_t)(32 * u)) + j * 32 * P32_ROW_BYTES));
            } else {
                const uint32_t at = mc_b + (uint32_t)(8 * u * 512) + ((((uint32_t)(wn0 >> 5) + j) ^ (uint32_t)((2 * u + h) & 3)) * 128);
#pragma unroll
                for (int e = 0; e < 4; e++) bf[slot][j][e] = *(const float*)(base + at + e * 512);
            }
        }
    };

    // One tile: accumulate into set CUR from LDS tile `buf` (whose first pieces are already in fragment slot 0); if STORE,
    // write set CUR ^ 1 (the tile `prev`) meanwhile.  The block's barrier sits before the last piece's MFMAs, when every
    // LDS read of this tile has returned: behind it the other LDS tile holds the next tile, whose first pieces are read
    // under those MFMAs, and the fetching waves may overwrite this one.
    auto tile_pass = [&](auto cur_c, auto store_c, int buf, const TileOrigin& prev) {
        constexpr int CUR = decltype(cur_c)::value;
        constexpr bool STORE = decltype(store_c)::value;
        const unsigned char* base = p32_smem + buf * P32_TILE_BYTES;
        const unsigned char* next_base = p32_smem + (buf ^ 1) * P32_TILE_BYTES;
        const __amdgpu_buffer_rsrc_t rc = buffer_rsrc((float*)g.C + (long long)prev.z * g.c_bs, c_span);
        static_for<0, KCH>([&](auto uc) {
            constexpr int u = decltype(uc)::value, slot = u & 1;
            if constexpr (u + 1 < KCH) {
                read_frags(base, u + 1, slot ^ 1);
            } else {
                __syncthreads();
                read_frags(next_base, 0, slot ^ 1);
            }
            static_for<0, 16>([&](auto sc) {
                constexpr int s = decltype(sc)::value, e = s >> 2, i = (s >> 1) & 1, j = s & 1;
                if constexpr (u == 0 && e == 0) {
                    const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    acc[CUR][i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[slot][i][e], bf[slot][j][e], zero, 0, 0, 0);
                } else {
                    acc[CUR][i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[slot][i][e], bf[slot][j][e], acc[CUR][i][j], 0, 0, 0);
                }
                if constexpr (STORE) {
                    // 64 stores over 16 * KCH MFMAs
                    constexpr int PER = 64 / KCH;                        // stores per u: 8 or 16
                    constexpr int EVERY = 16 / PER;                      // an MFMA in every EVERY carries one
                    if constexpr (s % EVERY == EVERY - 1) store_one(std::integral_constant<int, CUR ^ 1>{}, std::integral_constant<int, u * PER + s / EVERY>{}, prev, rc);
                    if constexpr (s % 2 == 1) __builtin_amdgcn_sched_barrier(0);
                }
            });
        });
    };

    __syncthreads();                                   // the first tile is in LDS
    TileOrigin prev = {0, 0, 0};
    int buf = 0, last = 0;
    unsigned id = first;
    if (id >= total) return;
    read_frags(p32_smem, 0, 0);
    if constexpr (BIAS) load_bias(tile_origin<P32_BM, P32_BN>(id, per_matrix, tiles_n));
    tile_pass(std::integral_constant<int, 0>{}, std::false_type{}, buf, prev);
    prev = tile_origin<P32_BM, P32_BN>(id, per_matrix, tiles_n);
    if constexpr (BIAS) { bias_prev[0] = bias_cur[0]; bias_prev[1] = bias_cur[1]; }
    buf ^= 1;
    id += stride;
    // two tiles per round, so that the accumulator sets are fixed registers
    while (id < total) {
        if constexpr (BIAS) load_bias(tile_origin<P32_BM, P32_BN>(id, per_matrix, tiles_n));
        tile_pass(std::integral_constant<int, 1>{}, std::true_type{}, buf, prev);
        prev = tile_origin<P32_BM, P32_BN>(id, per_matrix, tiles_n);
        if constexpr (BIAS) { bias_prev[0] = bias_cur[0]; bias_prev[1] = bias_cur[1]; }
        buf ^= 1;
        id += stride;
        last = 1;
        if (id >= total) break;
        if constexpr (BIAS) load_bias(tile_origin<P32_BM, P32_BN>(id, per_matrix, tiles_n));
        tile_pass(std::integral_constant<int, 0>{}, std::true_type{}, buf, prev);
        prev = tile_origin<P32_BM, P32_BN>(id, per_matrix, tiles_n);
        if constexpr (BIAS) { bias_prev[0] = bias_cur[0]; bias_prev[1] = bias_cur[1]; }
        buf ^= 1;
        id += stride;
        last = 0;
    }
    // the last tile's accumulators
    const __amdgpu_buffer_rsrc_t rc = buffer_rsrc((float*)g.C + (long long)prev.z * g.c_bs, c_span);
    if (last == 0) static_for<0, 64>([&](auto nc) { store_one(std::integral_constant<int, 0>{}, nc, prev, rc); });
    else static_for<0, 64>([&](auto nc) { store_one(std::integral_constant<int, 1>{}, nc, prev, rc); });
}

// ---- host side ----

// Whether this kernel takes the product: fp32, k <= 64 in whole 16-byte pieces, both operands with a unit stride and
// 16-byte aligned rows, C overwritten (a bias per column is taken; no accumulation, whose extra read of C leaves the
// product bound by memory at the tiled kernel's speed; no segments or folded store), and every byte offset the kernel
// forms from a batch entry's base within the 32-bit range of buffer addressing.
bool pipe32_takes(const GemmArgs& g) {
    if (g.k > P32_MAXK || g.k < 4 || g.k % 4 || g.m < 1 || g.n < 1 || g.batch < 1) return false;
    if ((long long)((g.m + P32_BM - 1) / P32_BM) * ((g.n + P32_BN - 1) / P32_BN) * g.batch >= (1ll << 30)) return false;
    if (g.accumulate || g.seg_k || g.seg_n || g.c_fold_from || g.bias_by_row || ((uintptr_t)g.bias & 3)) return false;
    const bool a_kc = g.a_cs == 1 && g.a_rs % 4 == 0, a_mc = g.a_rs == 1 && g.a_cs % 4 == 0;
    const bool b_kc = g.b_rs == 1 && g.b_cs % 4 == 0, b_mc = g.b_cs == 1 && g.b_rs % 4 == 0;
    if (!(a_kc || a_mc) || !(b_kc || b_mc) || g.a_bs % 4 || g.b_bs % 4 || g.a_rs < 0 || g.a_cs < 0 || g.b_rs < 0 || g.b_cs < 0 || g.c_rs < 0 || g.c_cs < 0) return false;
    if (((uintptr_t)g.A & 15) || ((uintptr_t)g.B & 15) || ((uintptr_t)g.C & 3)) return false;
    const long long lim = 1ll << 30;
    // free indices up to a whole tile past the last one are addressed (and read as zero, or as values that only reach
    // outputs which are not stored)
    const long long a_reach = (a_kc ? (long long)(g.m + P32_BM) * g.a_rs + P32_MAXK : (long long)P32_MAXK * g.a_cs + g.m + P32_BM) * 4;
    const long long b_reach = (b_kc ? (long long)(g.n + P32_BN) * g.b_cs + P32_MAXK : (long long)P32_MAXK * g.b_rs + g.n + P32_BN) * 4;
    const long long c_reach = ((long long)(g.m + P32_BM) * g.c_rs + (long long)(g.n + P32_BN) * g.c_cs) * 4;
    return a_reach < lim && b_reach < lim && c_reach < lim;
}

int launch_pipe32(const GemmArgs& g) {
    const int tiles_m = (g.m + P32_BM - 1) / P32_BM, tiles_n = (g.n + P32_BN - 1) / P32_BN;
    const long long total = (long long)tiles_m * tiles_n * g.batch;
    int cus = device_cu_count();
    if (cus <= 0) cus = 256;
    const unsigned blocks = (unsigned)(total < cus ? total : cus);          // one resident workgroup per CU walks its tiles
    const bool edge = (g.m % P32_BM) || (g.n % P32_BN);
    constexpr int smem = 2 * P32_TILE_BYTES;
    auto launch = [&](auto kern) {
        if (!check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem), "hipFuncSetAttribute")) return -1;
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(512), smem, current_stream(), g, tiles_m, tiles_n, (unsigned)total);
        return check_launch("gemm_pipe32_kernel") ? 0 : -1;
    };
    const bool a_mc = !(g.a_cs == 1 && g.a_rs % 4 == 0), b_mc = !(g.b_rs == 1 && g.b_cs % 4 == 0);
    auto pick = [&](auto kch_c, auto bias_c) {
        constexpr int KCH = decltype(kch_c)::value;
        constexpr bool BIAS = decltype(bias_c)::value;
        if (!a_mc && !b_mc) return edge ? launch(gemm_pipe32_kernel<KCH, false, false, true, BIAS>) : launch(gemm_pipe32_kernel<KCH, false, false, false, BIAS>);
        if (!a_mc && b_mc) return edge ? launch(gemm_pipe32_kernel<KCH, false, true, true, BIAS>) : launch(gemm_pipe32_kernel<KCH, false, true, false, BIAS>);
        if (a_mc && !b_mc) return edge ? launch(gemm_pipe32_kernel<KCH, true, false, true, BIAS>) : launch(gemm_pipe32_kernel<KCH, true, false, false, BIAS>);
        return edge ? launch(gemm_pipe32_kernel<KCH, true, true, true, BIAS>) : launch(gemm_pipe32_kernel<KCH, true, true, false, BIAS>);
    };
    if (g.k <= 32) return g.bias ? pick(std::integral_constant<int, 4>{}, std::true_type{}) : pick(std::integral_constant<int, 4>{}, std::false_type{});
    return g.bias ? pick(std::integral_constant<int, 8>{}, std::true_type{}) : pick(std::integral_constant<int, 8>{}, std::false_type{});
}

}  // namespace rp
