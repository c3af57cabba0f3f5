// fp32 GEMM with an output of at most 64 columns and many row tiles, e.g. O = P.V or dV = P^T.dO per head: 128 x 64
// outputs per tile from a 128 x k strip of A.  The fp32 twin of rp_gemm_pipe16k.hip: one block of eight waves stays on
// each CU and walks its tiles, and the unit of the pipeline is the k slab of 32.
//
//  - waves 4..7 only fetch: a slab of A (128 x 32) and of B (32 x 64) goes from memory straight into one of four LDS
//    stages (buffer loads with the LDS bit, 1 KB per instruction, no registers), three slabs ahead of the multipliers.
//    Operands with unit stride along k lie in LDS as rows of 32 k values (128 bytes) whose 16-byte pieces are XORed with
//    bits 1..3 of the row; operands with unit stride along their free index lie as k rows (A: 512 bytes, B: 256 bytes)
//    whose 128-byte pieces are XORed with bits 2.. of the k row, so that the two halves of a wave, which read k rows
//    four apart, use different banks.
//  - waves 0..3 multiply and store: wave w owns rows 32w .. 32w + 31 of the tile, all 64 columns, as two
//    v_mfma_f32_32x32x2_f32 tiles.  MFMA step (u, e) pairs k = 8u + e from the lanes with h = lane / 32 = 0 and
//    k = 8u + 4 + e from h = 1: a lane's four consecutive k of a k-contiguous operand are one 16-byte LDS read, and a sum
//    over k does not care about the order.  While slab s is multiplied the values of slab s + 1 are read into the
//    registers the MFMAs have just used.  A finished tile is stored straight from the accumulators (register v of a tile
//    is 32 adjacent columns of a row: a 128-byte line): 32 stores against 512 MFMAs.
//
// The fetching waves wait for loads only, the multiplying waves issue stores only; one block-wide barrier per slab says
// "slab s + 1 has landed, and the stage of slab s is free again".
#include "rp_gemm.h"

#include <type_traits>

namespace rp {

constexpr int K32_BM = 128, K32_BN = 64, K32_BK = 32, K32_NBUF = 4;
constexpr int K32_A_BYTES = K32_BM * K32_BK * 4;                   // 16 KB
constexpr int K32_B_BYTES = K32_BN * K32_BK * 4;                   //  8 KB
constexpr int K32_STAGE_BYTES = K32_A_BYTES + K32_B_BYTES;
constexpr int K32_SMEM_BYTES = K32_NBUF * K32_STAGE_BYTES;
constexpr int K32_FETCH = 6;                                       // load instructions per fetching wave and slab

typedef __attribute__((address_space(3))) void* k32_lds_t;

// (a bit cast applied directly to one element of a vector reads the wrong element with this compiler: pass the element by value)
__device__ __forceinline__ uint32_t k32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// A_MC / B_MC: the operand has unit stride along its free index (m, n) instead of along k.  EDGE: m not in whole tiles or n below 64.
// EPI: a bias per column and / or accumulation into C (g.bias, g.accumulate), with finish<float>'s order of additions;
// the old values of C are requested when the tile begins, so they have arrived when its last slab is done.
template <bool A_MC, bool B_MC, bool EDGE, bool EPI>
__global__ void __launch_bounds__(512) gemm_pipe32k_kernel(GemmArgs g, int tiles_m, unsigned total) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char k32_smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    unsigned first, walk_end, stride;
    resident_tile_walk(total, first, walk_end, stride);
    total = walk_end;                                               // this workgroup's tiles: first, first + stride, ... below total
    const int nslab = (g.k + K32_BK - 1) / K32_BK;
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;      // strides of the free index and of k

    if (wave >= 4) {
        // ---- fetch ----
        const int p = wave - 4;
        const long long a_span = (A_MC ? ((long long)(g.k - 1) * a_ks + g.m) : ((long long)(g.m - 1) * a_fs + g.k)) * 4;
        const long long b_span = (B_MC ? ((long long)(g.k - 1) * b_ks + g.n) : ((long long)(g.n - 1) * b_fs + g.k)) * 4;
        // per lane and instruction: byte offset from the slab's first element, and the slab-local k the 16 bytes start at
        uint32_t a_off[4], b_off[2];
        int a_k[4], b_k[2];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (!A_MC) {
                const int row = 8 * q + (lane >> 3);                                 // of the wave's 32 rows
                const int piece = (lane & 7) ^ ((row >> 1) & 7);
                a_off[q] = (uint32_t)(((long long)row * a_fs + piece * 4) * 4);
                a_k[q] = piece * 4;
            } else {
                const int krow = 2 * q + (lane >> 5);                                // of the wave's 8 k rows
                const int c128 = ((lane & 31) >> 3) ^ ((2 * p + (krow >> 2)) & 3);
                a_off[q] = (uint32_t)(((long long)krow * a_ks + (c128 * 8 + (lane & 7)) * 4) * 4);
                a_k[q] = 8 * p + krow;
            }
        }
#pragma unroll
        for (int q = 0; q < 2; q++) {
            if (!B_MC) {
                const int row = 8 * q + (lane >> 3);                                 // of the wave's 16 rows
                const int piece = (lane & 7) ^ ((row >> 1) & 7);
                b_off[q] = (uint32_t)(((long long)row * b_fs + piece * 4) * 4);
                b_k[q] = piece * 4;
            } else {
                const int krow = 4 * q + (lane >> 4);                                // of the wave's 8 k rows
                const int c128 = ((lane & 15) >> 3) ^ ((krow >> 2) & 1);
                b_off[q] = (uint32_t)(((long long)krow * b_ks + (c128 * 8 + (lane & 7)) * 4) * 4);
                b_k[q] = 8 * p + krow;
            }
        }
        // the slab iterator of the fetch: tile `f_id`, slab `f_s` of it, LDS stage `f_stage`
        unsigned f_id = first;
        int f_s = 0, f_stage = 0;
        auto fetch_next = [&]() -> bool {
            if (f_id >= total) return false;
            const unsigned z = f_id / (unsigned)tiles_m;
            const int m0 = (int)(f_id - z * (unsigned)tiles_m) * K32_BM, k0 = f_s * K32_BK, kleft = g.k - k0;
            const __amdgpu_buffer_rsrc_t ra = buffer_rsrc((const float*)g.A + (long long)z * g.a_bs, a_span);
            const __amdgpu_buffer_rsrc_t rb = buffer_rsrc((const float*)g.B + (long long)z * g.b_bs, b_span);
            const int sa = A_MC ? (int)((((long long)(k0 + 8 * p)) * a_ks + m0) * 4) : (int)(((long long)(m0 + 32 * p) * a_fs + k0) * 4);
            const int sb = B_MC ? (int)(((long long)(k0 + 8 * p)) * b_ks * 4) : (int)(((long long)(16 * p) * b_fs + k0) * 4);
            unsigned char* dst = k32_smem + f_stage * K32_STAGE_BYTES;
#pragma unroll
            for (int q = 0; q < 4; q++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (k32_lds_t)(dst + (A_MC ? 8 * p * 512 : 32 * p * 128) + q * 1024), 16,
                                                         a_k[q] < kleft ? (int)a_off[q] : (int)BUFFER_OOB, sa, 0, 0);
#pragma unroll
            for (int q = 0; q < 2; q++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (k32_lds_t)(dst + K32_A_BYTES + (B_MC ? 8 * p * 256 : 16 * p * 128) + q * 1024), 16,
                                                         b_k[q] < kleft ? (int)b_off[q] : (int)BUFFER_OOB, sb, 0, 0);
            f_stage = f_stage + 1 == K32_NBUF ? 0 : f_stage + 1;
            if (++f_s == nslab) { f_s = 0; f_id += stride; }
            return true;
        };
        // Loads return in order, so "slab x has landed" is "at most the loads of the younger fetches are outstanding";
        // where a fetch was skipped because the slabs ran out, the wait is for everything.
        bool full = true;
#pragma unroll
        for (int i = 0; i < K32_NBUF; i++) full = fetch_next() && full;
        if (full) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K32_FETCH * (K32_NBUF - 1)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                               // slab 0 is in LDS
        if (full) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K32_FETCH * (K32_NBUF - 2)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (unsigned id = first; id < total; id += stride) {
            for (int s = 0; s < nslab; s++) {
                __syncthreads();                                       // the next slab is in LDS; the stage of this one is free
                if (fetch_next()) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K32_FETCH * (K32_NBUF - 2)) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
        }
        return;
    }

    // ---- multiply and store ----
    const int r = lane & 31, h = lane >> 5;
    // LDS byte offsets inside a stage.  k-contiguous operand: the lane's 16 bytes of group u (k = 8u + 4h .. + 3) sit at
    // base ^ (32 u).  Other operands: the value of step (u, e), k row 8u + 4h + e, sits at base_h + (8u + e) rows, with
    // the 128-byte piece XORed by (k row / 4) % 4 (A) or % 2 (B): for A that is (2u + h) % 4, folded in per u below; for B
    // it is h, folded into the base.
    const uint32_t a_kc = (uint32_t)((32 * wave + r) * 128 + ((h ^ ((r >> 1) & 7)) * 16));
    const uint32_t a_mc = (uint32_t)(4 * h * 512 + r * 4);
    uint32_t b_base[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
        b_base[j] = B_MC ? (uint32_t)(K32_A_BYTES + 4 * h * 256 + ((j ^ h) * 128) + r * 4)
                         : (uint32_t)(K32_A_BYTES + (32 * j + r) * 128 + ((h ^ ((r >> 1) & 7)) * 16));
    const uint32_t c_lane = (uint32_t)(((long long)(4 * h) * g.c_rs + (long long)r * g.c_cs) * 4);
    const long long c_span = ((long long)(g.m - 1) * g.c_rs + (long long)(g.n - 1) * g.c_cs + 1) * 4;

    f32x16_t acc[2];                    // [j: columns 32 j .. 32 j + 31]
    float af[16], bf[2][16];            // [4u + e]: the lane's value for MFMA step (u, e)
    const bool has_bias = EPI && g.bias != nullptr, accum = EPI && g.accumulate != 0;
    float bias_v[2] = {0.f, 0.f};       // EPI: the bias of the lane's columns 32 j + r (the same for every tile: n <= 64)
    float old[EPI ? 32 : 1];            // EPI: the current tile's old values of C, [16 j + v]
    if constexpr (EPI) {
#pragma unroll
        for (int j = 0; j < 2; j++)
            if (has_bias && 32 * j + r < g.n) bias_v[j] = ((const float*)g.bias)[32 * j + r];
    }

    auto read_group = [&](const unsigned char* stage, auto u_c) {
        constexpr int u = decltype(u_c)::value;
        if constexpr (!A_MC) {
            const f32x4_t v = *(const f32x4_t*)(stage + (a_kc ^ (uint32_t)(32 * u)));
            af[4 * u + 0] = v[0]; af[4 * u + 1] = v[1]; af[4 * u + 2] = v[2]; af[4 * u + 3] = v[3];
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                af[4 * u + e] = *(const float*)(stage + a_mc + (8 * u + e) * 512 + (((uint32_t)wave ^ (uint32_t)((2 * u + h) & 3)) * 128));
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if constexpr (!B_MC) {
                const f32x4_t v = *(const f32x4_t*)(stage + (b_base[j] ^ (uint32_t)(32 * u)));
                bf[j][4 * u + 0] = v[0]; bf[j][4 * u + 1] = v[1]; bf[j][4 * u + 2] = v[2]; bf[j][4 * u + 3] = v[3];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) bf[j][4 * u + e] = *(const float*)(stage + b_base[j] + (8 * u + e) * 256);
            }
        }
    };

    // One slab, whose values are already in registers: behind each group's MFMAs the same group of the NEXT slab is read.
    auto slab_pass = [&](int next) {
        const unsigned char* next_base = k32_smem + next * K32_STAGE_BYTES;
        __syncthreads();                                   // the next slab is in LDS; this slab's values have all arrived in registers
        static_for<0, 4>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[4 * u + e], bf[j][4 * u + e], acc[j], 0, 0, 0);
            read_group(next_base, uc);
        });
    };

    __syncthreads();                                   // slab 0 is in LDS
    if (first >= total) return;
    static_for<0, 4>([&](auto uc) { read_group(k32_smem, uc); });
    int next = 1;
    for (unsigned id = first; id < total; id += stride) {
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[j][v] = 0.f;
        // register v of tile j is row 8(v / 4) + 4h + v % 4, columns 32 j + r
        const unsigned z = id / (unsigned)tiles_m;
        const int gm0 = (int)(id - z * (unsigned)tiles_m) * K32_BM + 32 * wave;
        const __amdgpu_buffer_rsrc_t rc = buffer_rsrc((float*)g.C + (long long)z * g.c_bs, c_span);
        auto place = [&](auto nc, int& soff, uint32_t& voff) {
            constexpr int n = decltype(nc)::value, j = n >> 4, v = n & 15, row = 8 * (v / 4) + (v % 4);
            const int gm = gm0 + row;
            soff = (int)(((long long)gm * g.c_rs + (long long)(32 * j) * g.c_cs) * 4);
            voff = c_lane;
            if constexpr (EDGE) voff = (gm + 4 * h < g.m && 32 * j + r < g.n) ? c_lane : BUFFER_OOB;
        };
        if constexpr (EPI) {
            if (accum) static_for<0, 32>([&](auto nc) {
                int soff; uint32_t voff;
                place(nc, soff, voff);
                old[decltype(nc)::value] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rc, (int)voff, soff, 0));
            });
        }
        for (int s = 0; s < nslab; s++) {
            slab_pass(next);
            next = next + 1 == K32_NBUF ? 0 : next + 1;
        }
        // the tile's stores
        static_for<0, 32>([&](auto nc) {
            constexpr int n = decltype(nc)::value, j = n >> 4, v = n & 15;
            int soff; uint32_t voff;
            place(nc, soff, voff);
            float val = acc[j][v];
            if constexpr (EPI) {
                if (has_bias) val = val + bias_v[j];
                if (accum) val = old[n] + val;
            }
            __builtin_amdgcn_raw_buffer_store_b32(k32_bits(val), rc, (int)voff, soff, 2);          // (streaming store)
        });
    }
}

// ---- host side ----

// Whether this kernel takes the product: fp32, n <= 64, k in whole fours, both operands with a unit stride and 16-byte
// aligned rows (no segments or folded store; a bias per column and accumulation into C are taken), and every byte offset
// the kernel forms from a batch entry's base within the 32-bit range of buffer addressing.
bool pipe32k_takes(const GemmArgs& g) {
    if (g.n > K32_BN || g.n < 1 || g.k < 4 || g.k % 4 || g.m < 1 || g.batch < 1) return false;
    if ((long long)((g.m + K32_BM - 1) / K32_BM) * g.batch >= (1ll << 30)) return false;
    if (g.seg_k || g.seg_n || g.c_fold_from || g.bias_by_row || ((uintptr_t)g.bias & 3)) return false;
    const bool a_kc = g.a_cs == 1 && g.a_rs % 4 == 0, a_mc = g.a_rs == 1 && g.a_cs % 4 == 0;
    const bool b_kc = g.b_rs == 1 && g.b_cs % 4 == 0, b_mc = g.b_cs == 1 && g.b_rs % 4 == 0;
    if (!(a_kc || a_mc) || !(b_kc || b_mc) || g.a_bs % 4 || g.b_bs % 4 || g.a_rs < 0 || g.a_cs < 0 || g.b_rs < 0 || g.b_cs < 0) return false;
    if (g.c_rs < 0 || g.c_cs < 0) return false;
    if (((uintptr_t)g.A & 15) || ((uintptr_t)g.B & 15) || ((uintptr_t)g.C & 3)) return false;
    const long long lim = 1ll << 30;
    // free indices up to a whole tile past the last one and k up to a whole slab past the end are addressed (and read as
    // zero, or as values that only reach outputs which are not stored)
    const long long kk = g.k + K32_BK;
    const long long a_reach = (a_kc ? (long long)(g.m + K32_BM) * g.a_rs + kk : kk * g.a_cs + g.m + K32_BM) * 4;
    const long long b_reach = (b_kc ? (long long)(g.n + K32_BN) * g.b_cs + kk : kk * g.b_rs + g.n + K32_BN) * 4;
    const long long c_reach = ((long long)(g.m + K32_BM) * g.c_rs + (long long)K32_BN * g.c_cs) * 4;
    return a_reach < lim && b_reach < lim && c_reach < lim;
}

int launch_pipe32k(const GemmArgs& g) {
    const int tiles_m = (g.m + K32_BM - 1) / K32_BM;
    const long long total = (long long)tiles_m * g.batch;
    int cus = device_cu_count();
    if (cus <= 0) cus = 256;
    const unsigned blocks = (unsigned)(total < cus ? total : cus);          // one resident workgroup per CU walks its tiles
    const bool edge = (g.m % K32_BM) || g.n != K32_BN;
    const bool a_mc = !(g.a_cs == 1 && g.a_rs % 4 == 0), b_mc = !(g.b_rs == 1 && g.b_cs % 4 == 0);
    auto launch = [&](auto kern) {
        if (!check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, K32_SMEM_BYTES), "hipFuncSetAttribute")) return -1;
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(512), K32_SMEM_BYTES, current_stream(), g, tiles_m, (unsigned)total);
        return check_launch("gemm_pipe32k_kernel") ? 0 : -1;
    };
    auto pick = [&](auto epi_c) {
        constexpr bool EPI = decltype(epi_c)::value;
        if (!a_mc && !b_mc) return edge ? launch(gemm_pipe32k_kernel<false, false, true, EPI>) : launch(gemm_pipe32k_kernel<false, false, false, EPI>);
        if (!a_mc && b_mc) return edge ? launch(gemm_pipe32k_kernel<false, true, true, EPI>) : launch(gemm_pipe32k_kernel<false, true, false, EPI>);
        if (a_mc && !b_mc) return edge ? launch(gemm_pipe32k_kernel<true, false, true, EPI>) : launch(gemm_pipe32k_kernel<true, false, false, EPI>);
        return edge ? launch(gemm_pipe32k_kernel<true, true, true, EPI>) : launch(gemm_pipe32k_kernel<true, true, false, EPI>);
    };
    return (g.bias || g.accumulate) ? pick(std::true_type{}) : pick(std::false_type{});
}

}  // namespace rp
