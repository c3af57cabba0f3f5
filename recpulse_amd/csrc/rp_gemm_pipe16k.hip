// bf16 / fp16 GEMM with an output of at most 64 columns and many row tiles, e.g. O = P.V or dV = P^T.dO per head:
// 128 x 64 outputs per tile from a 128 x k strip of A.  The product is bound by reading A, and a kernel that loads a
// k slab into registers, waits, and copies it to LDS never has enough bytes in flight to read at memory speed.
//
// One block of eight waves stays on each CU and walks its tiles; the unit of the pipeline is the k slab of 64:
//
//  - waves 4..7 only fetch: a slab of A (128 x 64) and of B (64 x 64) goes from memory straight into one of four LDS
//    stages (buffer loads with the LDS bit, 1 KB per instruction, no registers), three slabs ahead of the multipliers.
//    Operands with unit stride along k lie in LDS as rows of 64 k values (128 bytes) whose 16-byte pieces are XORed with
//    bits 1..3 of the row; operands with unit stride along their free index lie as k rows (A: 256 bytes, B: 128 bytes)
//    whose 32-byte pieces are XORed with the k row (A: its low three bits, B: bits 1..2): the fragment reads of both kinds
//    then spread over all banks.
//  - waves 0..3 multiply and store: wave w owns rows 32w .. 32w + 31 of the tile, all 64 columns, as two
//    v_mfma_f32_32x32x16 tiles with the operands SWAPPED (the MFMA computes the transposed tile), so a lane ends up with
//    one row of C and four adjacent columns per accumulator quad.  Fragments of k-contiguous operands are 16-byte LDS
//    reads; fragments of the others are two transposing reads (ds_read_b64_tr_b16).  While slab s is multiplied the
//    fragments of slab s + 1 are read into the registers the MFMAs have just used, so no MFMA waits for LDS.  A finished
//    tile is narrowed into 16 registers and leaves through a staging patch of LDS that belongs to the wave alone, as
//    whole rows, between the MFMAs of the next tile's first slab.
//
// The fetching waves wait for loads only, the multiplying waves issue stores only; one block-wide barrier per slab says
// "slab s + 1 has landed, and the stage of slab s is free again".
#include "rp_gemm.h"

#include <type_traits>

namespace rp {

constexpr int K16_BM = 128, K16_BN = 64, K16_BK = 64, K16_NBUF = 4;
constexpr int K16_A_BYTES = K16_BM * K16_BK * 2;                   // 16 KB
constexpr int K16_B_BYTES = K16_BN * K16_BK * 2;                   //  8 KB
constexpr int K16_STAGE_BYTES = K16_A_BYTES + K16_B_BYTES;
constexpr int K16_PATCH_BYTES = 32 * 128;                          // a wave's 32 x 64 outputs, 16 bit
constexpr int K16_SMEM_BYTES = K16_NBUF * K16_STAGE_BYTES + 4 * K16_PATCH_BYTES;
constexpr int K16_FETCH = 6;                                       // load instructions per fetching wave and slab

typedef __attribute__((address_space(3))) void* k16_lds_t;
typedef __attribute__((ext_vector_type(4))) short k16_s16x4_t;

template <typename T> struct k16_ops;
template <> struct k16_ops<bf16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    // two accumulators -> two bf16 in one word: adding 0x8000 carries into bit 16 exactly when the first dropped bit is set
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        return __builtin_amdgcn_perm(__float_as_uint(hi) + 0x8000u, __float_as_uint(lo) + 0x8000u, 0x07060302u);
    }
};
template <> struct k16_ops<f16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        return (uint32_t)narrow_f16_bits(lo) | ((uint32_t)narrow_f16_bits(hi) << 16);
    }
};

// half H (k values 4H .. 4H + 3 of the lane's eight) of a fragment of an operand that lies in LDS as k rows
template <int H>
__device__ __forceinline__ void k16_read_tr(s16x8_t& v, const unsigned char* p) {
    const k16_s16x4_t q = __builtin_amdgcn_ds_read_tr16_b64_v4i16((k16_s16x4_t __attribute__((address_space(3)))*)(p));
    v[4 * H + 0] = q[0]; v[4 * H + 1] = q[1]; v[4 * H + 2] = q[2]; v[4 * H + 3] = q[3];
}

// 16-bit storage -> fp32 and back for the epilogue's additions (one rounding per reference op, like finish<T>)
template <typename T> __device__ __forceinline__ float k16_widen_lo(uint32_t w);
template <typename T> __device__ __forceinline__ float k16_widen_hi(uint32_t w);
template <> __device__ __forceinline__ float k16_widen_lo<bf16_t>(uint32_t w) { return __uint_as_float(w << 16); }
template <> __device__ __forceinline__ float k16_widen_hi<bf16_t>(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
template <> __device__ __forceinline__ float k16_widen_lo<f16_t>(uint32_t w) { f16_t x; x.bits = (uint16_t)w; return widen(x); }
template <> __device__ __forceinline__ float k16_widen_hi<f16_t>(uint32_t w) { f16_t x; x.bits = (uint16_t)(w >> 16); return widen(x); }

// A_MC / B_MC: the operand has unit stride along its free index (m, n) instead of along k.  EDGE: m not in whole tiles or n below 64.
// EPI: a bias per column and / or accumulation into C (g.bias, g.accumulate): the tile is then stored right after its
// last slab instead of between the MFMAs of the next tile, the old rows of C having been requested when the tile began.
template <typename T, bool A_MC, bool B_MC, bool EDGE, bool EPI>
__global__ void __launch_bounds__(512) gemm_pipe16k_kernel(GemmArgs g, int tiles_m, unsigned total) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char k16_smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    unsigned first, walk_end, stride;
    resident_tile_walk(total, first, walk_end, stride);
    total = walk_end;                                               // this workgroup's tiles: first, first + stride, ... below total
    const int nslab = (g.k + K16_BK - 1) / K16_BK;
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;      // strides of the free index and of k

    if (wave >= 4) {
        // ---- fetch ----
        const int p = wave - 4;
        const long long a_span = (A_MC ? ((long long)(g.k - 1) * a_ks + g.m) : ((long long)(g.m - 1) * a_fs + g.k)) * 2;
        const long long b_span = (B_MC ? ((long long)(g.k - 1) * b_ks + g.n) : ((long long)(g.n - 1) * b_fs + g.k)) * 2;
        // per lane and instruction: byte offset from the slab's first element, and the slab-local k the 16 bytes start at
        uint32_t a_off[4], b_off[2];
        int a_k[4], b_k[2];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (!A_MC) {
                const int row = 8 * q + (lane >> 3);                                 // of the wave's 32 rows
                const int piece = (lane & 7) ^ ((row >> 1) & 7);
                a_off[q] = (uint32_t)(((long long)row * a_fs + piece * 8) * 2);
                a_k[q] = piece * 8;
            } else {
                const int krow = 4 * q + (lane >> 4);                                // of the wave's 16 k rows
                const int c32 = ((lane & 15) >> 1) ^ (krow & 7);
                a_off[q] = (uint32_t)(((long long)krow * a_ks + (c32 * 2 + (lane & 1)) * 8) * 2);
                a_k[q] = 16 * p + krow;
            }
        }
#pragma unroll
        for (int q = 0; q < 2; q++) {
            if (!B_MC) {
                const int row = 8 * q + (lane >> 3);                                 // of the wave's 16 rows
                const int piece = (lane & 7) ^ ((row >> 1) & 7);
                b_off[q] = (uint32_t)(((long long)row * b_fs + piece * 8) * 2);
                b_k[q] = piece * 8;
            } else {
                const int krow = 8 * q + (lane >> 3);                                // of the wave's 16 k rows
                const int c32 = ((lane & 7) >> 1) ^ ((krow >> 1) & 3);
                b_off[q] = (uint32_t)(((long long)krow * b_ks + (c32 * 2 + (lane & 1)) * 8) * 2);
                b_k[q] = 16 * p + krow;
            }
        }
        // the slab iterator of the fetch: tile `f_id`, slab `f_s` of it, LDS stage `f_stage`
        unsigned f_id = first;
        int f_s = 0, f_stage = 0;
        auto fetch_next = [&]() -> bool {
            if (f_id >= total) return false;
            const unsigned z = f_id / (unsigned)tiles_m;
            const int m0 = (int)(f_id - z * (unsigned)tiles_m) * K16_BM, k0 = f_s * K16_BK, kleft = g.k - k0;
            const __amdgpu_buffer_rsrc_t ra = buffer_rsrc((const uint16_t*)g.A + (long long)z * g.a_bs, a_span);
            const __amdgpu_buffer_rsrc_t rb = buffer_rsrc((const uint16_t*)g.B + (long long)z * g.b_bs, b_span);
            const int sa = A_MC ? (int)((((long long)(k0 + 16 * p)) * a_ks + m0) * 2) : (int)(((long long)(m0 + 32 * p) * a_fs + k0) * 2);
            const int sb = B_MC ? (int)(((long long)(k0 + 16 * p)) * b_ks * 2) : (int)(((long long)(16 * p) * b_fs + k0) * 2);
            unsigned char* dst = k16_smem + f_stage * K16_STAGE_BYTES;
#pragma unroll
            for (int q = 0; q < 4; q++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (k16_lds_t)(dst + (A_MC ? 16 * p * 256 : 32 * p * 128) + q * 1024), 16,
                                                         a_k[q] < kleft ? (int)a_off[q] : (int)BUFFER_OOB, sa, 0, 0);
#pragma unroll
            for (int q = 0; q < 2; q++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (k16_lds_t)(dst + K16_A_BYTES + 16 * p * 128 + q * 1024), 16,
                                                         b_k[q] < kleft ? (int)b_off[q] : (int)BUFFER_OOB, sb, 0, 0);
            f_stage = f_stage + 1 == K16_NBUF ? 0 : f_stage + 1;
            if (++f_s == nslab) { f_s = 0; f_id += stride; }
            return true;
        };
        // Loads return in order, so "slab x has landed" is "at most the loads of the younger fetches are outstanding";
        // where a fetch was skipped because the slabs ran out, the wait is for everything.
        bool full = true;
#pragma unroll
        for (int i = 0; i < K16_NBUF; i++) full = fetch_next() && full;
        if (full) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K16_FETCH * (K16_NBUF - 1)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                               // slab 0 is in LDS
        if (full) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K16_FETCH * (K16_NBUF - 2)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (unsigned id = first; id < total; id += stride) {
            for (int s = 0; s < nslab; s++) {
                __syncthreads();                                       // the next slab is in LDS; the stage of this one is free
                if (fetch_next()) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K16_FETCH * (K16_NBUF - 2)) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
        }
        return;
    }

    // ---- multiply and store ----
    const int r = lane & 31, h = lane >> 5, grp = lane >> 4, s16 = lane & 15;
    // fragment addresses inside a stage for k step 0
    //   k-contiguous operand: piece 2ks + h of the lane's row: base ^ (32 ks)
    //   other operands: the transposing read of a 16-lane group covers 4 k rows x 16 free indices; source lane s points at
    //   free indices 4(s % 4) .. + 3 of k row s / 4; the groups are (k octet, free half) = (grp / 2, grp % 2)
    uint32_t a_fr[2], b_fr[2][2];                                   // [H] and [H][in] (k-contiguous: only [0] / [0][in] are used)
    if (!A_MC) {
        a_fr[0] = (uint32_t)((32 * wave + r) * 128 + ((h ^ ((r >> 1) & 7)) * 16));
        a_fr[1] = 0;
    } else {
#pragma unroll
        for (int H = 0; H < 2; H++) {
            const int krow = 8 * (grp >> 1) + 4 * H + (s16 >> 2);
            a_fr[H] = (uint32_t)(krow * 256 + (((2 * wave + (grp & 1)) ^ (krow & 7)) * 32) + 8 * (s16 & 3));
        }
    }
#pragma unroll
    for (int in = 0; in < 2; in++) {
        if (!B_MC) {
            b_fr[0][in] = (uint32_t)(K16_A_BYTES + (32 * in + r) * 128 + ((h ^ ((r >> 1) & 7)) * 16));
            b_fr[1][in] = 0;
        } else {
#pragma unroll
            for (int H = 0; H < 2; H++) {
                const int krow = 8 * (grp >> 1) + 4 * H + (s16 >> 2);
                b_fr[H][in] = (uint32_t)(K16_A_BYTES + krow * 128 + (((2 * in + (grp & 1)) ^ ((krow >> 1) & 3)) * 32) + 8 * (s16 & 3));
            }
        }
    }
    // The wave's own staging patch (32 rows of 128 bytes, 16-byte pieces XORed like a k-contiguous operand).  A lane holds
    // row r of C and four adjacent columns per accumulator quad: 8 bytes at piece 4 in + q, half h.  Read back, a lane
    // holds 16 bytes of row lane / 8 (+ 8 per instruction), piece lane % 8: eight whole rows per store instruction.
    unsigned char* patch = k16_smem + K16_NBUF * K16_STAGE_BYTES + wave * K16_PATCH_BYTES;
    const uint32_t st_write = (uint32_t)(r * 128 + 8 * h), st_swz = (uint32_t)((r >> 1) & 7);
    const int rr = lane >> 3, rp = lane & 7;
    const uint32_t c_lane = (uint32_t)(((long long)rr * g.c_rs + 8 * rp) * 2);
    const long long c_span = ((long long)(g.m - 1) * g.c_rs + g.n) * 2;

    f32x16_t acc[2];                    // [in: columns 32 in .. 32 in + 31]
    u32x2_t packed[8];                  // the previous tile, narrowed: [in][q]
    u32x4_t rows[4];                    // its rows on their way from the staging patch to memory
    s16x8_t af[4], bf[4][2];            // [k step]([in]): eight k values of the lane's row / column
    // EPI: the bias of the lane's columns 32 in + 8 q + 4 h + e as fp32 (the same for every tile: n <= 64), and the old
    // rows of C of the current tile (pieces like `rows`)
    float bias_f[EPI ? 32 : 1];
    u32x4_t old[EPI ? 4 : 1];
    const bool has_bias = EPI && g.bias != nullptr, accum = EPI && g.accumulate != 0;
    if constexpr (EPI) {
#pragma unroll
        for (int n = 0; n < 8; n++) {
            const int col = 32 * (n >> 2) + 8 * (n & 3) + 4 * h;
            u32x2_t w = {0u, 0u};
            if (has_bias && col < g.n) w = *(const u32x2_t*)((const uint16_t*)g.bias + col);          // (n is a multiple of 8: four columns are inside or outside together)
            bias_f[4 * n + 0] = k16_widen_lo<T>(w[0]); bias_f[4 * n + 1] = k16_widen_hi<T>(w[0]);
            bias_f[4 * n + 2] = k16_widen_lo<T>(w[1]); bias_f[4 * n + 3] = k16_widen_hi<T>(w[1]);
        }
    }

    auto read_frags = [&](const unsigned char* stage, auto ks_c) {
        constexpr int ks = decltype(ks_c)::value;
        if constexpr (!A_MC) {
            af[ks] = *(const s16x8_t*)(stage + (a_fr[0] ^ (uint32_t)(32 * ks)));
        } else {
            k16_read_tr<0>(af[ks], stage + a_fr[0] + 16 * ks * 256);
            k16_read_tr<1>(af[ks], stage + a_fr[1] + 16 * ks * 256);
        }
#pragma unroll
        for (int in = 0; in < 2; in++) {
            if constexpr (!B_MC) {
                bf[ks][in] = *(const s16x8_t*)(stage + (b_fr[0][in] ^ (uint32_t)(32 * ks)));
            } else {
                k16_read_tr<0>(bf[ks][in], stage + b_fr[0][in] + 16 * ks * 128);
                k16_read_tr<1>(bf[ks][in], stage + b_fr[1][in] + 16 * ks * 128);
            }
        }
    };
    auto pack_all = [&]() {
        static_for<0, 8>([&](auto nc) {
            constexpr int n = decltype(nc)::value, in = n >> 2, q = n & 3;
            float v0 = acc[in][4 * q], v1 = acc[in][4 * q + 1], v2 = acc[in][4 * q + 2], v3 = acc[in][4 * q + 3];
            if constexpr (EPI) {
                if (has_bias) {                        // the product is rounded to the tensor type first, like the reference's matmul output
                    const uint32_t p01 = k16_ops<T>::pack(v0, v1), p23 = k16_ops<T>::pack(v2, v3);
                    v0 = k16_widen_lo<T>(p01) + bias_f[4 * n + 0]; v1 = k16_widen_hi<T>(p01) + bias_f[4 * n + 1];
                    v2 = k16_widen_lo<T>(p23) + bias_f[4 * n + 2]; v3 = k16_widen_hi<T>(p23) + bias_f[4 * n + 3];
                }
            }
            packed[n][0] = k16_ops<T>::pack(v0, v1);
            packed[n][1] = k16_ops<T>::pack(v2, v3);
        });
    };
    auto stage_write = [&](auto n_c) {
        constexpr int n = decltype(n_c)::value, in = n >> 2, q = n & 3;
        *(u32x2_t*)(patch + st_write + (((uint32_t)(4 * in + q) ^ st_swz) * 16)) = packed[n];
    };
    auto row_read = [&](auto e_c) {
        constexpr int e = decltype(e_c)::value;
        const int row = 8 * e + rr;
        rows[e] = *(const u32x4_t*)(patch + row * 128 + (((uint32_t)rp ^ (uint32_t)((row >> 1) & 7)) * 16));
    };
    auto row_store = [&](auto e_c, int pm0, const __amdgpu_buffer_rsrc_t& rc) {
        constexpr int e = decltype(e_c)::value;
        const int gm = pm0 + 32 * wave + 8 * e;
        const int soff = (int)((long long)gm * g.c_rs * 2);
        uint32_t voff = c_lane;
        if constexpr (EDGE) voff = (gm + rr < g.m && 8 * rp < g.n) ? c_lane : BUFFER_OOB;      // (n is a multiple of 8: a piece is inside or outside as a whole)
        __builtin_amdgcn_raw_buffer_store_b128(rows[e], rc, (int)voff, soff, 2);          // (streaming store: the output is not read again by this kernel)
    };

    // EPI: request the rows of C that tile (pm0, rc) will be added to; add them to the finished rows
    auto old_load = [&](auto e_c, int pm0, const __amdgpu_buffer_rsrc_t& rc) {
        constexpr int e = decltype(e_c)::value;
        const int gm = pm0 + 32 * wave + 8 * e;
        const int soff = (int)((long long)gm * g.c_rs * 2);
        uint32_t voff = c_lane;
        if constexpr (EDGE) voff = (gm + rr < g.m && 8 * rp < g.n) ? c_lane : BUFFER_OOB;
        old[e] = __builtin_amdgcn_raw_buffer_load_b128(rc, (int)voff, soff, 0);
    };
    auto row_add_old = [&](auto e_c) {
        constexpr int e = decltype(e_c)::value;
#pragma unroll
        for (int d = 0; d < 4; d++)
            rows[e][d] = k16_ops<T>::pack(k16_widen_lo<T>(old[e][d]) + k16_widen_lo<T>(rows[e][d]), k16_widen_hi<T>(old[e][d]) + k16_widen_hi<T>(rows[e][d]));
    };

    // One slab, whose fragments are already in registers: behind each k step's MFMAs the same fragments of the NEXT slab
    // are read (LDS stage `next`).  If STORE, the previous tile (narrowed, in `packed`) goes through the staging patch to
    // memory meanwhile: staging writes behind MFMAs 0-1, row reads behind 2-3, row stores behind 4-7.
    auto slab_pass = [&](auto store_c, int next, int pm0, const __amdgpu_buffer_rsrc_t& rc) {
        constexpr bool STORE = decltype(store_c)::value;
        const unsigned char* next_base = k16_smem + next * K16_STAGE_BYTES;
        __syncthreads();                                   // the next slab is in LDS; this slab's fragments have all arrived in registers
        static_for<0, 4>([&](auto ksc) {
            constexpr int ks = decltype(ksc)::value;
            static_for<0, 2>([&](auto ic) {
                constexpr int in = decltype(ic)::value, mi = 2 * ks + in;
                acc[in] = k16_ops<T>::mma(bf[ks][in], af[ks], acc[in]);          // operands swapped: the MFMA's rows are columns of C
                if constexpr (STORE) {
                    if constexpr (mi < 2) static_for<0, 4>([&](auto ec) { stage_write(std::integral_constant<int, 4 * mi + decltype(ec)::value>{}); });
                    else if constexpr (mi < 4) static_for<0, 2>([&](auto ec) { row_read(std::integral_constant<int, 2 * (mi - 2) + decltype(ec)::value>{}); });
                    else row_store(std::integral_constant<int, mi - 4>{}, pm0, rc);
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            read_frags(next_base, ksc);
        });
    };

    __syncthreads();                                   // slab 0 is in LDS
    if (first >= total) return;
    static_for<0, 4>([&](auto ksc) { read_frags(k16_smem, ksc); });
    int next = 1, pm0 = 0;
    bool pending = false;                              // a finished tile waits in `packed`
    __amdgpu_buffer_rsrc_t rc = buffer_rsrc(g.C, c_span);
    for (unsigned id = first; id < total; id += stride) {
#pragma unroll
        for (int in = 0; in < 2; in++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[in][v] = 0.f;
        if constexpr (EPI) {
            // this tile's place in C is known from the start: its old rows travel while the tile is multiplied
            const unsigned z = id / (unsigned)tiles_m;
            pm0 = (int)(id - z * (unsigned)tiles_m) * K16_BM;
            rc = buffer_rsrc((uint16_t*)g.C + (long long)z * g.c_bs, c_span);
            if (accum) static_for<0, 4>([&](auto ec) { old_load(ec, pm0, rc); });
            for (int s = 0; s < nslab; s++) {
                slab_pass(std::false_type{}, next, pm0, rc);
                next = next + 1 == K16_NBUF ? 0 : next + 1;
            }
            pack_all();
            static_for<0, 8>([&](auto nc) { stage_write(nc); });
            static_for<0, 4>([&](auto ec) { row_read(ec); });
            if (accum) static_for<0, 4>([&](auto ec) { row_add_old(ec); });
            static_for<0, 4>([&](auto ec) { row_store(ec, pm0, rc); });
            continue;
        }
        for (int s = 0; s < nslab; s++) {
            if (pending) slab_pass(std::true_type{}, next, pm0, rc);
            else slab_pass(std::false_type{}, next, pm0, rc);
            pending = false;
            next = next + 1 == K16_NBUF ? 0 : next + 1;
        }
        pack_all();
        const unsigned z = id / (unsigned)tiles_m;
        pm0 = (int)(id - z * (unsigned)tiles_m) * K16_BM;
        rc = buffer_rsrc((uint16_t*)g.C + (long long)z * g.c_bs, c_span);
        pending = true;
    }
    if constexpr (EPI) return;
    // the last tile
    static_for<0, 8>([&](auto nc) { stage_write(nc); });
    static_for<0, 4>([&](auto ec) { row_read(ec); });
    static_for<0, 4>([&](auto ec) { row_store(ec, pm0, rc); });
}

// ---- host side ----

// Whether this kernel takes the product: n <= 64 in whole eights, k in whole eights, both operands with a unit stride and
// 16-byte aligned rows, C row-major with 16-byte aligned rows (no segments or folded store; a bias per column, 8-byte
// aligned, and accumulation into C are taken), and every byte offset the kernel forms from a batch entry's base within
// the 32-bit range of buffer addressing.
bool pipe16k_takes(const GemmArgs& g) {
    if (g.n > K16_BN || g.n < 8 || g.n % 8 || g.k < 8 || g.k % 8 || g.m < 1 || g.batch < 1) return false;
    if ((long long)((g.m + K16_BM - 1) / K16_BM) * g.batch >= (1ll << 30)) return false;
    if (g.seg_k || g.seg_n || g.c_fold_from || g.bias_by_row || ((uintptr_t)g.bias & 7)) return false;
    const bool a_kc = g.a_cs == 1 && g.a_rs % 8 == 0, a_mc = g.a_rs == 1 && g.a_cs % 8 == 0 && g.m % 8 == 0;
    const bool b_kc = g.b_rs == 1 && g.b_cs % 8 == 0, b_mc = g.b_cs == 1 && g.b_rs % 8 == 0;
    if (!(a_kc || a_mc) || !(b_kc || b_mc) || g.a_bs % 8 || g.b_bs % 8 || g.a_rs < 0 || g.a_cs < 0 || g.b_rs < 0 || g.b_cs < 0) return false;
    if (g.c_cs != 1 || g.c_rs % 8 || g.c_bs % 8 || g.c_rs < 0) return false;
    if (((uintptr_t)g.A & 15) || ((uintptr_t)g.B & 15) || ((uintptr_t)g.C & 15)) return false;
    const long long lim = 1ll << 30;
    // free indices up to a whole tile past the last one and k up to a whole slab past the end are addressed (and read as
    // zero, or as values that only reach outputs which are not stored)
    const long long kk = g.k + K16_BK;
    const long long a_reach = (a_kc ? (long long)(g.m + K16_BM) * g.a_rs + kk : kk * g.a_cs + g.m + K16_BM) * 2;
    const long long b_reach = (b_kc ? (long long)(g.n + K16_BN) * g.b_cs + kk : kk * g.b_rs + g.n + K16_BN) * 2;
    const long long c_reach = ((long long)(g.m + K16_BM) * g.c_rs + K16_BN) * 2;
    return a_reach < lim && b_reach < lim && c_reach < lim;
}

template <typename T>
static int launch_pipe16k_t(const GemmArgs& g) {
    const int tiles_m = (g.m + K16_BM - 1) / K16_BM;
    const long long total = (long long)tiles_m * g.batch;
    int cus = device_cu_count();
    if (cus <= 0) cus = 256;
    const unsigned blocks = (unsigned)(total < cus ? total : cus);          // one resident workgroup per CU walks its tiles
    const bool edge = (g.m % K16_BM) || g.n != K16_BN;
    const bool a_mc = !(g.a_cs == 1 && g.a_rs % 8 == 0), b_mc = !(g.b_rs == 1 && g.b_cs % 8 == 0);
    auto launch = [&](auto kern) {
        if (!check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, K16_SMEM_BYTES), "hipFuncSetAttribute")) return -1;
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(512), K16_SMEM_BYTES, current_stream(), g, tiles_m, (unsigned)total);
        return check_launch("gemm_pipe16k_kernel") ? 0 : -1;
    };
    auto pick = [&](auto epi_c) {
        constexpr bool EPI = decltype(epi_c)::value;
        if (!a_mc && !b_mc) return edge ? launch(gemm_pipe16k_kernel<T, false, false, true, EPI>) : launch(gemm_pipe16k_kernel<T, false, false, false, EPI>);
        if (!a_mc && b_mc) return edge ? launch(gemm_pipe16k_kernel<T, false, true, true, EPI>) : launch(gemm_pipe16k_kernel<T, false, true, false, EPI>);
        if (a_mc && !b_mc) return edge ? launch(gemm_pipe16k_kernel<T, true, false, true, EPI>) : launch(gemm_pipe16k_kernel<T, true, false, false, EPI>);
        return edge ? launch(gemm_pipe16k_kernel<T, true, true, true, EPI>) : launch(gemm_pipe16k_kernel<T, true, true, false, EPI>);
    };
    return (g.bias || g.accumulate) ? pick(std::true_type{}) : pick(std::false_type{});
}

int launch_pipe16k(const GemmArgs& g, int dtype) {
    if (dtype == RP_DTYPE_BFLOAT16) return launch_pipe16k_t<bf16_t>(g);
    if (dtype == RP_DTYPE_FLOAT16) return launch_pipe16k_t<f16_t>(g);
    set_error("pipe16k GEMM: 16-bit types only");
    return -1;
}

}  // namespace rp
