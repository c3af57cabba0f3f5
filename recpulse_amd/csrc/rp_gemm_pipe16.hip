// bf16 / fp16 GEMM with a short reduction (k <= 64), e.g. S = Q.K^T per head (both operands contiguous along k) or the
// lowered convolution's dcol = W^T.dy (both contiguous along their free index); every combination is taken.
//
// 128 x 128 outputs per tile from 2 x 128 x 64 inputs: the product is bound by what it writes.  The arithmetic of a tile
// is 16 MFMAs per wave; what takes time is narrowing 64 accumulators per lane and getting 32 KB of stores out.  As in the
// fp32 kernel of the same shape (rp_gemm_pipe32.hip) one block of eight waves stays on each CU:
//
//  - waves 4..7 only fetch: rows of A and B (128 bytes each, zero-filled past k) go from memory straight into LDS,
//    three tiles of LDS in rotation: the multipliers read tile t + 1 into registers while they multiply tile t, and the
//    loads of tile t + 2 and t + 3 are in flight meanwhile.  A wave instruction fills eight consecutive LDS rows; the 16-byte piece a lane fetches is
//    the piece index XOR bits 1..3 of the row, so that the 16 lanes that later read one piece index of 16 consecutive rows
//    hit 16 different bank groups.
//  - waves 0..3 multiply and store.  Each owns a 64 x 64 patch as 2 x 2 tiles of v_mfma_f32_32x32x16 with the operands
//    SWAPPED: the MFMA computes the transposed tile, so a lane ends up with one row of C and, in four consecutive
//    accumulator registers, four adjacent columns of it, which narrow and pack into 8 bytes.  Stored like that, an
//    instruction would touch 32 rows with 16 bytes each (measured: 90 cycles per instruction, 41 us for S = Q.K^T of
//    192 x 512 x 512 x 64); so the narrowed tile goes through a staging patch of LDS that belongs to the wave alone (no
//    barrier) and leaves as whole 128-byte row segments, eight per instruction.  Tile t - 1 is staged and stored between
//    the MFMAs of tile t.
//
// The multiplying waves never wait for memory (they issue stores only), the fetching waves wait for loads only; one
// block-wide barrier per tile hands LDS tiles back and forth.
#include "rp_gemm.h"

#include <type_traits>

namespace rp {

constexpr int P16_BM = 128, P16_BN = 128, P16_MAXK = 64;
constexpr int P16_ROW_BYTES = 128;                                   // one LDS row: 64 16-bit values
constexpr int P16_TILE_BYTES = (P16_BM + P16_BN) * P16_ROW_BYTES;    // 32 KB: A rows, then B rows
constexpr int P16_NBUF = 3;                                          // LDS tiles in rotation

typedef __attribute__((address_space(3))) void* p16_lds_t;

template <typename T> struct p16_ops;
template <> struct p16_ops<bf16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    // two accumulators -> two bf16 in one word: adding 0x8000 carries into bit 16 exactly when the first dropped bit is set
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        return __builtin_amdgcn_perm(__float_as_uint(hi) + 0x8000u, __float_as_uint(lo) + 0x8000u, 0x07060302u);
    }
};
template <> struct p16_ops<f16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        return (uint32_t)narrow_f16_bits(lo) | ((uint32_t)narrow_f16_bits(hi) << 16);
    }
};

typedef __attribute__((ext_vector_type(4))) short p16_s16x4_t;

// half H (k values 4H .. 4H + 3 of the lane's eight) of a fragment of an operand that lies in LDS as k rows
template <int H>
__device__ __forceinline__ void p16_read_tr(s16x8_t& v, const unsigned char* p) {
    const p16_s16x4_t q = __builtin_amdgcn_ds_read_tr16_b64_v4i16((p16_s16x4_t __attribute__((address_space(3)))*)(p));
    v[4 * H + 0] = q[0]; v[4 * H + 1] = q[1]; v[4 * H + 2] = q[2]; v[4 * H + 3] = q[3];
}

// KST: k steps of 16 that are multiplied (4 for k <= 64, 2 for k <= 32); A_MC / B_MC: the operand has unit stride along
// its free index (m, n) instead of along k: it lies in LDS as 64 k rows of 128 free indices (256 bytes) whose 32-byte
// pieces are XORed with the low three bits of the k row, and its fragments are transposing reads (ds_read_b64_tr_b16);
// EDGE: m or n not whole tiles.
// BIAS: g.bias[n] is added to every row after the product has been rounded to the tensor type (the reference's two ops):
// on the 16-bit row pieces between the staging patch and memory, with the lane's eight bias values of a tile loaded
// while that tile is multiplied, one tile before its stores.
template <typename T, int KST, bool A_MC, bool B_MC, bool EDGE, bool BIAS>
__global__ void __launch_bounds__(512) gemm_pipe16_kernel(GemmArgs g, int tiles_m, int tiles_n, unsigned total) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char p16_smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const unsigned per_matrix = (unsigned)(tiles_m * tiles_n);
    unsigned first, walk_end, stride;
    resident_tile_walk(total, first, walk_end, stride);
    total = walk_end;                                               // this workgroup's tiles: first, first + stride, ... below total
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;      // strides of the free index and of k
    const long long a_span = (A_MC ? ((long long)(g.k - 1) * a_ks + g.m) : ((long long)(g.m - 1) * a_fs + g.k)) * 2;
    const long long b_span = (B_MC ? ((long long)(g.k - 1) * b_ks + g.n) : ((long long)(g.n - 1) * b_fs + g.k)) * 2;

    if (wave >= 4) {
        // ---- fetch: this wave brings rows [32p, 32p + 32) (k-contiguous operand) or k rows [16p, 16p + 16) (the other
        // layout) of A and of B for every tile; a wave instruction fills 1 KB of LDS: 8 rows, or 4 k rows ----
        const int p = wave - 4;
        uint32_t a_off[4], b_off[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int row = 8 * q + (lane >> 3);                        // row within the wave's 32
            const int piece = (lane & 7) ^ ((row >> 1) & 7);            // which 16 bytes of the global row land in this lane's LDS slot
            const int krow = 4 * q + (lane >> 4);                       // k row within the wave's 16
            const int c32 = ((lane & 15) >> 1) ^ (krow & 7);            // which 32 bytes of the global k row (its half: lane & 1)
            const int free = (c32 * 2 + (lane & 1)) * 8;
            a_off[q] = A_MC ? (16 * p + krow < g.k ? (uint32_t)(((long long)krow * a_ks + free) * 2) : BUFFER_OOB)
                            : (piece * 8 < g.k ? (uint32_t)(((long long)row * a_fs + piece * 8) * 2) : BUFFER_OOB);
            b_off[q] = B_MC ? (16 * p + krow < g.k ? (uint32_t)(((long long)krow * b_ks + free) * 2) : BUFFER_OOB)
                            : (piece * 8 < g.k ? (uint32_t)(((long long)row * b_fs + piece * 8) * 2) : BUFFER_OOB);
        }
        auto fetch = [&](unsigned id, int buf) {
            const TileOrigin t = tile_origin<P16_BM, P16_BN>(id, per_matrix, tiles_n);
            const __amdgpu_buffer_rsrc_t ra = buffer_rsrc((const uint16_t*)g.A + (long long)t.z * g.a_bs, a_span);
            const __amdgpu_buffer_rsrc_t rb = buffer_rsrc((const uint16_t*)g.B + (long long)t.z * g.b_bs, b_span);
            const int sa = A_MC ? (int)(((long long)(16 * p) * a_ks + t.m0) * 2) : (int)((long long)(t.m0 + 32 * p) * a_fs * 2);
            const int sb = B_MC ? (int)(((long long)(16 * p) * b_ks + t.n0) * 2) : (int)((long long)(t.n0 + 32 * p) * b_fs * 2);
            // (both layouts put the wave's share at the same place: 32 rows of 128 bytes = 16 k rows of 256 bytes = 4 KB)
            unsigned char* dst = p16_smem + buf * P16_TILE_BYTES + 32 * p * P16_ROW_BYTES;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (p16_lds_t)(dst + q * 1024), 16, (int)a_off[q], sa, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (p16_lds_t)(dst + P16_BM * P16_ROW_BYTES + q * 1024), 16, (int)b_off[q], sb, 0, 0);
            }
        };
        // The multipliers read tile t + 1 out of LDS while they multiply tile t, so at the barrier that starts tile t the
        // loads of tile t + 1 must have landed and the LDS tile of tile t is free again: it takes tile t + P16_NBUF.  Loads
        // return in order, so "tile x has landed" is "at most the loads of the younger fetches are outstanding" (8
        // instructions per fetch); where a fetch was skipped because the tiles ran out, the wait is for everything.
        unsigned ahead = first;
        int fbuf = 0;
#pragma unroll
        for (int i = 0; i < P16_NBUF; i++) {
            if (ahead < total) fetch(ahead, i);
            ahead += stride;
        }
        const bool full = ahead - stride < total;                      // every fetch above was issued
        if (full) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 * (P16_NBUF - 1)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                               // tile 0 is in LDS
        if (full) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 * (P16_NBUF - 2)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        for (unsigned id = first; id < total; id += stride) {
            __syncthreads();                                           // tile id + stride is in LDS; the LDS tile of tile id is free
            const bool more = ahead < total;
            if (more) fetch(ahead, fbuf);
            ahead += stride;
            fbuf = fbuf + 1 == P16_NBUF ? 0 : fbuf + 1;
            if (more) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 * (P16_NBUF - 2)) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        return;
    }

    // ---- multiply and store ----
    const int r = lane & 31, h = lane >> 5;
    const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
    // LDS byte addresses of the fragments of k step 0.  k-contiguous operand: piece 2s + h of the lane's row is at
    // base ^ (32 s) (rows are 128-byte aligned, so the XOR only touches the piece bits).  Other layout: the transposing read
    // of a 16-lane group covers 4 k rows x 16 free indices; source lane s points at free indices 4(s % 4) .. + 3 of k row
    // s / 4; the groups are (k octet, free half) = (grp / 2, grp % 2); k step s is 16 k rows further.
    const int grp = lane >> 4, s16 = lane & 15;
    uint32_t a_fr[2][2], b_fr[2][2];                                // [H][tile] (k-contiguous: only [0][tile] is used)
#pragma unroll
    for (int i = 0; i < 2; i++) {
        if (!A_MC) {
            a_fr[0][i] = (uint32_t)((wm0 + 32 * i + r) * P16_ROW_BYTES + ((h ^ ((r >> 1) & 7)) * 16));
            a_fr[1][i] = 0;
        } else {
#pragma unroll
            for (int H = 0; H < 2; H++) {
                const int krow = 8 * (grp >> 1) + 4 * H + (s16 >> 2), free = wm0 + 32 * i + 16 * (grp & 1) + 4 * (s16 & 3);
                a_fr[H][i] = (uint32_t)(krow * 256 + (((free >> 4) ^ (krow & 7)) * 32) + (free & 15) * 2);
            }
        }
        if (!B_MC) {
            b_fr[0][i] = (uint32_t)(P16_BM * P16_ROW_BYTES + (wn0 + 32 * i + r) * P16_ROW_BYTES + ((h ^ ((r >> 1) & 7)) * 16));
            b_fr[1][i] = 0;
        } else {
#pragma unroll
            for (int H = 0; H < 2; H++) {
                const int krow = 8 * (grp >> 1) + 4 * H + (s16 >> 2), free = wn0 + 32 * i + 16 * (grp & 1) + 4 * (s16 & 3);
                b_fr[H][i] = (uint32_t)(P16_BM * P16_ROW_BYTES + krow * 256 + (((free >> 4) ^ (krow & 7)) * 32) + (free & 15) * 2);
            }
        }
    }
    // The wave's own 64 x 64 staging patch (rows of 128 bytes, 16-byte pieces XORed like the operand tiles).  After the
    // swapped MFMA a lane holds row r of C and four adjacent columns per accumulator quad: 8 bytes, written at piece
    // 4 in + q, half h.  Read back, a lane holds 16 bytes of row lane / 8 (+ 8 per instruction), piece lane % 8: eight
    // whole 128-byte row segments per store instruction.
    unsigned char* stage = p16_smem + P16_NBUF * P16_TILE_BYTES + wave * (64 * P16_ROW_BYTES);
    const uint32_t st_write = (uint32_t)(r * P16_ROW_BYTES + 8 * h), st_swz = (uint32_t)((r >> 1) & 7);
    const int rr = lane >> 3, rp = lane & 7;
    const uint32_t c_lane = (uint32_t)(((long long)rr * g.c_rs + 8 * rp) * 2);
    const long long c_span = ((long long)(g.m - 1) * g.c_rs + g.n) * 2;

    f32x16_t acc[2][2];                 // [jm: rows of C][in: columns of C]
    u32x2_t packed[16];                 // the previous tile, narrowed: [jm][in][q]
    u32x4_t rows[8];                    // the previous tile's row segments on their way from the staging patch to memory
    s16x8_t af[KST][2], bf[KST][2];     // [k step][tile]: eight k values of the lane's row
    u32x4_t bias_prev = {0u, 0u, 0u, 0u}, bias_cur = {0u, 0u, 0u, 0u};      // BIAS: of columns n0 + wn0 + 8 rp .. + 7 of the tile being stored / multiplied
    auto load_bias = [&](const TileOrigin& t) {
        const int gn = t.n0 + wn0 + 8 * rp;
        bias_cur = gn < g.n ? *(const u32x4_t*)((const uint16_t*)g.bias + gn) : u32x4_t{0u, 0u, 0u, 0u};       // (n is a multiple of 8)
    };
    auto widen_lo = [](uint32_t w) { T x; x.bits = (uint16_t)w; return widen(x); };
    auto widen_hi = [](uint32_t w) { T x; x.bits = (uint16_t)(w >> 16); return widen(x); };

    auto pack_all = [&]() {
        static_for<0, 16>([&](auto nc) {
            constexpr int n = decltype(nc)::value, jm = n >> 3, in = (n >> 2) & 1, q = n & 3;
            const float v0 = acc[jm][in][4 * q], v1 = acc[jm][in][4 * q + 1], v2 = acc[jm][in][4 * q + 2], v3 = acc[jm][in][4 * q + 3];
            packed[n][0] = p16_ops<T>::pack(v0, v1);
            packed[n][1] = p16_ops<T>::pack(v2, v3);
        });
    };
    // staging write n (0..15): quad q of MFMA tile (jm, in)
    auto stage_write = [&](auto n_c) {
        constexpr int n = decltype(n_c)::value, jm = n >> 3, in = (n >> 2) & 1, q = n & 3;
        *(u32x2_t*)(stage + st_write + 32 * jm * P16_ROW_BYTES + (((uint32_t)(4 * in + q) ^ st_swz) * 16)) = packed[n];
    };
    // rows 8e .. 8e + 7 of the patch (e = 0..7): out of the staging patch (rows below 32 need staging writes 0..7 only) ...
    auto row_read = [&](auto e_c) {
        constexpr int e = decltype(e_c)::value;
        const int row = 8 * e + rr;
        rows[e] = *(const u32x4_t*)(stage + row * P16_ROW_BYTES + (((uint32_t)rp ^ (uint32_t)((row >> 1) & 7)) * 16));
        if constexpr (BIAS) {
#pragma unroll
            for (int d = 0; d < 4; d++)
                rows[e][d] = p16_ops<T>::pack(widen_lo(rows[e][d]) + widen_lo(bias_prev[d]), widen_hi(rows[e][d]) + widen_hi(bias_prev[d]));
        }
    };
    // ... and to memory
    auto row_store = [&](auto e_c, const TileOrigin& t, const __amdgpu_buffer_rsrc_t& rc) {
        constexpr int e = decltype(e_c)::value;
        const int gm = t.m0 + wm0 + 8 * e, gn = t.n0 + wn0;
        const int soff = (int)(((long long)gm * g.c_rs + gn) * 2);
        uint32_t voff = c_lane;
        if constexpr (EDGE) voff = (gm + rr < g.m && gn + 8 * rp < g.n) ? c_lane : BUFFER_OOB;      // (n is a multiple of 8: a piece is inside or outside as a whole)
        __builtin_amdgcn_raw_buffer_store_b128(rows[e], rc, (int)voff, soff, 2);          // (streaming store: the output is not read again by this kernel)
    };

    auto read_frags = [&](const unsigned char* base, auto s_c) {
        constexpr int s = decltype(s_c)::value;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if constexpr (!A_MC) af[s][i] = *(const s16x8_t*)(base + (a_fr[0][i] ^ (uint32_t)(32 * s)));
            else { p16_read_tr<0>(af[s][i], base + a_fr[0][i] + 16 * s * 256); p16_read_tr<1>(af[s][i], base + a_fr[1][i] + 16 * s * 256); }
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if constexpr (!B_MC) bf[s][j] = *(const s16x8_t*)(base + (b_fr[0][j] ^ (uint32_t)(32 * s)));
            else { p16_read_tr<0>(bf[s][j], base + b_fr[0][j] + 16 * s * 256); p16_read_tr<1>(bf[s][j], base + b_fr[1][j] + 16 * s * 256); }
        }
    };

    // One tile, whose operand pieces are already in registers: behind each k step's MFMAs the same pieces of the NEXT tile
    // are read (LDS tile `next`), so no MFMA ever waits for LDS.  If STORE, the previous tile (narrowed, in `packed`) goes
    // through the staging patch to memory meanwhile, in quarters of the MFMAs: staging writes 0..7 | writes 8..15 and row
    // reads 0..3 | row stores 0..3 and row reads 4..7 | row stores 4..7, so that no instruction waits for the one before it.
    auto tile_pass = [&](auto store_c, int next, const TileOrigin& prev) {
        constexpr bool STORE = decltype(store_c)::value;
        constexpr int NM = 4 * KST, Q = NM / 4;                    // MFMAs per tile and per quarter
        constexpr int WR = 8 / Q, RD = 4 / Q;                       // staging writes and row reads / stores per MFMA in their quarters
        const unsigned char* next_base = p16_smem + next * P16_TILE_BYTES;
        const __amdgpu_buffer_rsrc_t rc = buffer_rsrc((uint16_t*)g.C + (long long)prev.z * g.c_bs, c_span);
        __syncthreads();                                   // the next tile is in LDS; this tile's pieces have all arrived in registers
        static_for<0, KST>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            static_for<0, 4>([&](auto tc) {
                constexpr int t4 = decltype(tc)::value, jm = t4 >> 1, in = t4 & 1, mi = s * 4 + t4, phase = mi / Q, idx = mi % Q;
                // operands swapped: the MFMA's rows are columns of C
                if constexpr (s == 0) {
                    const f32x16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    acc[jm][in] = p16_ops<T>::mma(bf[s][in], af[s][jm], zero);
                } else {
                    acc[jm][in] = p16_ops<T>::mma(bf[s][in], af[s][jm], acc[jm][in]);
                }
                if constexpr (STORE) {
                    if constexpr (phase == 0) static_for<0, WR>([&](auto ec) { stage_write(std::integral_constant<int, idx * WR + decltype(ec)::value>{}); });
                    if constexpr (phase == 1) {
                        static_for<0, WR>([&](auto ec) { stage_write(std::integral_constant<int, 8 + idx * WR + decltype(ec)::value>{}); });
                        static_for<0, RD>([&](auto ec) { row_read(std::integral_constant<int, idx * RD + decltype(ec)::value>{}); });
                    }
                    if constexpr (phase == 2) {
                        static_for<0, RD>([&](auto ec) { row_store(std::integral_constant<int, idx * RD + decltype(ec)::value>{}, prev, rc); });
                        static_for<0, RD>([&](auto ec) { row_read(std::integral_constant<int, 4 + idx * RD + decltype(ec)::value>{}); });
                    }
                    if constexpr (phase == 3) static_for<0, RD>([&](auto ec) { row_store(std::integral_constant<int, 4 + idx * RD + decltype(ec)::value>{}, prev, rc); });
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            read_frags(next_base, sc);
        });
        pack_all();
    };

    __syncthreads();                                   // the first tile is in LDS
    TileOrigin prev = {0, 0, 0};
    int next = 1;                                      // LDS tile of the tile after the current one
    unsigned id = first;
    if (id >= total) return;
    static_for<0, KST>([&](auto sc) { read_frags(p16_smem, sc); });
    if constexpr (BIAS) load_bias(tile_origin<P16_BM, P16_BN>(id, per_matrix, tiles_n));
    tile_pass(std::false_type{}, next, prev);
    prev = tile_origin<P16_BM, P16_BN>(id, per_matrix, tiles_n);
    if constexpr (BIAS) bias_prev = bias_cur;
    next = next + 1 == P16_NBUF ? 0 : next + 1;
    id += stride;
    for (; id < total; id += stride) {
        if constexpr (BIAS) load_bias(tile_origin<P16_BM, P16_BN>(id, per_matrix, tiles_n));
        tile_pass(std::true_type{}, next, prev);
        prev = tile_origin<P16_BM, P16_BN>(id, per_matrix, tiles_n);
        if constexpr (BIAS) bias_prev = bias_cur;
        next = next + 1 == P16_NBUF ? 0 : next + 1;
    }
    // the last tile
    const __amdgpu_buffer_rsrc_t rc = buffer_rsrc((uint16_t*)g.C + (long long)prev.z * g.c_bs, c_span);
    static_for<0, 16>([&](auto nc) { stage_write(nc); });
    static_for<0, 8>([&](auto ec) { row_read(ec); });
    static_for<0, 8>([&](auto ec) { row_store(ec, prev, rc); });
}

// ---- host side ----

// Whether this kernel takes the product: k <= 64 in whole 16-byte pieces, both operands with a unit stride and
// 16-byte aligned rows, C row-major with 16-byte aligned rows and n in whole eights, overwritten (a bias per column,
// 16-byte aligned, is taken; no accumulation, whose extra read of C leaves the product bound by memory at the tiled
// kernel's speed; no segments or folded store), and every byte offset the kernel forms from a batch entry's base within
// the 32-bit range of buffer addressing.
bool pipe16_takes(const GemmArgs& g) {
    if (g.k > P16_MAXK || g.k < 8 || g.k % 8 || g.m < 1 || g.n < 8 || g.n % 8 || g.batch < 1) return false;
    if ((long long)((g.m + P16_BM - 1) / P16_BM) * ((g.n + P16_BN - 1) / P16_BN) * g.batch >= (1ll << 30)) return false;
    if (g.accumulate || g.seg_k || g.seg_n || g.c_fold_from || g.bias_by_row || ((uintptr_t)g.bias & 15)) return false;
    const bool a_kc = g.a_cs == 1 && g.a_rs % 8 == 0, a_mc = g.a_rs == 1 && g.a_cs % 8 == 0;
    const bool b_kc = g.b_rs == 1 && g.b_cs % 8 == 0, b_mc = g.b_cs == 1 && g.b_rs % 8 == 0;
    if (!(a_kc || a_mc) || !(b_kc || b_mc) || g.a_bs % 8 || g.b_bs % 8 || g.a_rs < 0 || g.a_cs < 0 || g.b_rs < 0 || g.b_cs < 0) return false;
    if (g.c_cs != 1 || g.c_rs % 8 || g.c_bs % 8 || g.c_rs < 0) return false;
    if (((uintptr_t)g.A & 15) || ((uintptr_t)g.B & 15) || ((uintptr_t)g.C & 15)) return false;
    const long long lim = 1ll << 30;
    // free indices up to a whole tile past the last one are addressed (and read as zero, or as values that only reach
    // outputs which are not stored)
    const long long a_reach = (a_kc ? (long long)(g.m + P16_BM) * g.a_rs + P16_MAXK : (long long)P16_MAXK * g.a_cs + g.m + P16_BM) * 2;
    const long long b_reach = (b_kc ? (long long)(g.n + P16_BN) * g.b_cs + P16_MAXK : (long long)P16_MAXK * g.b_rs + g.n + P16_BN) * 2;
    const long long c_reach = ((long long)(g.m + P16_BM) * g.c_rs + g.n + P16_BN) * 2;
    return a_reach < lim && b_reach < lim && c_reach < lim;
}

template <typename T>
static int launch_pipe16_t(const GemmArgs& g) {
    const int tiles_m = (g.m + P16_BM - 1) / P16_BM, tiles_n = (g.n + P16_BN - 1) / P16_BN;
    const long long total = (long long)tiles_m * tiles_n * g.batch;
    int cus = device_cu_count();
    if (cus <= 0) cus = 256;
    const unsigned blocks = (unsigned)(total < cus ? total : cus);          // one resident workgroup per CU walks its tiles
    const bool edge = (g.m % P16_BM) || (g.n % P16_BN);
    constexpr int smem = P16_NBUF * P16_TILE_BYTES + 4 * 64 * P16_ROW_BYTES;          // the operand tiles and a staging patch per multiplying wave
    auto launch = [&](auto kern) {
        if (!check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem), "hipFuncSetAttribute")) return -1;
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(512), smem, current_stream(), g, tiles_m, tiles_n, (unsigned)total);
        return check_launch("gemm_pipe16_kernel") ? 0 : -1;
    };
    const bool a_mc = !(g.a_cs == 1 && g.a_rs % 8 == 0), b_mc = !(g.b_rs == 1 && g.b_cs % 8 == 0);
    auto pick = [&](auto kst_c, auto bias_c) {
        constexpr int KST = decltype(kst_c)::value;
        constexpr bool BIAS = decltype(bias_c)::value;
        if (!a_mc && !b_mc) return edge ? launch(gemm_pipe16_kernel<T, KST, false, false, true, BIAS>) : launch(gemm_pipe16_kernel<T, KST, false, false, false, BIAS>);
        if (!a_mc && b_mc) return edge ? launch(gemm_pipe16_kernel<T, KST, false, true, true, BIAS>) : launch(gemm_pipe16_kernel<T, KST, false, true, false, BIAS>);
        if (a_mc && !b_mc) return edge ? launch(gemm_pipe16_kernel<T, KST, true, false, true, BIAS>) : launch(gemm_pipe16_kernel<T, KST, true, false, false, BIAS>);
        return edge ? launch(gemm_pipe16_kernel<T, KST, true, true, true, BIAS>) : launch(gemm_pipe16_kernel<T, KST, true, true, false, BIAS>);
    };
    if (g.k <= 32) return g.bias ? pick(std::integral_constant<int, 2>{}, std::true_type{}) : pick(std::integral_constant<int, 2>{}, std::false_type{});
    return g.bias ? pick(std::integral_constant<int, 4>{}, std::true_type{}) : pick(std::integral_constant<int, 4>{}, std::false_type{});
}

int launch_pipe16(const GemmArgs& g, int dtype) {
    if (dtype == RP_DTYPE_BFLOAT16) return launch_pipe16_t<bf16_t>(g);
    if (dtype == RP_DTYPE_FLOAT16) return launch_pipe16_t<f16_t>(g);
    set_error("pipe16 GEMM: 16-bit types only");
    return -1;
}

}  // namespace rp
