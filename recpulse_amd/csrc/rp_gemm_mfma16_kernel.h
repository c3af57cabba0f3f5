// bf16 / fp16 MFMA GEMM kernel template (fp32 accumulate) and its launch helper; included by the
// per-tile translation units.
#pragma once
#include "rp_gemm.h"

#include <type_traits>

namespace rp {

// ============================================================================
// mfma16: bf16 / fp16 inputs, fp32 accumulate.
//
// Block tile BM x BN, k slab 64, 256 threads = 4 waves (one per SIMD) in a
// WGM x (4/WGM) grid, each wave owning a (BM/WGM) x (BN/(4/WGM)) patch of
// 32x32x16 MFMA tiles.  With SPLITK the grid's z axis splits k: every block
// writes its fp32 partial tile to a workspace [matrix][split][m][n] and a
// combine kernel finishes.
//
// Software pipeline, per slab s (4 k-steps of 16):
//   k-steps 0-2  MFMAs on fragments(ks) | read fragments(ks+1) | a third of: registers of slab s+1 -> other
//                LDS buffer, then the global load of slab s+2 into the register just freed
//   barrier      (slab s+1 is now complete in LDS, and nobody reads this slab's buffer any more)
//   k-step 3     MFMAs on fragments(3) | read fragments(0) of slab s+1
// so LDS reads run one k-step ahead of the MFMAs that use them, global loads
// have a full slab of MFMA time to land, and the single barrier per slab sits
// where only one MFMA group is left to issue.  Every MFMA is followed by its
// share of DS / VMEM work and a scheduling barrier, which pins the interleaving.
// The 256 x 256 tile multiplies with 16x16x32 MFMAs instead (m16_mfma_tile): two
// k-steps of 32 per slab, 8 x 8 tiles per wave, the slab traffic all in the first
// k-step, one DS / VMEM instruction per MFMA, A fragments in a single slot that is
// refilled row by row.
//
// LDS layouts (16-bit elements):
//   KC operand: [rows][64 + 8]   row pitch 144 B: a ds_read_b128 whose lanes hold row lane % 32, k octet lane / 32
//               (32 x 32 tiles) runs at the full rate of one instruction per 16 cycles and wave.  With 16 x 16 tiles
//               (row lane % 16, octet lane / 16) that pitch takes twice as long (measured: 32 cycles); 160 B does not.
//   MC operand: [64][cols + 32]  row pitch 2*cols + 64 B -> the 4 k-rows a
//               16-lane group reads with ds_read_b64_tr_b16 start 16 banks apart
// The epilogue narrows the accumulators, stages them through the (now idle) LDS
// and stores 8 adjacent columns per lane with one 16-byte store.
// ============================================================================
template <typename T> struct mfma16_ops;
template <> struct mfma16_ops<bf16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    // 16 x 16 x 32, accumulating in place.  Written as an instruction with the accumulator tied to the result: through the
    // builtin the register allocator gives the result another register than the accumulator it came from and moves all
    // 256 accumulator registers around the loop (three copies per MFMA).
    static __device__ __forceinline__ f32x4_t mma(s16x8_t a, s16x8_t b, f32x4_t c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
        return c;
    }
};
template <> struct mfma16_ops<f16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t mma(s16x8_t a, s16x8_t b, f32x4_t c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
        return c;
    }
};

// MFMA shape of a block tile: the 256 x 256 tile multiplies with 16 x 16 x 32 (k-steps of 32), the others with 32 x 32 x 16.
// Both run 512 multiply-adds per cycle, but the deeper instruction moves fewer register bytes per multiply-add
// (2 KB of operands and 2 KB of accumulators per 8 192 against 2 KB and 8 KB per 16 384), and under the power limit
// that governs a large GEMM the chip sustains a higher clock on it: a loop of nothing but MFMAs on N(0,1) operands
// measured 1.84 PFLOP/s at 2.16 GHz against 1.65 PFLOP/s at 1.83 GHz.
__host__ __device__ constexpr int m16_mfma_tile(int bm, int bn) { return (bm == 256 && bn == 256) ? 16 : 32; }

__host__ __device__ constexpr int m16_kc_pitch(int mt) { return mt == 16 ? M16_BK + 16 : M16_BK + 8; }    // elements, by MFMA tile edge
__host__ __device__ constexpr int m16_mc_pitch(int cols) { return cols + 32; }
__host__ __device__ constexpr int m16_tile_elems(int rows, bool mc, int mt) {
    return mc ? M16_BK * m16_mc_pitch(rows) : rows * m16_kc_pitch(mt);
}
__host__ __device__ constexpr int m16_epi_cols(int wn) { return wn >= 64 ? 64 : wn; }      // columns staged per epilogue pass
// `stages` is 2, or 1 when k fits a single slab (the loop then never touches the second stage), which lets twice
// as many blocks of a short-k batched GEMM share a CU and overlap their load, multiply and store phases.
__host__ __device__ constexpr size_t m16_smem_bytes(int bm, int bn, int wgm, bool a_mc, bool b_mc, int stages, int mt) {
    size_t loop = stages * (size_t)(m16_tile_elems(bm, a_mc, mt) + m16_tile_elems(bn, b_mc, mt)) * 2;
    size_t epi = 4 * (size_t)(bm / wgm) * (m16_epi_cols(bn / (4 / wgm)) + 4) * 4;      // split-k: fp32, 64 columns per pass
    size_t epi16 = 4 * (size_t)(bm / wgm) * (bn / (4 / wgm) + 8) * 2;                  // otherwise: the whole patch as 16-bit values
    if (epi16 > epi) epi = epi16;
    return loop > epi ? loop : epi;
}

typedef uint16_t __attribute__((address_space(3))) lds_u16;



// Per-thread constants of one operand's slab traffic: NL 16-byte pieces per slab; piece i sits a fixed
// number of rows (KC) or k-rows (MC) after piece 0, so LDS offsets are piece 0's plus a compile-time step.
template <int ROWS, bool MC, int MT>
struct SlabMap {
    static constexpr int KCP = m16_kc_pitch(MT);
    static constexpr int NL = ROWS * 8 / 256;
    static constexpr int PIECE_ROWS = MC ? 256 / (ROWS / 8) : 32;        // k-rows (MC) or free rows (KC) between consecutive pieces
    static constexpr int LDS_STEP = MC ? PIECE_ROWS * m16_mc_pitch(ROWS) : PIECE_ROWS * KCP;   // elements
    // piece 0 of thread t: free index r (first of 8 for MC) and slab-local k (first of 8 for KC)
    static __device__ __forceinline__ void coords0(int t, int& r, int& kk) {
        if (MC) { kk = t / (ROWS / 8); r = (t % (ROWS / 8)) * 8; }
        else    { r = t / 8; kk = (t % 8) * 8; }
    }
    static __device__ __forceinline__ int lds_off(int r, int kk) {          // element offset inside the operand's LDS tile
        return MC ? kk * m16_mc_pitch(ROWS) + r : r * KCP + kk;
    }
};

// Lane's base element offset for MFMA fragments of an operand tile whose wave patch starts at free index w0.
// Fragment (tile i, k-step ks, read h) then sits at base + step(i, ks, h), a compile-time constant.
// MT: the MFMA's tile edge, 32 (k-step 16: a lane holds free index lane % 32, k octet lane / 32) or 16 (k-step 32:
// free index lane % 16, k octet lane / 16).
template <int ROWS, bool MC, int MT>
struct FragMap {
    static constexpr int KSTEP = MT == 32 ? 16 : 32;
    static constexpr int KCP = m16_kc_pitch(MT);
    static __device__ __forceinline__ int base(int w0, int lane) {
        if (!MC) return (w0 + (lane % MT)) * KCP + (lane / MT) * 8;
        // ds_read_b64_tr_b16: inside each 16-lane group, source lane s points at 4 consecutive free
        // indices of k-row s/4; destination lane j receives free index j of k-rows 0..3.
        int grp = lane >> 4, s = lane & 15;
        if (MT == 32) return (8 * (grp >> 1) + (s >> 2)) * m16_mc_pitch(ROWS) + w0 + 16 * (grp & 1) + 4 * (s & 3);
        return (8 * grp + (s >> 2)) * m16_mc_pitch(ROWS) + w0 + 4 * (s & 3);          // the four groups are the four k octets of the same 16 free indices
    }
    static constexpr int READS = MC ? 2 : 1;                 // DS instructions per fragment
    static constexpr int step(int i, int ks, int h) {
        return MC ? ks * KSTEP * m16_mc_pitch(ROWS) + i * MT + h * 4 * m16_mc_pitch(ROWS)
                  : i * MT * KCP + ks * KSTEP;
    }
    // DS read H of the fragment into v (KC: the whole fragment; MC: k values 4H .. 4H+3)
    template <int H>
    static __device__ __forceinline__ void read(s16x8_t& v, const uint16_t* p) {
        if constexpr (!MC) {
            v = *(const s16x8_t*)p;
        } else {
            s16x4_t q = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(lds_u16*)p);
            v[4 * H + 0] = q[0]; v[4 * H + 1] = q[1]; v[4 * H + 2] = q[2]; v[4 * H + 3] = q[3];
        }
    }
};

template <typename T, int BM, int BN, int WGM, bool A_MC, bool B_MC, bool EDGE, bool SPLITK>
__global__ void __launch_bounds__(256) gemm_mfma16_kernel(GemmArgs g, int tiles_m, int tiles_n, float* partials, int k_per_split, int sched_total) {
    constexpr int WGN = 4 / WGM;
    constexpr int WM = BM / WGM, WN = BN / WGN;       // wave patch
    constexpr int MT = SPLITK ? 32 : m16_mfma_tile(BM, BN);      // MFMA tile edge; k-steps of 16 (MT 32) or 32 (MT 16)
    constexpr int NKS = MT == 32 ? 4 : 2;             // k-steps per slab
    constexpr int NV = MT == 32 ? 16 : 4;             // accumulator registers per MFMA tile
    using acc_t = std::conditional_t<MT == 32, f32x16_t, f32x4_t>;
    constexpr int TMI = WM / MT, TNI = WN / MT;       // MFMA tiles per wave
    constexpr int A_ELEMS = m16_tile_elems(BM, A_MC, MT), B_ELEMS = m16_tile_elems(BN, B_MC, MT);
    constexpr int STAGE = A_ELEMS + B_ELEMS;          // stage s: A at smem + s*STAGE, B right after it
    using MapA = SlabMap<BM, A_MC, MT>;
    using MapB = SlabMap<BN, B_MC, MT>;
    using FragA = FragMap<BM, A_MC, MT>;
    using FragB = FragMap<BN, B_MC, MT>;
    constexpr int NA = MapA::NL, NB = MapB::NL;
    constexpr int RD_A = TMI * FragA::READS, RD_B = TNI * FragB::READS;      // DS read instructions per k-step
    constexpr int NMFMA = TMI * TNI;
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

    int first_slot, z;
    batched_block(tiles_m, tiles_n, first_slot, z);
    // A workgroup walks the schedule with the grid's stride.  The launcher starts one workgroup per slot of the schedule,
    // except for the 256 x 256 tile, which fills a CU by itself: there one workgroup per CU stays resident and takes its
    // tiles one after the other, so that a tile's output stores drain, and the next tile's first loads fly, while MFMAs
    // run; a workgroup per tile would hold the CU idle until its last store was acknowledged.  A stride that is a
    // multiple of 8 keeps a workgroup's tiles on the XCD the schedule assigned them to.
    for (int tile_id = first_slot; tile_id < sched_total; tile_id += gridDim.x) {
    TileCoord tc = schedule_tile(tile_id, tiles_m, tiles_n);
    if (!tc.valid) continue;
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    // k range of this block: all of k, or the z-th split of it
    const int kbeg = SPLITK ? blockIdx.z * k_per_split : 0;
    const int kend = SPLITK ? (kbeg + k_per_split < g.k ? kbeg + k_per_split : g.k) : g.k;

    // A: free axis = m (stride a_rs), k stride a_cs.  B: free axis = n (stride b_cs), k stride b_rs.
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;
    const uint16_t* a_mat = (const uint16_t*)g.A + (long long)z * g.a_bs;
    const uint16_t* b_mat = (const uint16_t*)g.B + (long long)z * g.b_bs;
    // uniform pointers to the tile's current slab and one past the operand's last valid element
    const char* a_slab = (const char*)(a_mat + (long long)m0 * a_fs + (long long)kbeg * a_ks);
    const bool n_segmented = !B_MC && g.seg_n > 0;           // B's columns are a list of segments: offsets are taken from B itself, not from the tile
    const char* b_slab = (const char*)(b_mat + (n_segmented ? 0ll : (long long)n0 * b_fs) + (long long)kbeg * b_ks);
    const char* a_end = (const char*)(a_mat + ((long long)(g.m - 1) * a_fs + (long long)(kend - 1) * a_ks + 1));
    const int seg_slabs = g.seg_k / M16_BK;
    const bool segmented = seg_slabs > 0;                 // B's k axis is a list of segments (never together with SPLITK)
    const char* b_end = (segmented || n_segmented) ? (const char*)(b_mat + g.b_extent)
                                  : (const char*)(b_mat + ((long long)(g.n - 1) * b_fs + (long long)(kend - 1) * b_ks + 1));
    const long long a_step = (long long)M16_BK * a_ks * 2, b_step = (long long)M16_BK * b_ks * 2;
    // From the last slab of a segment the pointer goes back to the segment's start and on to the next one's: one
    // step along seg_sw, or, after the seg_w-th segment of a row, to the start of the next row of segments.
    const long long seg_next = segmented ? g.seg_sw * 2 - (long long)(seg_slabs - 1) * b_step : b_step;
    const long long seg_wrap = segmented ? (g.seg_sh - (long long)g.seg_w * g.seg_sw) * 2 : 0;
    int seg_left = segmented ? seg_slabs : 0x7fffffff, seg_col = 0;
    auto advance_b = [&]() {
        if (--seg_left == 0) {
            seg_left = seg_slabs;
            b_slab += seg_next;
            if (++seg_col == g.seg_w) { seg_col = 0; b_slab += seg_wrap; }
        } else {
            b_slab += b_step;
        }
    };

    // Per-thread piece offsets (bytes from the slab pointer).  The buffer descriptor ends at the operand's last
    // element, which zero-fills rows past the free extent (KC) or k past the end (MC); the other axis of each
    // layout is masked explicitly by swapping in an offset no descriptor covers.
    uint32_t a_goff[NA], b_goff[NB];
    int a_r0, a_kk0, b_r0, b_kk0;
    MapA::coords0(t, a_r0, a_kk0);
    MapB::coords0(t, b_r0, b_kk0);
#pragma unroll
    for (int i = 0; i < NA; i++) {
        int r = a_r0 + (A_MC ? 0 : i * MapA::PIECE_ROWS), kk = a_kk0 + (A_MC ? i * MapA::PIECE_ROWS : 0);
        a_goff[i] = (uint32_t)(((long long)r * a_fs + (long long)kk * a_ks) * 2);
        if (EDGE && A_MC && m0 + r >= g.m) a_goff[i] = BUFFER_OOB;
    }
#pragma unroll
    for (int i = 0; i < NB; i++) {
        int r = b_r0 + (B_MC ? 0 : i * MapB::PIECE_ROWS), kk = b_kk0 + (B_MC ? i * MapB::PIECE_ROWS : 0);
        b_goff[i] = (uint32_t)(((long long)r * b_fs + (long long)kk * b_ks) * 2);
        if (EDGE && B_MC && n0 + r >= g.n) b_goff[i] = BUFFER_OOB;
        if (n_segmented) {
            const int j = n0 + r, seg = j / g.seg_n, c = j - seg * g.seg_n;
            const long long at = (long long)(seg / g.seg_w) * g.seg_sh + (long long)(seg % g.seg_w) * g.seg_sw + (long long)c * b_fs + (long long)kk * b_ks;
            b_goff[i] = (EDGE && j >= g.n) ? BUFFER_OOB : (uint32_t)(at * 2);        // the descriptor's end no longer stands for "past the last column"
        }
    }
    const int a_wr0 = MapA::lds_off(a_r0, a_kk0), b_wr0 = A_ELEMS + MapB::lds_off(b_r0, b_kk0);     // LDS element offsets of piece 0
    const int a_fr0 = FragA::base(wm0, lane), b_fr0 = A_ELEMS + FragB::base(wn0, lane);

    acc_t acc[TMI][TNI];
#pragma unroll
    for (int i = 0; i < TMI; i++)
#pragma unroll
        for (int j = 0; j < TNI; j++)
#pragma unroll
            for (int v = 0; v < NV; v++) acc[i][j][v] = 0.f;

    u32x4_t ra[NA], rb[NB];
    const int nslabs = (kend - kbeg + M16_BK - 1) / M16_BK;
    __amdgpu_buffer_rsrc_t a_rsrc, b_rsrc;
    int kleft = 0;        // k still in range counted from the slab the descriptors point at (EDGE, KC operands)

    auto point_at_slab = [&](int k0) {
        a_rsrc = buffer_rsrc(a_slab, EDGE ? (long long)(a_end - a_slab) : 0x7fffffffll);
        b_rsrc = buffer_rsrc(b_slab, EDGE ? (long long)(b_end - b_slab) : 0x7fffffffll);
        kleft = kend - kbeg - k0;
    };
    // Without edges piece i sits a uniform number of bytes after piece 0: one lane offset per operand plus a scalar
    // offset per piece, instead of a register per piece.
    const int a_piece_step = (int)((long long)MapA::PIECE_ROWS * (A_MC ? a_ks : a_fs) * 2);
    const int b_piece_step = (int)((long long)MapB::PIECE_ROWS * (B_MC ? b_ks : b_fs) * 2);
    auto load_piece_a = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (!EDGE) {
            ra[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)a_goff[0], i * a_piece_step, 0);
        } else {
            uint32_t off = a_goff[i];
            if (!A_MC && a_kk0 >= kleft) off = BUFFER_OOB;
            ra[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (int)off, 0, 0);
        }
    };
    auto load_piece_b = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (!EDGE) {
            rb[i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, n_segmented ? (int)b_goff[i] : (int)b_goff[0], n_segmented ? 0 : i * b_piece_step, 0);
        } else {
            uint32_t off = b_goff[i];
            if (!B_MC && b_kk0 >= kleft) off = BUFFER_OOB;
            rb[i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, (int)off, 0, 0);
        }
    };
    auto store_piece_a = [&](uint16_t* stage, auto ic) {
        constexpr int i = decltype(ic)::value;
        *(u32x4_t*)(stage + a_wr0 + i * MapA::LDS_STEP) = ra[i];
    };
    auto store_piece_b = [&](uint16_t* stage, auto ic) {
        constexpr int i = decltype(ic)::value;
        *(u32x4_t*)(stage + b_wr0 + i * MapB::LDS_STEP) = rb[i];
    };

    // B fragments have two slots (the next k-step's are read while this one's are multiplied).  With 32 x 32 tiles
    // so have A's.  With 16 x 16 tiles (8 x 8 of them per wave) that would be 128 registers: A's have ONE slot, and
    // since the MFMAs run A-tile-major, tile i's register is refilled for the next k-step as soon as its row of MFMAs
    // has been issued.
    constexpr int A_SLOTS = MT == 32 ? 2 : 1;
    s16x8_t af[A_SLOTS][TMI], bf[2][TNI];
    // DS read number r (0 .. RD_A+RD_B-1) of the fragments for k-step KS into fragment slot SLOT
    auto read_item = [&](const uint16_t* stage, auto ksc, auto slotc, auto rc) {
        constexpr int KS = decltype(ksc)::value, SLOT = decltype(slotc)::value, r = decltype(rc)::value;
        if constexpr (r < RD_A) {
            constexpr int i = r / FragA::READS, h = r % FragA::READS;
            FragA::template read<h>(af[SLOT % A_SLOTS][i], stage + a_fr0 + FragA::step(i, KS, h));
        } else {
            constexpr int q = r - RD_A, j = q / FragB::READS, h = q % FragB::READS;
            FragB::template read<h>(bf[SLOT][j], stage + b_fr0 + FragB::step(j, KS, h));
        }
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;

    // ---- prologue: slab 0 into LDS buffer 0, slab 1 into registers, fragments(0) of slab 0 ----
    point_at_slab(0);
    static_for<0, NA>([&](auto ic) { load_piece_a(ic); });
    static_for<0, NB>([&](auto ic) { load_piece_b(ic); });
    if (tile_id != first_slot) __syncthreads();            // the previous tile's epilogue has read its staged rows out of LDS
    static_for<0, NA>([&](auto ic) { store_piece_a(smem, ic); });
    static_for<0, NB>([&](auto ic) { store_piece_b(smem, ic); });
    a_slab += a_step;
    advance_b();
    if (nslabs > 1) {
        point_at_slab(M16_BK);
        static_for<0, NA>([&](auto ic) { load_piece_a(ic); });
        static_for<0, NB>([&](auto ic) { load_piece_b(ic); });
    }
    a_slab += a_step;
    advance_b();
    __syncthreads();
    static_for<0, RD_A + RD_B>([&](auto rc) { read_item(smem, I0{}, I0{}, rc); });

    // Pieces of both operands in one list: 0 .. NA-1 are A's, NA .. NA+NB-1 are B's.
    auto store_piece = [&](uint16_t* stage, auto pc) {
        constexpr int p = decltype(pc)::value;
        if constexpr (p < NA) store_piece_a(stage, std::integral_constant<int, p>{});
        else store_piece_b(stage, std::integral_constant<int, p - NA>{});
    };
    auto load_piece = [&](auto pc) {
        constexpr int p = decltype(pc)::value;
        if constexpr (p < NA) load_piece_a(std::integral_constant<int, p>{});
        else load_piece_b(std::integral_constant<int, p - NA>{});
    };

    // One k-step: NMFMA micro-steps, each one MFMA on fragment slot MSLOT followed by its share of the side
    // work: fragment reads for k-step RKS into the other slot, and pieces [P0, P1) of slab traffic (LDS store of
    // the registers holding slab s+1 when WR, then the global load of slab s+2 into the same registers when LD).
    // A scheduling barrier closes every micro-step so the interleaving is the one written.
    auto kstep = [&](auto mslotc, auto rksc, auto readc, auto p0c, auto p1c, auto wrc, auto ldc,
                     const uint16_t* rd_stage, uint16_t* wr_stage) {
        constexpr int MSLOT = decltype(mslotc)::value;
        constexpr bool DO_READ = decltype(readc)::value, WR = decltype(wrc)::value, LD = decltype(ldc)::value;
        constexpr int P0 = decltype(p0c)::value, NP = decltype(p1c)::value - P0;
        constexpr int NR = DO_READ ? RD_A + RD_B : 0;
        static_for<0, NMFMA>([&](auto qc) {
            constexpr int q = decltype(qc)::value, i = q / TNI, j = q % TNI;
            acc[i][j] = mfma16_ops<T>::mma(af[MSLOT % A_SLOTS][i], bf[MSLOT][j], acc[i][j]);
            if constexpr (A_SLOTS == 2) {
                static_for<(NR * q) / NMFMA, (NR * (q + 1)) / NMFMA>([&](auto rc) {
                    read_item(rd_stage, rksc, std::integral_constant<int, MSLOT ^ 1>{}, rc);
                });
            } else {
                // 16 x 16 x 32: an MFMA lasts 16 cycles, about what one LDS or buffer instruction takes to issue, so a
                // micro-step carries at most one of them (two at a row's end).  Row i of MFMAs (j = 0 .. 7): B reads at
                // j = 0, 2; LDS stores of pieces 2i, 2i+1 at j = 1, 3; the loads that refill those registers at
                // j = 4, 5; A tile i's read for the next k-step after the row's last MFMA, j = 7.
                static_assert(TNI == 8 && TMI == 8, "the 16 x 16 x 32 schedule is written for 8 x 8 tiles per wave");
                constexpr int BPR = RD_B / TMI;                       // B reads per row: 1 or 2
                constexpr int PPR = (NP + TMI - 1) / TMI;             // pieces per row (all of the slab's traffic sits in one k-step): 2
                static_assert(BPR <= 2 && PPR <= 2, "row schedule");
                if constexpr (DO_READ) {
                    if constexpr (j == 0) read_item(rd_stage, rksc, std::integral_constant<int, MSLOT ^ 1>{}, std::integral_constant<int, RD_A + i * BPR>{});
                    if constexpr (j == 2 && BPR == 2) read_item(rd_stage, rksc, std::integral_constant<int, MSLOT ^ 1>{}, std::integral_constant<int, RD_A + i * BPR + 1>{});
                    if constexpr (j == TNI - 1) {
                        static_for<i * FragA::READS, (i + 1) * FragA::READS>([&](auto rc) {
                            read_item(rd_stage, rksc, std::integral_constant<int, MSLOT ^ 1>{}, rc);
                        });
                    }
                }
                if constexpr (j == 1 || j == 3) {
                    constexpr int p = P0 + i * PPR + (j == 3 ? 1 : 0);
                    if constexpr (WR && (j == 1 || PPR == 2) && p < P0 + NP) store_piece(wr_stage, std::integral_constant<int, p>{});
                }
                if constexpr (j == 4 || j == 5) {
                    constexpr int p = P0 + i * PPR + (j == 5 ? 1 : 0);
                    if constexpr (LD && (j == 4 || PPR == 2) && p < P0 + NP) load_piece(std::integral_constant<int, p>{});
                }
            }
            if constexpr (A_SLOTS == 1) {
                // (slab traffic placed above)
            } else if constexpr (NMFMA >= 4) {
                // a piece's LDS store and the global load that refills its register go to neighbouring micro-steps,
                // so no MFMA has both (and a fragment read) to wait behind
                constexpr int D = NMFMA - 1;
                if constexpr (q < D) {
                    static_for<P0 + (NP * q) / D, P0 + (NP * (q + 1)) / D>([&](auto pc) {
                        if constexpr (WR) store_piece(wr_stage, pc);
                    });
                }
                if constexpr (q > 0) {
                    static_for<P0 + (NP * (q - 1)) / D, P0 + (NP * q) / D>([&](auto pc) {
                        if constexpr (LD) load_piece(pc);
                    });
                }
            } else {
                static_for<P0 + (NP * q) / NMFMA, P0 + (NP * (q + 1)) / NMFMA>([&](auto pc) {
                    if constexpr (WR) store_piece(wr_stage, pc);
                    if constexpr (LD) load_piece(pc);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    int cur = 0;
    // Slab traffic is spread over the three k-steps that precede the barrier.
    constexpr int NP_ALL = NA + NB, CUT1 = (NP_ALL + 2) / 3, CUT2 = (2 * NP_ALL + 2) / 3;
    // One slab of the pipeline.  NEXT: slab s+1 exists (its registers are written to LDS here and the barrier runs);
    // NEXT2: slab s+2 exists (its global loads are issued here).
    auto slab_step = [&](int s, auto next_tag, auto next2_tag) {
        constexpr bool NEXT = decltype(next_tag)::value;
        using C0 = std::integral_constant<int, 0>;
        using C1 = std::integral_constant<int, CUT1>;
        using C2 = std::integral_constant<int, CUT2>;
        using C3 = std::integral_constant<int, NP_ALL>;
        const uint16_t* stage = smem + cur * STAGE;
        uint16_t* other = smem + (cur ^ 1) * STAGE;
        if constexpr (decltype(next2_tag)::value) point_at_slab((s + 2) * M16_BK);
        if constexpr (NKS == 4) {
            kstep(I0{}, I1{}, std::true_type{}, C0{}, C1{}, next_tag, next2_tag, stage, other);
            kstep(I1{}, I2{}, std::true_type{}, C1{}, C2{}, next_tag, next2_tag, stage, other);
            kstep(I0{}, I3{}, std::true_type{}, C2{}, C3{}, next_tag, next2_tag, stage, other);
        } else {
            // two k-steps of 32: the first carries all of the slab traffic (it is as long as two of the others)
            kstep(I0{}, I1{}, std::true_type{}, C0{}, C3{}, next_tag, next2_tag, stage, other);
        }
        if constexpr (NEXT) __syncthreads();
        kstep(I1{}, I0{}, next_tag, C0{}, C0{}, std::false_type{}, std::false_type{}, other, other);
        a_slab += a_step;
        advance_b();
        cur ^= 1;
    };

    using yes = std::true_type;
    using no = std::false_type;
    int s = 0;
    for (; s + 2 < nslabs; s++) slab_step(s, yes{}, yes{});
    if (s + 1 < nslabs) { slab_step(s, yes{}, no{}); s++; }
    slab_step(s, no{}, no{});

    if constexpr (MT == 16) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");      // the in-place MFMAs above are opaque to the compiler: let the last ones drain before their results are read
    // ---- epilogue ----
    T* C = (T*)g.C + (long long)z * g.c_bs;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    if constexpr (!SPLITK) {
        // Each lane narrows its accumulators (and adds the bias of its column) first, then the wave's whole patch
        // goes through its private LDS region as 16-bit values, so that every lane stores 8 adjacent columns of one
        // output row with one 16-byte store and the read side has no arithmetic left unless C is accumulated into.
        constexpr int EP = WN + 8;                       // 16-bit elements per staged row (16-byte aligned pitch)
        constexpr int LPR = WN / 8, RPS = 64 / LPR;      // lanes per row, rows per step
        uint16_t* region = smem + wave * (WM * EP);
        const bool c_vec = (g.c_cs == 1) && (g.c_rs % 8 == 0) && (((uintptr_t)C & 15) == 0);
        __syncthreads();                                 // every wave is done with the main loop's LDS
        // (compile-time tile indices: a loop that the compiler declines to unroll would index the accumulators at run
        // time and move all of them to scratch memory for the whole kernel)
        static_for<0, TNI>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int col = j * MT + (lane % MT), gnl = n0 + wn0 + col;
            const bool by_row = g.bias_by_row != 0;
            const float bcol = (has_bias && !by_row && (!EDGE || gnl < g.n)) ? widen(bias[gnl]) : 0.f;
            auto stage = [&](auto with_bias, auto row_bias) {
                if constexpr (std::is_same<T, f16_t>::value && !decltype(with_bias)::value) {
                    // fp16 without a bias: when every value of this column of tiles narrows to a normal number (one
                    // unsigned maximum per value to find out, wave-uniform), the two-instruction narrowing is exact
                    uint32_t worst = 0;
                    static_for<0, TMI * NV>([&](auto ivc) {
                        constexpr int i = decltype(ivc)::value / NV, v = decltype(ivc)::value % NV;
                        const uint32_t key = f16_range_key(acc[i][j][v]);
                        worst = key > worst ? key : worst;
                    });
                    if (__builtin_amdgcn_ballot_w64(worst >= F16_NORMAL_SPAN) == 0) {
                        static_for<0, TMI * NV>([&](auto ivc) {
                            constexpr int i = decltype(ivc)::value / NV, v = decltype(ivc)::value % NV;
                            const int row = MT == 32 ? i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4) : i * 16 + 4 * (lane >> 4) + v;
                            region[row * EP + col] = narrow_f16_normal_bits(acc[i][j][v]);
                        });
                        return;
                    }
                }
                static_for<0, TMI * NV>([&](auto ivc) {
                    {
                        constexpr int i = decltype(ivc)::value / NV, v = decltype(ivc)::value % NV;
                        // accumulator register v: 32 x 32 tiles hold rows 8 * (v / 4) + 4 * (lane / 32) + v % 4, 16 x 16 tiles rows 4 * (lane / 16) + v
                        const int row = MT == 32 ? i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4) : i * 16 + 4 * (lane >> 4) + v;
                        T y = narrow<T>(acc[i][j][v]);
                        if constexpr (decltype(row_bias)::value) {
                            const int gmr = m0 + wm0 + row;
                            y = narrow<T>(widen(y) + ((!EDGE || gmr < g.m) ? widen(bias[gmr]) : 0.f));
                        } else if constexpr (decltype(with_bias)::value) {
                            y = narrow<T>(widen(y) + bcol);
                        }
                        region[row * EP + col] = y.bits;
                    }
                });
            };
            if (has_bias && by_row) stage(std::true_type{}, std::true_type{});
            else if (has_bias) stage(std::true_type{}, std::false_type{});
            else stage(std::false_type{}, std::false_type{});
        });
        __syncthreads();
        const int ecol = (lane % LPR) * 8, erow = lane / LPR;
        const int gn = n0 + wn0 + ecol;
        // folded output: this lane's 8 columns keep their place inside a run of c_fold_from columns, the runs
        // move together to c_fold_to columns each, and the columns past c_fold_to of a run are not stored
        int gn_out = gn;
        bool live = true;
        if (g.c_fold_from > 0) {
            const int run = gn / g.c_fold_from, within = gn - run * g.c_fold_from;
            live = within < g.c_fold_to;
            gn_out = run * g.c_fold_to + within;
        }
#pragma unroll 4
        for (int r = erow; r < WM; r += RPS) {
            const int gm = m0 + wm0 + r;
            if (EDGE && gm >= g.m) break;
            const u32x4_t staged = *(const u32x4_t*)(region + r * EP + ecol);
            T* crow = C + (long long)gm * g.c_rs;
            if (c_vec && (!EDGE || gn + 8 <= g.n)) {
                if (!live) continue;
                u32x4_t o = staged;
                if (accum) {
                    T y[8], old[8], out[8];
                    const u32x4_t was = *(const u32x4_t*)(crow + gn_out);
                    memcpy(y, &staged, 16);
                    memcpy(old, &was, 16);
#pragma unroll
                    for (int e = 0; e < 8; e++) out[e] = narrow<T>(widen(old[e]) + widen(y[e]));
                    memcpy(&o, out, 16);
                }
                __builtin_nontemporal_store(o, (u32x4_t*)(crow + gn_out));  // written once, never re-read: keep it out of the way of the operand panels in L2
            } else {
                T y[8];
                memcpy(y, &staged, 16);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    if (EDGE && gn + e >= g.n) break;
                    T* pc = crow + (long long)(gn + e) * g.c_cs;
                    *pc = accum ? narrow<T>(widen(*pc) + widen(y[e])) : y[e];
                }
            }
        }
    } else {
        // Split-k: fp32 partial tiles [split][m][n].  Pass p covers CN columns of every wave's patch: accumulators go
        // to the wave's private fp32 LDS region [WM][CN + 4]; then each lane stores 8 adjacent columns of one row.
        constexpr int CN = m16_epi_cols(WN), EP = CN + 4, TJ = CN / 32, PASSES = WN / CN;
        constexpr int LPR = CN / 8;                 // lanes per row
        constexpr int RPS = 64 / LPR;               // rows per step
        float* region = (float*)smem + wave * (WM * EP);
        const int ecol = (lane % LPR) * 8, erow = lane / LPR;
#pragma unroll
        for (int p = 0; p < PASSES; p++) {
            __syncthreads();                        // main loop (or the previous pass) is done with LDS
#pragma unroll
            for (int i = 0; i < TMI; i++)
#pragma unroll
                for (int jj = 0; jj < TJ; jj++)
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        int row = i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                        region[row * EP + jj * 32 + (lane & 31)] = acc[i][p * TJ + jj][v];
                    }
            __syncthreads();
            const int gn = n0 + wn0 + p * CN + ecol;
#pragma unroll 2
            for (int r = erow; r < WM; r += RPS) {
                const int gm = m0 + wm0 + r;
                if (EDGE && gm >= g.m) break;
                // n is a multiple of 8 on this path, so the 8 columns are all in or all out
                if (!EDGE || gn + 8 <= g.n) {
                    float* prow = partials + (((long long)z * gridDim.z + blockIdx.z) * g.m + gm) * g.n + gn;
                    *(f32x4_t*)prow = *(const f32x4_t*)(region + r * EP + ecol);
                    *(f32x4_t*)(prow + 4) = *(const f32x4_t*)(region + r * EP + ecol + 4);
                }
            }
        }
    }
    }   // tiles of this workgroup
}

// Launch one instantiation.  nsplit > 1 selects the split-k variant: partials must hold batch * nsplit * m * n floats.
template <typename T, int BM, int BN, int WGM, bool A_MC, bool B_MC, bool EDGE, bool SPLITK>
static int m16_launch(const GemmArgs& g, float* partials, int nsplit, int k_per_split) {
    int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    const int sched_total = scheduled_grid(tiles_m, tiles_n);
    int blocks = sched_total;
    if (BM == 256 && BN == 256 && !SPLITK && g.batch == 1) {
        // one resident workgroup per CU (rounded down to whole rounds of the 8 XCDs)
        const int cus = device_cu_count() / 8 * 8;
        if (cus >= 8 && blocks > cus) blocks = cus;
    }
    dim3 grid(blocks, g.batch, SPLITK ? nsplit : 1);
    size_t smem = m16_smem_bytes(BM, BN, WGM, A_MC, B_MC, (!SPLITK && g.k <= M16_BK) ? 1 : 2, SPLITK ? 32 : m16_mfma_tile(BM, BN));
    auto kern = gemm_mfma16_kernel<T, BM, BN, WGM, A_MC, B_MC, EDGE, SPLITK>;
    if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, current_stream(), g, tiles_m, tiles_n, partials, k_per_split, sched_total);
    return check_launch("gemm_mfma16_kernel") ? 0 : -1;
}

// Layout and edge dispatch for one tile shape (no split-k).
template <typename T, int BM, int BN, int WGM>
static int m16_launch_tile(const GemmArgs& g, const Plan& p) {
    if (p.edge) {
        if (!p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, false, true, true, false>(g, nullptr, 1, 0);
        if (!p.a_mc && !p.b_mc) return m16_launch<T, BM, BN, WGM, false, false, true, false>(g, nullptr, 1, 0);
        if (p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, true, true, true, false>(g, nullptr, 1, 0);
        return m16_launch<T, BM, BN, WGM, true, false, true, false>(g, nullptr, 1, 0);
    }
    if (!p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, false, true, false, false>(g, nullptr, 1, 0);
    if (!p.a_mc && !p.b_mc) return m16_launch<T, BM, BN, WGM, false, false, false, false>(g, nullptr, 1, 0);
    if (p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, true, true, false, false>(g, nullptr, 1, 0);
    return m16_launch<T, BM, BN, WGM, true, false, false, false>(g, nullptr, 1, 0);
}

template <int BM, int BN, int WGM>
static int m16_launch_tile_dtype(const GemmArgs& g, const Plan& p, int dtype) {
    if (dtype == RP_DTYPE_BFLOAT16) return m16_launch_tile<bf16_t, BM, BN, WGM>(g, p);
    if (dtype == RP_DTYPE_FLOAT16) return m16_launch_tile<f16_t, BM, BN, WGM>(g, p);
    set_error("mfma16 GEMM: unsupported dtype %d", dtype);
    return -1;
}

}  // namespace rp
