// fp32 / fp64 MFMA GEMM kernels and their launcher.
#include "rp_gemm.h"

#include <type_traits>

namespace rp {

// ============================================================================
// mfmaw: fp32 (32x32x2) and fp64 (16x16x4) MFMA, one element per lane per
// operand.  Both operands sit in LDS k-major, [BK][tile + pad]: a lane reads
// the element (k, free) it feeds to the MFMA, and a half-wave reads a run of
// consecutive free indices (no bank conflicts).  KC operands are transposed on
// the way into LDS (a thread loads V consecutive k of one row and writes them
// to V k-rows).
// ============================================================================
template <typename T> struct mfmaw_cfg;
template <> struct mfmaw_cfg<float> {
    static constexpr int MT = 32, KS = 2, NV = 16, VEC = 4, BK = 32, PAD = 4;
    using acc_t = f32x16_t;
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
    // row of accumulator register v inside the MFMA tile
    static __device__ __forceinline__ int acc_row(int v, int lane) { return 8 * (v / 4) + 4 * (lane >> 5) + (v % 4); }
};
template <> struct mfmaw_cfg<double> {
    static constexpr int MT = 16, KS = 4, NV = 4, VEC = 2, BK = 16, PAD = 2;
    using acc_t = f64x4_t;
    static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int acc_row(int v, int lane) { return 4 * v + (lane >> 4); }
};

// One operand's slab traffic, a 16-byte piece per thread at a time: piece i of thread t covers V consecutive
// elements along the operand's unit-stride axis.  LDS is k-major, [BK][ROWS + PAD]; a KC piece (V consecutive k
// of one row) is transposed on the way in with V scalar writes.
template <typename T, int ROWS, bool MC, bool EDGE>
struct MwSlab {
    using cfg = mfmaw_cfg<T>;
    static constexpr int V = cfg::VEC, NP = ROWS * cfg::BK / V / 256, PITCH = ROWS + cfg::PAD;
    static __device__ __forceinline__ void coords(int t, int i, int& r, int& kk) {
        int id = t + 256 * i;
        if (MC) { kk = id / (ROWS / V); r = (id % (ROWS / V)) * V; }
        else    { r = id / (cfg::BK / V); kk = (id % (cfg::BK / V)) * V; }
    }
    // piece i of the slab that starts at k0 (relative to the block's k range of length k_extent)
    static __device__ __forceinline__ uint4 load(const T* base, long long free_stride, long long k_stride, int row0, int k0,
                                                 int free_extent, int k_extent, int t, int i) {
        int r, kk;
        coords(t, i, r, kk);
        if (EDGE && !((row0 + r < free_extent) && (k0 + kk < k_extent))) return uint4{0u, 0u, 0u, 0u};
        return load_at(base + (long long)(row0 + r) * free_stride + (long long)(k0 + kk) * k_stride);
    }
    // the same piece with the offset of its free index given (a free axis that is a list of segments)
    static __device__ __forceinline__ uint4 load_free_at(const T* base, long long free_offset, long long k_stride, int row0, int k0,
                                                         int free_extent, int k_extent, int t, int i) {
        int r, kk;
        coords(t, i, r, kk);
        if (EDGE && !((row0 + r < free_extent) && (k0 + kk < k_extent))) return uint4{0u, 0u, 0u, 0u};
        return load_at(base + free_offset + (long long)(k0 + kk) * k_stride);
    }
    // 16 bytes from an address that is a multiple of the element size only (segment offsets shift whole elements)
    static __device__ __forceinline__ uint4 load_at(const T* p) {
        uint4 v;
        __builtin_memcpy(&v, p, 16);
        return v;
    }
    static __device__ __forceinline__ void store(T* lds, uint4 raw, int t, int i) {
        int r, kk;
        coords(t, i, r, kk);
        if (MC) {
            *(uint4*)(lds + kk * PITCH + r) = raw;
        } else {
            T e[V];
            memcpy(e, &raw, 16);
#pragma unroll
            for (int q = 0; q < V; q++) lds[(kk + q) * PITCH + r] = e[q];
        }
    }
};

// ============================================================================
// Block tile BM x BN, 4 waves in a 2 x 2 grid, k slab BK, two LDS stages.
// Software pipeline per slab s (NKS k-steps of one MFMA depth each):
//   k-steps 0 .. NKS-2   MFMAs(ks) | fragments(ks+1) from LDS | a share of: registers holding slab s+1 -> the
//                        other LDS stage, then the global load of slab s+2 into the register just freed
//   barrier              slab s+1 is complete in LDS and nobody reads this slab's stage any more
//   k-step NKS-1         MFMAs | fragments(0) of slab s+1
// so LDS reads run a k-step ahead of the MFMAs, global loads get a whole slab to land, and one barrier per
// slab sits where a single MFMA group is left to issue.  The epilogue stages accumulators through LDS, 32
// columns per pass, so that every lane stores 16 bytes of one output row.
// With SPLITK the grid's z axis splits k (k_per_split a multiple of BK): blocks write fp32 partial tiles
// [split][m][n] and the shared combine kernel finishes (fp32 only).
// ============================================================================
template <typename T> __host__ __device__ constexpr int mw_epi_pitch() { return 32 + 16 / (int)sizeof(T); }
template <typename T>
__host__ __device__ constexpr size_t mw_smem_bytes(int bm, int bn) {
    size_t loop = 2 * (size_t)mfmaw_cfg<T>::BK * (bm + bn + 2 * mfmaw_cfg<T>::PAD) * sizeof(T);
    size_t epi = 4 * (size_t)(bm / 2) * mw_epi_pitch<T>() * sizeof(T);
    return loop > epi ? loop : epi;
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC, bool EDGE, bool SPLITK>
__global__ void __launch_bounds__(256, 2) gemm_mfmaw_kernel(GemmArgs g, int tiles_m, int tiles_n, float* partials, int k_per_split) {
    using cfg = mfmaw_cfg<T>;
    constexpr int MT = cfg::MT, BK = cfg::BK, NKS = BK / cfg::KS;
    constexpr int WM = BM / 2, WN = BN / 2, TMI = WM / MT, TNI = WN / MT;
    constexpr int PA = BM + cfg::PAD, PB = BN + cfg::PAD;
    constexpr int A_ELEMS = BK * PA, B_ELEMS = BK * PB, STAGE = A_ELEMS + B_ELEMS;
    using SlabA = MwSlab<T, BM, A_MC, EDGE>;
    using SlabB = MwSlab<T, BN, B_MC, EDGE>;
    constexpr int NA = SlabA::NP, NB = SlabB::NP, NP_ALL = NA + NB;
    extern __shared__ __attribute__((aligned(16))) unsigned char mw_smem_raw[];
    T* smem = (T*)mw_smem_raw;

    TileCoord tc = schedule_tile(blockIdx.x, tiles_m, tiles_n);
    if (!tc.valid) return;
    const int z = blockIdx.y;
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;
    const int kbeg = SPLITK ? blockIdx.z * k_per_split : 0;
    const int kend = SPLITK ? (kbeg + k_per_split < g.k ? kbeg + k_per_split : g.k) : g.k;
    const int klen = kend - kbeg;              // loaders see a k axis that starts at kbeg and is klen long
    const T* A = (const T*)g.A + (long long)z * g.a_bs + (long long)kbeg * a_ks;
    const T* B = (const T*)g.B + (long long)z * g.b_bs + (long long)kbeg * b_ks;

    typename cfg::acc_t acc[TMI][TNI];
#pragma unroll
    for (int i = 0; i < TMI; i++)
#pragma unroll
        for (int j = 0; j < TNI; j++)
#pragma unroll
            for (int v = 0; v < cfg::NV; v++) acc[i][j][v] = (T)0;

    uint4 regs[NP_ALL];                        // pieces 0 .. NA-1 are A's, the rest B's
    const int nslabs = (klen + BK - 1) / BK;
    // B as a list of segments (GemmArgs::seg_*; never with SPLITK).  Along k (B_MC): every slab lies inside one segment,
    // whose start replaces B's for that slab.  Along n (!B_MC): each piece's column has its own offset, fixed for
    // the whole loop.
    const bool k_segmented = B_MC && g.seg_k > 0, n_segmented = !B_MC && g.seg_n > 0;
    long long b_free_off[NB];
    if (n_segmented) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            int r, kk;
            SlabB::coords(t, i, r, kk);
            const int j = n0 + r < g.n ? n0 + r : g.n - 1, seg = j / g.seg_n;
            b_free_off[i] = (long long)(seg / g.seg_w) * g.seg_sh + (long long)(seg % g.seg_w) * g.seg_sw + (long long)(j - seg * g.seg_n) * b_fs;
        }
    }
    auto load_piece = [&](auto pc, int k0) {
        constexpr int p = decltype(pc)::value;
        if constexpr (p < NA) {
            regs[p] = SlabA::load(A, a_fs, a_ks, m0, k0, g.m, klen, t, p);
        } else if (n_segmented) {
            regs[p] = SlabB::load_free_at(B, b_free_off[p - NA], b_ks, n0, k0, g.n, klen, t, p - NA);
        } else {
            const T* base = B;
            if (k_segmented) {
                const int seg = k0 / g.seg_k;
                base = B + (long long)(seg / g.seg_w) * g.seg_sh + (long long)(seg % g.seg_w) * g.seg_sw - (long long)seg * g.seg_k * b_ks;
            }
            regs[p] = SlabB::load(base, b_fs, b_ks, n0, k0, g.n, klen, t, p - NA);
        }
    };
    auto store_piece = [&](auto pc, T* stage) {
        constexpr int p = decltype(pc)::value;
        if constexpr (p < NA) SlabA::store(stage, regs[p], t, p);
        else SlabB::store(stage + A_ELEMS, regs[p], t, p - NA);
    };

    const int lf = lane % MT, lk = lane / MT;         // lane's free index and k index inside one MFMA
    T af[2][TMI], bf[2][TNI];
    auto read_frags = [&](const T* stage, int ks, int slot) {
        const int kk = ks * cfg::KS + lk;
#pragma unroll
        for (int i = 0; i < TMI; i++) af[slot][i] = stage[kk * PA + wm0 + i * MT + lf];
#pragma unroll
        for (int j = 0; j < TNI; j++) bf[slot][j] = stage[A_ELEMS + kk * PB + wn0 + j * MT + lf];
    };

    // prologue: slab 0 into stage 0, slab 1 into registers, fragments(0) of slab 0
    static_for<0, NP_ALL>([&](auto pc) { load_piece(pc, 0); });
    static_for<0, NP_ALL>([&](auto pc) { store_piece(pc, smem); });
    if (nslabs > 1) static_for<0, NP_ALL>([&](auto pc) { load_piece(pc, BK); });
    __syncthreads();
    read_frags(smem, 0, 0);

    // One slab.  NEXT: slab s+1 exists (its registers go to LDS here and the barrier runs); NEXT2: slab s+2 exists
    // (its global loads are issued here).  Both are compile-time so that the steady-state loop issues its loads
    // unconditionally and the waits the compiler places before each LDS store count them exactly.
    auto slab_step = [&](int s, auto next_tag, auto next2_tag) {
        constexpr bool NEXT = decltype(next_tag)::value, NEXT2 = decltype(next2_tag)::value;
        const T* stage = smem + (s & 1) * STAGE;
        T* other = smem + ((s & 1) ^ 1) * STAGE;
        static_for<0, NKS>([&](auto ksc) {
            constexpr int ks = decltype(ksc)::value, slot = ks & 1;
            if constexpr (ks + 1 < NKS) {
                read_frags(stage, ks + 1, slot ^ 1);
                // this k-step's share of the slab traffic
                constexpr int P0 = (NP_ALL * ks) / (NKS - 1), P1 = (NP_ALL * (ks + 1)) / (NKS - 1);
                if constexpr (NEXT) {
                    static_for<P0, P1>([&](auto pc) {
                        store_piece(pc, other);
                        if constexpr (NEXT2) load_piece(pc, (s + 2) * BK);
                    });
                }
            } else if constexpr (NEXT) {
                __syncthreads();
                read_frags(other, 0, slot ^ 1);
            }
#pragma unroll
            for (int i = 0; i < TMI; i++)
#pragma unroll
                for (int j = 0; j < TNI; j++) acc[i][j] = cfg::mma(af[slot][i], bf[slot][j], acc[i][j]);
        });
    };
    using yes = std::true_type;
    using no = std::false_type;
    int s = 0;
    for (; s + 2 < nslabs; s++) slab_step(s, yes{}, yes{});
    if (s + 1 < nslabs) { slab_step(s, yes{}, no{}); s++; }
    slab_step(s, no{}, no{});

    // ---- epilogue: 32 columns of every wave's patch per pass through the wave's private LDS region ----
    constexpr int V = cfg::VEC, CN = 32, EP = mw_epi_pitch<T>(), TJ = CN / MT, PASSES = WN / CN;
    constexpr int LPR = CN / V, RPS = 64 / LPR;          // lanes per row, rows per step
    T* region = smem + wave * (WM * EP);
    T* C = (T*)g.C + (long long)z * g.c_bs;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    const bool c_vec = (g.c_cs == 1) && (g.c_rs % V == 0) && (((uintptr_t)C & 15) == 0);
    const int ecol = (lane % LPR) * V, erow = lane / LPR;
#pragma unroll
    for (int p = 0; p < PASSES; p++) {
        __syncthreads();                        // the main loop (or the previous pass) is done with LDS
#pragma unroll
        for (int i = 0; i < TMI; i++)
#pragma unroll
            for (int jj = 0; jj < TJ; jj++)
#pragma unroll
                for (int v = 0; v < cfg::NV; v++)
                    region[(i * MT + cfg::acc_row(v, lane)) * EP + jj * MT + lf] = acc[i][p * TJ + jj][v];
        __syncthreads();
        const int gn = n0 + wn0 + p * CN + ecol;
        const bool by_row = g.bias_by_row != 0;
        T bv[V];
#pragma unroll
        for (int e = 0; e < V; e++) bv[e] = (has_bias && !by_row && (!EDGE || gn + e < g.n)) ? bias[gn + e] : (T)0;
        // folded output (GemmArgs::c_fold_*): the vector keeps its place inside a run of c_fold_from columns, the runs
        // move together to c_fold_to columns each, vectors past c_fold_to of a run are not stored
        int gn_out = gn;
        bool live = true;
        if (g.c_fold_from > 0) {
            const int run = gn / g.c_fold_from, within = gn - run * g.c_fold_from;
            live = within < g.c_fold_to;
            gn_out = run * g.c_fold_to + within;
        }
#pragma unroll 2
        for (int r = erow; r < WM; r += RPS) {
            const int gm = m0 + wm0 + r;
            if (EDGE && gm >= g.m) break;
            uint4 raw = *(const uint4*)(region + r * EP + ecol);
            T vals[V];
            memcpy(vals, &raw, 16);
            if constexpr (SPLITK) {
                // fp32 partial tile [split][m][n]; n is a multiple of 4 on this path, so the vector is wholly in or out
                if (!EDGE || gn + V <= g.n) *(uint4*)(partials + (((long long)z * gridDim.z + blockIdx.z) * g.m + gm) * g.n + gn) = raw;
                continue;
            }
            T* crow = C + (long long)gm * g.c_rs;
            if (has_bias && by_row) {
#pragma unroll
                for (int e = 0; e < V; e++) bv[e] = bias[gm];
            }
            if (c_vec && (!EDGE || gn + V <= g.n)) {
                if (!live) continue;
                T old[V], out[V];
                if (accum) { uint4 o = *(const uint4*)(crow + gn_out); memcpy(old, &o, 16); }
#pragma unroll
                for (int e = 0; e < V; e++) out[e] = finish<T>(vals[e], has_bias, bv[e], accum, accum ? old[e] : (T)0);
                uint4 o;
                memcpy(&o, out, 16);
                *(uint4*)(crow + gn_out) = o;
            } else {
#pragma unroll
                for (int e = 0; e < V; e++) {
                    if (EDGE && gn + e >= g.n) break;
                    T* pc = crow + (long long)(gn + e) * g.c_cs;
                    T old = accum ? *pc : (T)0;
                    *pc = finish<T>(vals[e], has_bias, bv[e], accum, old);
                }
            }
        }
    }
}

// ============================================================================
// Short reductions (k of at most two slabs: 64 for fp32), many tiles.
// A tile of such a product has no k loop to pipeline: load, wait, multiply for a few microseconds, store.  In the
// kernel above those phases follow one another inside a workgroup, and the 64 KB a tile writes wait at the end of
// it for a write path that takes about 8 bytes per clock from a CU: the epilogue costs more than the multiplies
// (S = Q.K^T of 192 x 512 x 64 x 512: prologue 4.5 K, MFMAs 12.5 K, epilogue 17 K cycles per tile).  Here the
// workgroups are resident and walk the tiles (of all batch entries): the whole k of the NEXT tile is loaded into
// registers while this tile is multiplied, and the accumulators are stored straight from registers (register v of a
// 32 x 32 MFMA tile is 32 adjacent columns of one row across 32 lanes, a full 128-byte line), so the stores of a
// tile drain while the next one is multiplied and no tile waits for memory at its start or its end.
// ============================================================================
template <typename T, int BM, int BN, bool A_MC, bool B_MC, bool EDGE>
__global__ void __launch_bounds__(256, (BM <= 64 ? 4 : 2)) gemm_mfmaw_shortk_kernel(GemmArgs g, int tiles_m, int tiles_n, long long total) {
    using cfg = mfmaw_cfg<T>;
    constexpr int MT = cfg::MT, BK = cfg::BK, NKS = BK / cfg::KS;
    constexpr int WM = BM / 2, WN = BN / 2, TMI = WM / MT, TNI = WN / MT;
    constexpr int PA = BM + cfg::PAD, PB = BN + cfg::PAD;
    constexpr int A_ELEMS = BK * PA, B_ELEMS = BK * PB, STAGE = A_ELEMS + B_ELEMS;
    using SlabA = MwSlab<T, BM, A_MC, EDGE>;
    using SlabB = MwSlab<T, BN, B_MC, EDGE>;
    constexpr int NA = SlabA::NP, NB = SlabB::NP, NP_ALL = NA + NB;
    extern __shared__ __attribute__((aligned(16))) unsigned char mw_smem_raw[];
    T* smem = (T*)mw_smem_raw;                 // stage 0: k [0, BK), stage 1: k [BK, 2 BK)
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;
    const int slabs = g.k > BK ? 2 : 1;
    const int per_matrix = tiles_m * tiles_n;
    const int lf = lane % MT, lk = lane / MT;

    uint4 regs[2][NP_ALL];
    auto load_tile = [&](long long id) {
        const int z = (int)(id / per_matrix), tile = (int)(id % per_matrix);
        const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN;
        const T* A = (const T*)g.A + (long long)z * g.a_bs;
        const T* B = (const T*)g.B + (long long)z * g.b_bs;
        static_for<0, 2>([&](auto sc) {
            constexpr int sl = decltype(sc)::value;
            if (sl < slabs) {
                static_for<0, NP_ALL>([&](auto pc) {
                    constexpr int p = decltype(pc)::value;
                    if constexpr (p < NA) regs[sl][p] = SlabA::load(A, a_fs, a_ks, m0, sl * BK, g.m, g.k, t, p);
                    else regs[sl][p] = SlabB::load(B, b_fs, b_ks, n0, sl * BK, g.n, g.k, t, p - NA);
                });
            }
        });
    };

    long long id = blockIdx.x;
    if (id < total) load_tile(id);
    for (; id < total; id += gridDim.x) {
        const int z = (int)(id / per_matrix), tile = (int)(id % per_matrix);
        const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN;
        // this tile's operands: registers -> LDS (every wave has finished reading the previous tile: barrier at the loop's end)
        static_for<0, 2>([&](auto sc) {
            constexpr int sl = decltype(sc)::value;
            if (sl < slabs) {
                static_for<0, NP_ALL>([&](auto pc) {
                    constexpr int p = decltype(pc)::value;
                    if constexpr (p < NA) SlabA::store(smem + sl * STAGE, regs[sl][p], t, p);
                    else SlabB::store(smem + sl * STAGE + A_ELEMS, regs[sl][p], t, p - NA);
                });
            }
        });
        __syncthreads();
        if (id + gridDim.x < total) load_tile(id + gridDim.x);       // lands while this tile is multiplied

        typename cfg::acc_t acc[TMI][TNI];
#pragma unroll
        for (int i = 0; i < TMI; i++)
#pragma unroll
            for (int j = 0; j < TNI; j++)
#pragma unroll
                for (int v = 0; v < cfg::NV; v++) acc[i][j][v] = (T)0;
        T af[2][TMI], bf[2][TNI];
        auto read_frags = [&](const T* stage, int ks, int slot) {
            const int kk = ks * cfg::KS + lk;
#pragma unroll
            for (int i = 0; i < TMI; i++) af[slot][i] = stage[kk * PA + wm0 + i * MT + lf];
#pragma unroll
            for (int j = 0; j < TNI; j++) bf[slot][j] = stage[A_ELEMS + kk * PB + wn0 + j * MT + lf];
        };
        read_frags(smem, 0, 0);
        for (int sl = 0; sl < slabs; sl++) {
            const T* stage = smem + sl * STAGE;
            static_for<0, NKS>([&](auto ksc) {
                constexpr int ks = decltype(ksc)::value, slot = ks & 1;
                if constexpr (ks + 1 < NKS) read_frags(stage, ks + 1, slot ^ 1);
                else if (sl + 1 < slabs) read_frags(stage + STAGE, 0, slot ^ 1);
#pragma unroll
                for (int i = 0; i < TMI; i++)
#pragma unroll
                    for (int j = 0; j < TNI; j++) acc[i][j] = cfg::mma(af[slot][i], bf[slot][j], acc[i][j]);
            });
        }

        // epilogue straight from the accumulators: one store instruction is MT adjacent columns of 64 / MT rows
        T* C = (T*)g.C + (long long)z * g.c_bs;
        const T* bias = (const T*)g.bias;
        const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
#pragma unroll
        for (int j = 0; j < TNI; j++) {
            const int gn = n0 + wn0 + j * MT + lf;
            const bool col_ok = !EDGE || gn < g.n;
            const T bv = (has_bias && col_ok) ? bias[gn] : (T)0;
#pragma unroll
            for (int i = 0; i < TMI; i++)
#pragma unroll
                for (int v = 0; v < cfg::NV; v++) {
                    const int gm = m0 + wm0 + i * MT + cfg::acc_row(v, lane);
                    if (EDGE && !(col_ok && gm < g.m)) continue;
                    T* pc = C + (long long)gm * g.c_rs + (long long)gn * g.c_cs;
                    if (accum) *pc = finish<T>(acc[i][j][v], has_bias, bv, true, *pc);
                    else *pc = finish<T>(acc[i][j][v], has_bias, bv, false, (T)0);
                }
        }
        __syncthreads();                       // every wave is done with this tile's LDS
    }
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC>
static int mw_launch_shortk(const GemmArgs& g, bool edge) {
    const int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    const long long total = (long long)tiles_m * tiles_n * g.batch;
    constexpr size_t smem = 2 * (size_t)mfmaw_cfg<T>::BK * (BM + BN + 2 * mfmaw_cfg<T>::PAD) * sizeof(T);
    int cus = device_cu_count();
    if (cus <= 0) cus = 256;
    const long long blocks = total < 2ll * cus ? total : 2ll * cus;         // two resident workgroups per CU
    auto launch = [&](auto kern) {
        if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
        hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), smem, current_stream(), g, tiles_m, tiles_n, total);
        return check_launch("gemm_mfmaw_shortk_kernel") ? 0 : -1;
    };
    if (edge) return launch(gemm_mfmaw_shortk_kernel<T, BM, BN, A_MC, B_MC, true>);
    return launch(gemm_mfmaw_shortk_kernel<T, BM, BN, A_MC, B_MC, false>);
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC, bool EDGE, bool SPLITK>
static int mw_launch(const GemmArgs& g, dim3 grid, int tiles_m, int tiles_n, float* partials, int k_per_split) {
    constexpr size_t smem = mw_smem_bytes<T>(BM, BN);
    auto kern = gemm_mfmaw_kernel<T, BM, BN, A_MC, B_MC, EDGE, SPLITK>;
    if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, current_stream(), g, tiles_m, tiles_n, partials, k_per_split);
    return check_launch("gemm_mfmaw_kernel") ? 0 : -1;
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC>
static int launch_mfmaw_edge(const GemmArgs& g, bool edge, float* partials, int nsplit, int k_per_split) {
    int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    if (nsplit > 1) {
        if constexpr (sizeof(T) == 4) {           // split-k partials are fp32; always the predicated variant
            dim3 grid(scheduled_grid(tiles_m, tiles_n), g.batch, nsplit);
            return mw_launch<T, BM, BN, A_MC, B_MC, true, true>(g, grid, tiles_m, tiles_n, partials, k_per_split);
        }
        set_error("mfmaw GEMM: split-k is fp32 only");
        return -1;
    }
    dim3 grid(scheduled_grid(tiles_m, tiles_n), g.batch);
    if (edge) return mw_launch<T, BM, BN, A_MC, B_MC, true, false>(g, grid, tiles_m, tiles_n, nullptr, 0);
    return mw_launch<T, BM, BN, A_MC, B_MC, false, false>(g, grid, tiles_m, tiles_n, nullptr, 0);
}

template <typename T, int BM, int BN>
static int launch_mfmaw_layout(const GemmArgs& g, const Plan& p, float* partials, int nsplit, int k_per_split) {
    if (!p.a_mc && p.b_mc) return launch_mfmaw_edge<T, BM, BN, false, true>(g, p.edge, partials, nsplit, k_per_split);
    if (!p.a_mc && !p.b_mc) return launch_mfmaw_edge<T, BM, BN, false, false>(g, p.edge, partials, nsplit, k_per_split);
    if (p.a_mc && p.b_mc) return launch_mfmaw_edge<T, BM, BN, true, true>(g, p.edge, partials, nsplit, k_per_split);
    return launch_mfmaw_edge<T, BM, BN, true, false>(g, p.edge, partials, nsplit, k_per_split);
}

template <typename T>
static int launch_mfmaw_t(const GemmArgs& g, const Plan& p) {
    // Small outputs with a deep k leave most CUs idle: split k so that about 256 blocks run (each split at
    // least two slabs deep), and add the partials [matrix][split][m][n] in split order afterwards.  fp32 only; a batch
    // is split the same way while all its tiles together leave CUs idle.
    int nsplit = 1, k_per_split = 0;
    constexpr int BK = mfmaw_cfg<T>::BK;
    if (sizeof(T) == 4 && p.bm == 64 && g.n % 4 == 0 && g.seg_k == 0 && g.seg_n == 0 && g.c_fold_from == 0 && !g.bias_by_row) {   // (segments and the folded store: never split)
        int tiles = ((g.m + 63) / 64) * ((g.n + 63) / 64) * g.batch;
        int want = (256 + tiles - 1) / tiles, deep = g.k / (2 * BK);
        nsplit = want < deep ? want : deep;
        if (nsplit > 1) {
            k_per_split = ((g.k + nsplit - 1) / nsplit + BK - 1) / BK * BK;
            nsplit = (g.k + k_per_split - 1) / k_per_split;
        }
        if (nsplit < 2) nsplit = 1;
    }
    void* ws = nullptr;
    if (nsplit > 1 && gemm_workspace(&ws, (size_t)g.batch * nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
    int rc = (p.bm == 128) ? launch_mfmaw_layout<T, 128, 128>(g, p, (float*)ws, nsplit, k_per_split)
                           : launch_mfmaw_layout<T, 64, 64>(g, p, (float*)ws, nsplit, k_per_split);
    if (rc == 0 && nsplit > 1) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, traits<T>::code);
    if (ws) gemm_workspace_release(ws);          // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

int launch_mfmaw(const GemmArgs& g, const Plan& p, int dtype) {
    // fp32, k of at most two slabs, at least 128 tiles of 128 x 128: the resident, cross-tile pipelined kernel
    if (dtype == RP_DTYPE_FLOAT32 && p.bm == 128 && g.k <= 2 * mfmaw_cfg<float>::BK && !path_disabled("shortk") && g.seg_k == 0 && g.seg_n == 0 && g.c_fold_from == 0 && !g.bias_by_row) {
        const bool edge = p.edge || g.k != 2 * mfmaw_cfg<float>::BK;
        if (!p.a_mc && p.b_mc) return mw_launch_shortk<float, 128, 128, false, true>(g, edge);
        if (!p.a_mc && !p.b_mc) return mw_launch_shortk<float, 128, 128, false, false>(g, edge);
        if (p.a_mc && p.b_mc) return mw_launch_shortk<float, 128, 128, true, true>(g, edge);
        return mw_launch_shortk<float, 128, 128, true, false>(g, edge);
    }
    if (dtype == RP_DTYPE_FLOAT32) return launch_mfmaw_t<float>(g, p);
    if (dtype == RP_DTYPE_FLOAT64) return launch_mfmaw_t<double>(g, p);
    set_error("mfmaw GEMM: unsupported dtype %d", dtype);
    return -1;
}

}  // namespace rp
