// GEMM kernels for gfx950 and their dispatcher.
//
//   C_z[m,n] = A_z[m,k] · B_z[k,n] (+ bias[n]) (+ C_z)      z in [0, batch)
//
// Operands are described by (batch, row, column) strides in elements, so
// transposed and permuted views are read in place.  Each operand is in one of
// two fast layouts, chosen from its strides:
//   KC  the reduction (k) axis is the unit-stride one      (A row-major, or Bᵀ stored)
//   MC  the free (m or n) axis is the unit-stride one       (B row-major, or Aᵀ stored)
// Anything else (both strides > 1, misaligned bases, odd extents) takes the
// generic strided kernel.
//
// Kernel families:
//   mfma16   bf16 / fp16 inputs, fp32 accumulate, v_mfma_f32_32x32x16_{bf16,f16};
//            KC tiles are read from LDS with ds_read_b128, MC tiles with the
//            transposing ds_read_b64_tr_b16, so no layout needs a copy.
//   mfmaw    fp32 (v_mfma_f32_32x32x2_f32) and fp64 (v_mfma_f64_16x16x4_f64).
//   skinny   m <= 8 against a row-major B: a split-k streaming kernel bound by HBM.
//   generic  any strides, any shape; LDS-tiled scalar FMA.
#include "rp_common.h"

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
};

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) double f64x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

// ============================================================================
// generic: 64x64 output tile, 16-deep k slabs, 256 threads each owning 4x4.
// ============================================================================
template <typename T>
__global__ void __launch_bounds__(256) gemm_generic_kernel(GemmArgs g) {
    using Acc = typename traits<T>::acc;
    constexpr int TM = 64, TN = 64, TK = 16;
    __shared__ Acc As[TK][TM + 1];
    __shared__ Acc Bs[TK][TN + 1];

    const int z = blockIdx.z;
    const T* A = (const T*)g.A + (long long)z * g.a_bs;
    const T* B = (const T*)g.B + (long long)z * g.b_bs;
    T* C = (T*)g.C + (long long)z * g.c_bs;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    const int t = threadIdx.x;
    const int ty = t / 16, tx = t % 16;
    const bool a_kfast = (g.a_cs == 1), b_nfast = (g.b_cs == 1);

    Acc acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (Acc)0;

    for (int k0 = 0; k0 < g.k; k0 += TK) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = t + 256 * i;
            int kk = a_kfast ? id % TK : id / TM;
            int r = a_kfast ? id / TK : id % TM;
            int gm = m0 + r, gk = k0 + kk;
            Acc v = (Acc)0;
            if (gm < g.m && gk < g.k) v = widen(A[(long long)gm * g.a_rs + (long long)gk * g.a_cs]);
            As[kk][r] = v;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = t + 256 * i;
            int kk = b_nfast ? id / TN : id % TK;
            int c = b_nfast ? id % TN : id / TK;
            int gn = n0 + c, gk = k0 + kk;
            Acc v = (Acc)0;
            if (gn < g.n && gk < g.k) v = widen(B[(long long)gk * g.b_rs + (long long)gn * g.b_cs]);
            Bs[kk][c] = v;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; kk++) {
            Acc a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }

    const T* bias = (const T*)g.bias;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int gm = m0 + ty * 4 + i;
        if (gm >= g.m) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int gn = n0 + tx * 4 + j;
            if (gn >= g.n) continue;
            T* p = C + (long long)gm * g.c_rs + (long long)gn * g.c_cs;
            T old = g.accumulate ? *p : T{};
            T bv = bias ? bias[gn] : T{};
            *p = finish<T>(acc[i][j], bias != nullptr, bv, g.accumulate != 0, old);
        }
    }
}

// ============================================================================
// Tile scheduling shared by the MFMA kernels.
// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so a
// linear block id is first split into (xcd, slot); every XCD then walks its
// own sequence of 4x8-tile super-tiles, which keeps the 32 tiles resident on an
// XCD at one time inside a compact window of the output (4 A row panels and
// 8 B column panels shared through that XCD's L2).
// ============================================================================
struct TileCoord { int tm, tn; bool valid; };

constexpr int SCHED_MIN_TILES = 64;      // below this a launch does not fill the chip and plain row-major order is used

__device__ __forceinline__ TileCoord schedule_tile(int bid, int tiles_m, int tiles_n) {
    constexpr int XCDS = 8, GM = 4, GN = 8, PER = GM * GN;
    if (tiles_m * tiles_n < SCHED_MIN_TILES) {
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
    if (tiles_m * tiles_n < SCHED_MIN_TILES) return tiles_m * tiles_n;
    int sup = ((tiles_m + GM - 1) / GM) * ((tiles_n + GN - 1) / GN);
    int rounds = (sup + XCDS - 1) / XCDS;
    return rounds * XCDS * PER;
}

// ============================================================================
// mfma16: bf16 / fp16 inputs, fp32 accumulate.
//
// Block tile BM x BN, k slab 64, 256 threads = 4 waves in a 2x2 grid, each wave
// owning a (BM/2) x (BN/2) patch built from 32x32x16 MFMA tiles.  Global loads
// of slab i+1 are issued into registers before the MFMAs of slab i and stored
// to the other LDS buffer afterwards (one barrier per slab).
//
// LDS layouts (16-bit elements):
//   KC operand: [rows][64 + 8]   row pitch 144 B -> the 16 rows a quarter-wave
//               reads with ds_read_b128 land in 16 different 16-byte bank groups
//   MC operand: [64][cols + 32]  row pitch 2*cols + 64 B -> the 4 k-rows a
//               16-lane group reads with ds_read_b64_tr_b16 start 16 banks apart
// ============================================================================
template <typename T> struct mfma16_ops;
template <> struct mfma16_ops<bf16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};
template <> struct mfma16_ops<f16_t> {
    static __device__ __forceinline__ f32x16_t mma(s16x8_t a, s16x8_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};

constexpr int M16_BK = 64;
constexpr int M16_KC_PITCH = M16_BK + 8;                       // elements
__host__ __device__ constexpr int m16_mc_pitch(int cols) { return cols + 32; }
__host__ __device__ constexpr int m16_tile_elems(int rows, bool mc) {
    return mc ? M16_BK * m16_mc_pitch(rows) : rows * M16_KC_PITCH;
}

typedef uint16_t __attribute__((address_space(3))) lds_u16;

// Global -> registers for one operand slab.  `rows` = BM or BN, the operand's
// free extent inside the block tile; row0 = first free index of the tile,
// k0 = first k of the slab; free_extent / k_extent bound the EDGE variant.
template <int ROWS, bool MC, bool EDGE>
__device__ __forceinline__ void m16_load_slab(uint4 (&regs)[ROWS * 8 / 256], const uint16_t* base, long long free_stride,
                                              long long k_stride, int row0, int k0, int free_extent, int k_extent, int t) {
    constexpr int N = ROWS * 8 / 256;
#pragma unroll
    for (int i = 0; i < N; i++) {
        int id = t + 256 * i;
        int r, kk;          // r: free index inside the tile (first of 8 for MC); kk: k inside the slab (first of 8 for KC)
        if (MC) { kk = id / (ROWS / 8); r = (id % (ROWS / 8)) * 8; }
        else    { r = id / 8; kk = (id % 8) * 8; }
        const uint16_t* p = base + (long long)(row0 + r) * free_stride + (long long)(k0 + kk) * k_stride;
        bool ok = true;
        if (EDGE) ok = (row0 + r < free_extent) && (k0 + kk < k_extent);
        regs[i] = ok ? *(const uint4*)p : make_uint4(0, 0, 0, 0);
    }
}

template <int ROWS, bool MC>
__device__ __forceinline__ void m16_store_slab(const uint4 (&regs)[ROWS * 8 / 256], uint16_t* lds, int t) {
    constexpr int N = ROWS * 8 / 256;
#pragma unroll
    for (int i = 0; i < N; i++) {
        int id = t + 256 * i;
        int off;
        if (MC) { int kk = id / (ROWS / 8), r = (id % (ROWS / 8)) * 8; off = kk * m16_mc_pitch(ROWS) + r; }
        else    { int r = id / 8, kk = (id % 8) * 8; off = r * M16_KC_PITCH + kk; }
        *(uint4*)(lds + off) = regs[i];
    }
}

// One 32 x 16 MFMA operand fragment (8 values per lane) for free-index base r0
// and k step ks (16 k per step) out of an LDS slab.
template <int ROWS, bool MC>
__device__ __forceinline__ s16x8_t m16_read_frag(const uint16_t* lds, int r0, int ks, int lane) {
    if (!MC) {
        int row = r0 + (lane & 31);
        int kk = ks * 16 + (lane >> 5) * 8;
        return *(const s16x8_t*)(lds + row * M16_KC_PITCH + kk);
    } else {
        // ds_read_b64_tr_b16: inside each 16-lane group, source lane s points at
        // 4 consecutive free indices of k-row s/4; destination lane j receives
        // free index j of k-rows 0..3.  Two reads give the lane its 8 k values.
        int grp = lane >> 4, s = lane & 15;
        int fbase = r0 + 16 * (grp & 1) + 4 * (s & 3);
        int kbase = ks * 16 + 8 * (grp >> 1) + (s >> 2);
        const uint16_t* p0 = lds + kbase * m16_mc_pitch(ROWS) + fbase;
        const uint16_t* p1 = p0 + 4 * m16_mc_pitch(ROWS);
        s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(lds_u16*)p0);
        s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(lds_u16*)p1);
        s16x8_t r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    }
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC, bool EDGE>
__global__ void __launch_bounds__(256) gemm_mfma16_kernel(GemmArgs g, int tiles_m, int tiles_n) {
    constexpr int WM = BM / 2, WN = BN / 2;           // wave patch
    constexpr int TMI = WM / 32, TNI = WN / 32;       // MFMA tiles per wave
    constexpr int A_ELEMS = m16_tile_elems(BM, A_MC), B_ELEMS = m16_tile_elems(BN, B_MC);
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    constexpr int STAGE = A_ELEMS + B_ELEMS;          // stage s: A at smem + s*STAGE, B right after it

    TileCoord tc = schedule_tile(blockIdx.x, tiles_m, tiles_n);
    if (!tc.valid) return;
    const int z = blockIdx.y;
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;

    const uint16_t* A = (const uint16_t*)g.A + (long long)z * g.a_bs;
    const uint16_t* B = (const uint16_t*)g.B + (long long)z * g.b_bs;
    // A: free axis = m (stride a_rs), k stride a_cs.  B: free axis = n (stride b_cs), k stride b_rs.
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;

    f32x16_t acc[TMI][TNI];
#pragma unroll
    for (int i = 0; i < TMI; i++)
#pragma unroll
        for (int j = 0; j < TNI; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    uint4 ra[BM * 8 / 256], rb[BN * 8 / 256];
    const int nslabs = (g.k + M16_BK - 1) / M16_BK;

    m16_load_slab<BM, A_MC, EDGE>(ra, A, a_fs, a_ks, m0, 0, g.m, g.k, t);
    m16_load_slab<BN, B_MC, EDGE>(rb, B, b_fs, b_ks, n0, 0, g.n, g.k, t);
    m16_store_slab<BM, A_MC>(ra, smem, t);
    m16_store_slab<BN, B_MC>(rb, smem + A_ELEMS, t);
    __syncthreads();

    for (int s = 0; s < nslabs; s++) {
        const int cur = s & 1;
        const bool more = (s + 1 < nslabs);
        if (more) {
            m16_load_slab<BM, A_MC, EDGE>(ra, A, a_fs, a_ks, m0, (s + 1) * M16_BK, g.m, g.k, t);
            m16_load_slab<BN, B_MC, EDGE>(rb, B, b_fs, b_ks, n0, (s + 1) * M16_BK, g.n, g.k, t);
        }
        const uint16_t* a_lds = smem + cur * STAGE;
        const uint16_t* b_lds = a_lds + A_ELEMS;
#pragma unroll
        for (int ks = 0; ks < M16_BK / 16; ks++) {
            s16x8_t af[TMI], bf[TNI];
#pragma unroll
            for (int i = 0; i < TMI; i++) af[i] = m16_read_frag<BM, A_MC>(a_lds, wm0 + i * 32, ks, lane);
#pragma unroll
            for (int j = 0; j < TNI; j++) bf[j] = m16_read_frag<BN, B_MC>(b_lds, wn0 + j * 32, ks, lane);
#pragma unroll
            for (int i = 0; i < TMI; i++)
#pragma unroll
                for (int j = 0; j < TNI; j++) acc[i][j] = mfma16_ops<T>::mma(af[i], bf[j], acc[i][j]);
        }
        if (more) {
            m16_store_slab<BM, A_MC>(ra, smem + (cur ^ 1) * STAGE, t);
            m16_store_slab<BN, B_MC>(rb, smem + (cur ^ 1) * STAGE + A_ELEMS, t);
        }
        __syncthreads();
    }

    // epilogue: acc register v of tile (i, j) holds row 8*(v/4) + 4*(lane/32) + v%4, column lane%32
    T* C = (T*)g.C + (long long)z * g.c_bs;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
#pragma unroll
    for (int j = 0; j < TNI; j++) {
        int gn = n0 + wn0 + j * 32 + (lane & 31);
        bool n_ok = !EDGE || gn < g.n;
        T bv = (has_bias && n_ok) ? bias[gn] : T{};
#pragma unroll
        for (int i = 0; i < TMI; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                int gm = m0 + wm0 + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                if (n_ok && (!EDGE || gm < g.m)) {
                    T* p = C + (long long)gm * g.c_rs + (long long)gn * g.c_cs;
                    T old = accum ? *p : T{};
                    *p = finish<T>(acc[i][j][v], has_bias, bv, accum, old);
                }
            }
        }
    }
}

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
    static constexpr int MT = 32, KS = 2, NV = 16, VEC = 4, BK = 16, PAD = 4;
    using acc_t = f32x16_t;
    static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
    // row of accumulator register v inside the MFMA tile
    static __device__ __forceinline__ int acc_row(int v, int lane) { return 8 * (v / 4) + 4 * (lane >> 5) + (v % 4); }
};
template <> struct mfmaw_cfg<double> {
    static constexpr int MT = 16, KS = 4, NV = 4, VEC = 2, BK = 8, PAD = 2;
    using acc_t = f64x4_t;
    static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int acc_row(int v, int lane) { return 4 * v + (lane >> 4); }
};

template <typename T, int ROWS, bool MC, bool EDGE>
__device__ __forceinline__ void mw_load_slab(T (&regs)[ROWS * mfmaw_cfg<T>::BK / 256], const T* base, long long free_stride, long long k_stride,
                                             int row0, int k0, int free_extent, int k_extent, int t) {
    using cfg = mfmaw_cfg<T>;
    constexpr int V = cfg::VEC, NVEC = ROWS * cfg::BK / V / 256;
#pragma unroll
    for (int i = 0; i < NVEC; i++) {
        int id = t + 256 * i;
        int r, kk;
        if (MC) { kk = id / (ROWS / V); r = (id % (ROWS / V)) * V; }
        else    { r = id / (cfg::BK / V); kk = (id % (cfg::BK / V)) * V; }
        const T* p = base + (long long)(row0 + r) * free_stride + (long long)(k0 + kk) * k_stride;
        bool ok = true;
        if (EDGE) ok = (row0 + r < free_extent) && (k0 + kk < k_extent);
        if (ok) {
            uint4 raw = *(const uint4*)p;
            memcpy(&regs[i * V], &raw, 16);
        } else {
#pragma unroll
            for (int e = 0; e < V; e++) regs[i * V + e] = (T)0;
        }
    }
}

template <typename T, int ROWS, bool MC>
__device__ __forceinline__ void mw_store_slab(const T (&regs)[ROWS * mfmaw_cfg<T>::BK / 256], T* lds, int t) {
    using cfg = mfmaw_cfg<T>;
    constexpr int V = cfg::VEC, NVEC = ROWS * cfg::BK / V / 256, PITCH = ROWS + cfg::PAD;
#pragma unroll
    for (int i = 0; i < NVEC; i++) {
        int id = t + 256 * i;
        if (MC) {
            int kk = id / (ROWS / V), r = (id % (ROWS / V)) * V;
            uint4 raw;
            memcpy(&raw, &regs[i * V], 16);
            *(uint4*)(lds + kk * PITCH + r) = raw;
        } else {
            int r = id / (cfg::BK / V), kk = (id % (cfg::BK / V)) * V;
#pragma unroll
            for (int e = 0; e < V; e++) lds[(kk + e) * PITCH + r] = regs[i * V + e];
        }
    }
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC, bool EDGE>
__global__ void __launch_bounds__(256) gemm_mfmaw_kernel(GemmArgs g, int tiles_m, int tiles_n) {
    using cfg = mfmaw_cfg<T>;
    constexpr int MT = cfg::MT, BK = cfg::BK;
    constexpr int WM = BM / 2, WN = BN / 2, TMI = WM / MT, TNI = WN / MT;
    constexpr int PA = BM + cfg::PAD, PB = BN + cfg::PAD;
    constexpr int A_ELEMS = BK * PA, B_ELEMS = BK * PB;
    __shared__ __attribute__((aligned(16))) T smem[2 * (A_ELEMS + B_ELEMS)];
    constexpr int STAGE = A_ELEMS + B_ELEMS;

    TileCoord tc = schedule_tile(blockIdx.x, tiles_m, tiles_n);
    if (!tc.valid) return;
    const int z = blockIdx.y;
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const T* A = (const T*)g.A + (long long)z * g.a_bs;
    const T* B = (const T*)g.B + (long long)z * g.b_bs;
    const long long a_fs = g.a_rs, a_ks = g.a_cs, b_fs = g.b_cs, b_ks = g.b_rs;

    typename cfg::acc_t acc[TMI][TNI];
#pragma unroll
    for (int i = 0; i < TMI; i++)
#pragma unroll
        for (int j = 0; j < TNI; j++)
#pragma unroll
            for (int v = 0; v < cfg::NV; v++) acc[i][j][v] = (T)0;

    T ra[BM * BK / 256], rb[BN * BK / 256];
    const int nslabs = (g.k + BK - 1) / BK;
    mw_load_slab<T, BM, A_MC, EDGE>(ra, A, a_fs, a_ks, m0, 0, g.m, g.k, t);
    mw_load_slab<T, BN, B_MC, EDGE>(rb, B, b_fs, b_ks, n0, 0, g.n, g.k, t);
    mw_store_slab<T, BM, A_MC>(ra, smem, t);
    mw_store_slab<T, BN, B_MC>(rb, smem + A_ELEMS, t);
    __syncthreads();

    const int lf = lane % MT, lk = lane / MT;         // lane's free index and k index inside one MFMA
    for (int s = 0; s < nslabs; s++) {
        const int cur = s & 1;
        const bool more = (s + 1 < nslabs);
        if (more) {
            mw_load_slab<T, BM, A_MC, EDGE>(ra, A, a_fs, a_ks, m0, (s + 1) * BK, g.m, g.k, t);
            mw_load_slab<T, BN, B_MC, EDGE>(rb, B, b_fs, b_ks, n0, (s + 1) * BK, g.n, g.k, t);
        }
        const T* a_lds = smem + cur * STAGE;
        const T* b_lds = a_lds + A_ELEMS;
#pragma unroll
        for (int ks = 0; ks < BK / cfg::KS; ks++) {
            T af[TMI], bf[TNI];
            int kk = ks * cfg::KS + lk;
#pragma unroll
            for (int i = 0; i < TMI; i++) af[i] = a_lds[kk * PA + wm0 + i * MT + lf];
#pragma unroll
            for (int j = 0; j < TNI; j++) bf[j] = b_lds[kk * PB + wn0 + j * MT + lf];
#pragma unroll
            for (int i = 0; i < TMI; i++)
#pragma unroll
                for (int j = 0; j < TNI; j++) acc[i][j] = cfg::mma(af[i], bf[j], acc[i][j]);
        }
        if (more) {
            mw_store_slab<T, BM, A_MC>(ra, smem + (cur ^ 1) * STAGE, t);
            mw_store_slab<T, BN, B_MC>(rb, smem + (cur ^ 1) * STAGE + A_ELEMS, t);
        }
        __syncthreads();
    }

    T* C = (T*)g.C + (long long)z * g.c_bs;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
#pragma unroll
    for (int j = 0; j < TNI; j++) {
        int gn = n0 + wn0 + j * MT + lf;
        bool n_ok = !EDGE || gn < g.n;
        T bv = (has_bias && n_ok) ? bias[gn] : (T)0;
#pragma unroll
        for (int i = 0; i < TMI; i++) {
#pragma unroll
            for (int v = 0; v < cfg::NV; v++) {
                int gm = m0 + wm0 + i * MT + cfg::acc_row(v, lane);
                if (n_ok && (!EDGE || gm < g.m)) {
                    T* p = C + (long long)gm * g.c_rs + (long long)gn * g.c_cs;
                    T old = accum ? *p : (T)0;
                    *p = finish<T>(acc[i][j][v], has_bias, bv, accum, old);
                }
            }
        }
    }
}

// ============================================================================
// skinny: m <= 8 rows of A against a row-major B (unit column stride).
// The cost is streaming B once from HBM.  Each lane owns VEC adjacent columns
// (one 16-byte load per k row), a wave covers 64*VEC columns, the 4 waves of a
// block split the block's k range and combine through LDS, and the grid's
// second axis splits k further.  Split partials go to a workspace; the block
// that arrives last for a column group adds them in split order (so the result
// does not depend on scheduling) and runs the epilogue.
// ============================================================================
constexpr int SK_MAX_M = 8;
constexpr int SK_MAX_GROUPS = 4096;
__device__ unsigned int g_skinny_arrivals[SK_MAX_GROUPS];     // zero at load; the last block of a group re-zeroes its slot

template <typename T, int MROWS>
__global__ void __launch_bounds__(256) gemm_skinny_kernel(GemmArgs g, float* partials, int k_per_block) {
    using Acc = typename traits<T>::acc;
    constexpr int VEC = 16 / sizeof(T);
    extern __shared__ __attribute__((aligned(16))) float a_lds[];          // [k_per_block][MROWS], fp32
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col0 = (blockIdx.x * 64 + lane) * VEC;
    const int split = blockIdx.y, nsplit = gridDim.y;
    const bool col_ok = col0 < g.n;          // n is a multiple of VEC, so a vector is wholly in or out
    const T* A = (const T*)g.A;
    const T* B = (const T*)g.B;

    Acc acc[MROWS][VEC];
#pragma unroll
    for (int r = 0; r < MROWS; r++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[r][e] = (Acc)0;

    const int kb = split * k_per_block;
    const int ke = kb + k_per_block < g.k ? kb + k_per_block : g.k;
    const int klen = ke - kb;
    // this block's slice of A, widened once, rows beyond m as zeros
    for (int i = threadIdx.x; i < MROWS * klen; i += 256) {
        int r = i / klen, kl = i % klen;
        a_lds[kl * MROWS + r] = (r < g.m) ? widen(A[(long long)r * g.a_rs + (long long)(kb + kl) * g.a_cs]) : 0.f;
    }
    __syncthreads();

    // the 4 waves take interleaved k rows of the block's range
    if (col_ok) {
        const T* bp = B + col0 + (long long)kb * g.b_rs;
        constexpr int U = 8;
        int kl = wave;
        for (; kl + 4 * (U - 1) < klen; kl += 4 * U) {
            u32x4_t raw[U];
#pragma unroll
            for (int u = 0; u < U; u++) raw[u] = __builtin_nontemporal_load((const u32x4_t*)(bp + (long long)(kl + 4 * u) * g.b_rs));
#pragma unroll
            for (int u = 0; u < U; u++) {
                T bv[VEC];
                memcpy(bv, &raw[u], 16);
                Acc bw[VEC];
#pragma unroll
                for (int e = 0; e < VEC; e++) bw[e] = widen(bv[e]);
#pragma unroll
                for (int r = 0; r < MROWS; r++) {
                    Acc a = a_lds[(kl + 4 * u) * MROWS + r];
#pragma unroll
                    for (int e = 0; e < VEC; e++) acc[r][e] += a * bw[e];
                }
            }
        }
        for (; kl < klen; kl += 4) {
            uint4 raw = *(const uint4*)(bp + (long long)kl * g.b_rs);
            T bv[VEC];
            memcpy(bv, &raw, 16);
#pragma unroll
            for (int r = 0; r < MROWS; r++) {
                Acc a = a_lds[kl * MROWS + r];
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[r][e] += a * widen(bv[e]);
            }
        }
    }

    // combine the 4 waves (fixed order 0,1,2,3)
    __shared__ Acc red[3][MROWS][VEC][64];
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < MROWS; r++)
#pragma unroll
            for (int e = 0; e < VEC; e++) red[wave - 1][r][e][lane] = acc[r][e];
    }
    __syncthreads();
    __shared__ bool last;
    if (wave == 0) {
#pragma unroll
        for (int w = 0; w < 3; w++)
#pragma unroll
            for (int r = 0; r < MROWS; r++)
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[r][e] += red[w][r][e][lane];
    }

    T* C = (T*)g.C;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    if (nsplit == 1) {
        if (wave == 0 && col_ok) {
#pragma unroll
            for (int r = 0; r < MROWS; r++) {
                if (r >= g.m) break;
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    T* p = C + (long long)r * g.c_rs + (long long)(col0 + e) * g.c_cs;
                    T old = accum ? *p : T{};
                    *p = finish<T>(acc[r][e], has_bias, has_bias ? bias[col0 + e] : T{}, accum, old);
                }
            }
        }
        return;
    }

    // partial layout: [split][row][n] in the accumulate type
    Acc* part = (Acc*)partials;
    if (wave == 0 && col_ok) {
#pragma unroll
        for (int r = 0; r < MROWS; r++) {
            if (r >= g.m) break;
#pragma unroll
            for (int e = 0; e < VEC; e++) part[((long long)split * g.m + r) * g.n + col0 + e] = acc[r][e];
        }
    }
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned int done = atomicAdd(&g_skinny_arrivals[blockIdx.x], 1u);
        last = (done == (unsigned)nsplit - 1);
    }
    __syncthreads();
    if (!last) return;
    __threadfence();
    if (wave == 0 && col_ok) {
#pragma unroll
        for (int r = 0; r < MROWS; r++) {
            if (r >= g.m) break;
            Acc sum[VEC];
#pragma unroll
            for (int e = 0; e < VEC; e++) sum[e] = (Acc)0;
            for (int s = 0; s < nsplit; s++) {
                const volatile Acc* q = (const volatile Acc*)&part[((long long)s * g.m + r) * g.n + col0];
#pragma unroll
                for (int e = 0; e < VEC; e++) sum[e] += q[e];
            }
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                T* p = C + (long long)r * g.c_rs + (long long)(col0 + e) * g.c_cs;
                T old = accum ? *p : T{};
                *p = finish<T>(sum[e], has_bias, has_bias ? bias[col0 + e] : T{}, accum, old);
            }
        }
    }
    if (threadIdx.x == 0) g_skinny_arrivals[blockIdx.x] = 0;
}

// ============================================================================
// dispatch
// ============================================================================
enum Family { FAM_GENERIC = 0, FAM_SKINNY, FAM_MFMA16, FAM_MFMAW };

struct Plan {
    Family fam;
    int bm, bn;
    bool a_mc, b_mc, edge;
    const char* name;
};

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

static bool force_generic() {
    static int v = -1;
    if (v < 0) { const char* e = getenv("RP_HIP_FORCE_GENERIC"); v = (e && e[0] == '1') ? 1 : 0; }
    return v == 1;
}

// Decide the kernel family and tile from shapes and strides alone (pointer
// alignment is checked by the caller, which may still fall back to generic).
static Plan make_plan(int batch, int m, int k, int n, long long a_rs, long long a_cs, long long b_rs, long long b_cs,
                      long long c_rs, long long c_cs, long long a_bs, long long b_bs, int dtype) {
    Plan p{FAM_GENERIC, 64, 64, false, false, true, "generic"};
    if (force_generic()) return p;
    const int vec = 16 / (int)dtype_size(dtype);                // elements per 16-byte vector
    // operand layouts: KC = unit stride along k, MC = unit stride along the free axis.
    // Extent-1 axes make the other stride irrelevant, but vector loads still need alignment of the non-unit stride.
    bool a_kc = (a_cs == 1) && (a_rs % vec == 0) && (k % vec == 0);
    bool a_mc = (a_rs == 1) && (a_cs % vec == 0) && (m % vec == 0);
    bool b_mc = (b_cs == 1) && (b_rs % vec == 0) && (n % vec == 0);
    bool b_kc = (b_rs == 1) && (b_cs % vec == 0) && (k % vec == 0);
    bool batch_ok = (batch == 1) || ((a_bs % vec == 0) && (b_bs % vec == 0));
    (void)c_rs; (void)c_cs;

    // skinny: few rows, row-major B, enough columns and depth to be worth streaming
    if (batch == 1 && m <= SK_MAX_M && b_mc && n >= 64 * vec && (long long)k * n >= (1ll << 20) &&
        (n + 64 * vec - 1) / (64 * vec) <= SK_MAX_GROUPS) {
        p.fam = FAM_SKINNY; p.name = "skinny"; p.b_mc = true;
        return p;
    }
    if (!(a_kc || a_mc) || !(b_kc || b_mc) || !batch_ok) return p;
    p.a_mc = !a_kc;             // when both qualify (extent-1 corner cases) keep the row-major reading
    p.b_mc = b_mc;

    if (dtype == RP_DTYPE_FLOAT16 || dtype == RP_DTYPE_BFLOAT16) {
        p.fam = FAM_MFMA16;
        long long tiles256 = (long long)((m + 255) / 256) * ((n + 255) / 256) * batch;
        if (m >= 256 && n >= 256 && tiles256 >= 128) { p.bm = 256; p.bn = 256; p.name = "mfma16_256x256"; }
        else if (m > 64 || n > 64) { p.bm = 128; p.bn = 128; p.name = "mfma16_128x128"; }
        else { p.bm = 64; p.bn = 64; p.name = "mfma16_64x64"; }
        p.edge = (m % p.bm) || (n % p.bn) || (k % M16_BK);
    } else {
        p.fam = FAM_MFMAW;
        if (m > 64 || n > 64) { p.bm = 128; p.bn = 128; p.name = (dtype == RP_DTYPE_FLOAT32) ? "mfma32_128x128" : "mfma64_128x128"; }
        else { p.bm = 64; p.bn = 64; p.name = (dtype == RP_DTYPE_FLOAT32) ? "mfma32_64x64" : "mfma64_64x64"; }
        p.edge = (m % p.bm) || (n % p.bn) || (k % (dtype == RP_DTYPE_FLOAT32 ? 16 : 8));
    }
    return p;
}

template <typename T>
static int launch_generic(const GemmArgs& g) {
    dim3 grid((g.n + 63) / 64, (g.m + 63) / 64, g.batch);
    hipLaunchKernelGGL(gemm_generic_kernel<T>, grid, dim3(256), 0, current_stream(), g);
    return check_launch("gemm_generic_kernel") ? 0 : -1;
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC>
static int launch_mfma16_edge(const GemmArgs& g, bool edge) {
    int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    dim3 grid(scheduled_grid(tiles_m, tiles_n), g.batch);
    size_t smem = 2 * (size_t)(m16_tile_elems(BM, A_MC) + m16_tile_elems(BN, B_MC)) * 2;
    if (edge) {
        auto kern = gemm_mfma16_kernel<T, BM, BN, A_MC, B_MC, true>;
        if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
        hipLaunchKernelGGL(kern, grid, dim3(256), smem, current_stream(), g, tiles_m, tiles_n);
    } else {
        auto kern = gemm_mfma16_kernel<T, BM, BN, A_MC, B_MC, false>;
        if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
        hipLaunchKernelGGL(kern, grid, dim3(256), smem, current_stream(), g, tiles_m, tiles_n);
    }
    return check_launch("gemm_mfma16_kernel") ? 0 : -1;
}

template <typename T, int BM, int BN>
static int launch_mfma16_layout(const GemmArgs& g, const Plan& p) {
    if (!p.a_mc && p.b_mc) return launch_mfma16_edge<T, BM, BN, false, true>(g, p.edge);
    if (!p.a_mc && !p.b_mc) return launch_mfma16_edge<T, BM, BN, false, false>(g, p.edge);
    if (p.a_mc && p.b_mc) return launch_mfma16_edge<T, BM, BN, true, true>(g, p.edge);
    return launch_mfma16_edge<T, BM, BN, true, false>(g, p.edge);
}

template <typename T>
static int launch_mfma16(const GemmArgs& g, const Plan& p) {
    if (p.bm == 256) return launch_mfma16_layout<T, 256, 256>(g, p);
    if (p.bm == 128) return launch_mfma16_layout<T, 128, 128>(g, p);
    return launch_mfma16_layout<T, 64, 64>(g, p);
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC>
static int launch_mfmaw_edge(const GemmArgs& g, bool edge) {
    int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    dim3 grid(scheduled_grid(tiles_m, tiles_n), g.batch);
    if (edge) hipLaunchKernelGGL((gemm_mfmaw_kernel<T, BM, BN, A_MC, B_MC, true>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n);
    else      hipLaunchKernelGGL((gemm_mfmaw_kernel<T, BM, BN, A_MC, B_MC, false>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n);
    return check_launch("gemm_mfmaw_kernel") ? 0 : -1;
}

template <typename T, int BM, int BN>
static int launch_mfmaw_layout(const GemmArgs& g, const Plan& p) {
    if (!p.a_mc && p.b_mc) return launch_mfmaw_edge<T, BM, BN, false, true>(g, p.edge);
    if (!p.a_mc && !p.b_mc) return launch_mfmaw_edge<T, BM, BN, false, false>(g, p.edge);
    if (p.a_mc && p.b_mc) return launch_mfmaw_edge<T, BM, BN, true, true>(g, p.edge);
    return launch_mfmaw_edge<T, BM, BN, true, false>(g, p.edge);
}

template <typename T>
static int launch_mfmaw(const GemmArgs& g, const Plan& p) {
    if (p.bm == 128) return launch_mfmaw_layout<T, 128, 128>(g, p);
    return launch_mfmaw_layout<T, 64, 64>(g, p);
}

template <typename T>
static int launch_skinny(const GemmArgs& g) {
    using Acc = typename traits<T>::acc;
    constexpr int VEC = 16 / sizeof(T);
    int groups = (g.n + 64 * VEC - 1) / (64 * VEC);
    // aim for ~8 blocks per CU in flight overall, at least 32 k rows per wave
    int want = (256 * 8 + groups - 1) / groups;
    int max_split = g.k / 128 > 0 ? g.k / 128 : 1;
    int nsplit = want < max_split ? want : max_split;
    if (nsplit < 1) nsplit = 1;
    int k_per_block = (g.k + nsplit - 1) / nsplit;
    if (k_per_block > 1024) k_per_block = 1024;          // bounds the LDS copy of A (1024 x 8 floats = 32 KB)
    k_per_block = (k_per_block + 3) & ~3;
    nsplit = (g.k + k_per_block - 1) / k_per_block;
    if (nsplit > 65535) { set_error("gemm skinny: k too large"); return -1; }
    void* ws = nullptr;
    if (nsplit > 1 && rp_hip_malloc(&ws, (size_t)nsplit * g.m * g.n * sizeof(Acc)) != 0) return -1;
    dim3 grid(groups, nsplit);
    if (g.m <= 1)      hipLaunchKernelGGL((gemm_skinny_kernel<T, 1>), grid, dim3(256), (size_t)k_per_block * 1 * 4, current_stream(), g, (float*)ws, k_per_block);
    else if (g.m <= 2) hipLaunchKernelGGL((gemm_skinny_kernel<T, 2>), grid, dim3(256), (size_t)k_per_block * 2 * 4, current_stream(), g, (float*)ws, k_per_block);
    else if (g.m <= 4) hipLaunchKernelGGL((gemm_skinny_kernel<T, 4>), grid, dim3(256), (size_t)k_per_block * 4 * 4, current_stream(), g, (float*)ws, k_per_block);
    else               hipLaunchKernelGGL((gemm_skinny_kernel<T, 8>), grid, dim3(256), (size_t)k_per_block * 8 * 4, current_stream(), g, (float*)ws, k_per_block);
    bool ok = check_launch("gemm_skinny_kernel");
    if (ws) rp_hip_free(ws);      // stream-ordered reuse: the pool hands it out again only to later work on this stream
    return ok ? 0 : -1;
}

template <typename T>
static int run_gemm(const GemmArgs& g, int dtype) {
    Plan p = make_plan(g.batch, g.m, g.k, g.n, g.a_rs, g.a_cs, g.b_rs, g.b_cs, g.c_rs, g.c_cs, g.a_bs, g.b_bs, dtype);
    if (p.fam != FAM_GENERIC && !(aligned16(g.A) && aligned16(g.B))) p.fam = FAM_GENERIC;
    if constexpr (sizeof(T) == 2) {
        if (p.fam == FAM_MFMA16) return launch_mfma16<T>(g, p);
    } else {
        if (p.fam == FAM_MFMAW) return launch_mfmaw<T>(g, p);
    }
    if (p.fam == FAM_SKINNY) {
        if constexpr (sizeof(T) != 8) return launch_skinny<T>(g);
    }
    return launch_generic<T>(g);
}

}  // namespace rp

using namespace rp;

extern "C" {

int rp_hip_gemm_strided_batched(void* C, const void* A, const void* B, const void* bias,
                                int batch, int m, int k, int n,
                                long long a_bs, long long a_rs, long long a_cs,
                                long long b_bs, long long b_rs, long long b_cs,
                                long long c_bs, long long c_rs, long long c_cs,
                                int accumulate, int dtype) {
    if (!C || !A || !B || batch <= 0 || m <= 0 || k <= 0 || n <= 0) {
        set_error("rp_hip_gemm_strided_batched: null operand or non-positive extent (batch=%d m=%d k=%d n=%d)", batch, m, k, n);
        return -1;
    }
    if (!dtype_size(dtype)) { set_error("rp_hip_gemm_strided_batched: unsupported dtype %d", dtype); return -1; }
    if (a_rs < 0 || a_cs < 0 || b_rs < 0 || b_cs < 0 || c_rs < 0 || c_cs < 0 || a_bs < 0 || b_bs < 0 || c_bs < 0) {
        set_error("rp_hip_gemm_strided_batched: negative stride");
        return -1;
    }
    if (batch > 65535) { set_error("rp_hip_gemm_strided_batched: batch %d exceeds 65535", batch); return -1; }
    GemmArgs g{C, A, B, bias, batch, m, k, n, a_bs, a_rs, a_cs, b_bs, b_rs, b_cs, c_bs, c_rs, c_cs, accumulate};
    RP_DISPATCH_DTYPE(dtype, return run_gemm<T>(g, dtype));
    return -1;
}

int matmul_kernel_device(void* C, const void* A, const void* B, int m, int k, int n, int dtype) {
    return rp_hip_gemm_strided_batched(C, A, B, nullptr, 1, m, k, n, 0, k, 1, 0, n, 1, 0, n, 1, 0, dtype);
}

const char* rp_hip_gemm_kernel_name(int batch, int m, int k, int n, long long a_rs, long long a_cs,
                                    long long b_rs, long long b_cs, long long c_rs, long long c_cs, int dtype) {
    if (batch <= 0 || m <= 0 || k <= 0 || n <= 0 || !dtype_size(dtype)) return "invalid";
    Plan p = make_plan(batch, m, k, n, a_rs, a_cs, b_rs, b_cs, c_rs, c_cs, 0, 0, dtype);
    if (p.fam == FAM_SKINNY && dtype == RP_DTYPE_FLOAT64) return "generic";
    return p.name;
}

}  // extern "C"
