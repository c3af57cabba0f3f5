// fp32 / fp64 MFMA GEMM kernels and their launcher.
#include "rp_gemm.h"

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

// With SPLITK the grid's z axis splits k (k_per_split is a multiple of BK): every block writes its fp32 partial
// tile [split][m][n] to a workspace and the shared combine kernel finishes (fp32 only).
template <typename T, int BM, int BN, bool A_MC, bool B_MC, bool EDGE, bool SPLITK>
__global__ void __launch_bounds__(256) gemm_mfmaw_kernel(GemmArgs g, int tiles_m, int tiles_n, float* partials, int k_per_split) {
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

    T ra[BM * BK / 256], rb[BN * BK / 256];
    const int nslabs = (klen + BK - 1) / BK;
    mw_load_slab<T, BM, A_MC, EDGE>(ra, A, a_fs, a_ks, m0, 0, g.m, klen, t);
    mw_load_slab<T, BN, B_MC, EDGE>(rb, B, b_fs, b_ks, n0, 0, g.n, klen, t);
    mw_store_slab<T, BM, A_MC>(ra, smem, t);
    mw_store_slab<T, BN, B_MC>(rb, smem + A_ELEMS, t);
    __syncthreads();

    const int lf = lane % MT, lk = lane / MT;         // lane's free index and k index inside one MFMA
    for (int s = 0; s < nslabs; s++) {
        const int cur = s & 1;
        const bool more = (s + 1 < nslabs);
        if (more) {
            mw_load_slab<T, BM, A_MC, EDGE>(ra, A, a_fs, a_ks, m0, (s + 1) * BK, g.m, klen, t);
            mw_load_slab<T, BN, B_MC, EDGE>(rb, B, b_fs, b_ks, n0, (s + 1) * BK, g.n, klen, t);
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
                    if constexpr (SPLITK) {
                        partials[((long long)blockIdx.z * g.m + gm) * g.n + gn] = (float)acc[i][j][v];
                    } else {
                        T* p = C + (long long)gm * g.c_rs + (long long)gn * g.c_cs;
                        T old = accum ? *p : (T)0;
                        *p = finish<T>(acc[i][j][v], has_bias, bv, accum, old);
                    }
                }
            }
        }
    }
}

template <typename T, int BM, int BN, bool A_MC, bool B_MC>
static int launch_mfmaw_edge(const GemmArgs& g, bool edge, float* partials, int nsplit, int k_per_split) {
    int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    if (nsplit > 1) {
        if constexpr (sizeof(T) == 4) {           // split-k partials are fp32; always the predicated variant
            dim3 grid(scheduled_grid(tiles_m, tiles_n), g.batch, nsplit);
            hipLaunchKernelGGL((gemm_mfmaw_kernel<T, BM, BN, A_MC, B_MC, true, true>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n, partials, k_per_split);
            return check_launch("gemm_mfmaw_kernel") ? 0 : -1;
        }
        set_error("mfmaw GEMM: split-k is fp32 only");
        return -1;
    }
    dim3 grid(scheduled_grid(tiles_m, tiles_n), g.batch);
    if (edge) hipLaunchKernelGGL((gemm_mfmaw_kernel<T, BM, BN, A_MC, B_MC, true, false>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n, nullptr, 0);
    else      hipLaunchKernelGGL((gemm_mfmaw_kernel<T, BM, BN, A_MC, B_MC, false, false>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n, nullptr, 0);
    return check_launch("gemm_mfmaw_kernel") ? 0 : -1;
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
    // least four slabs deep), and add the partials in split order afterwards.  fp32 only, one matrix at a time.
    int nsplit = 1, k_per_split = 0;
    constexpr int BK = mfmaw_cfg<T>::BK;
    if (sizeof(T) == 4 && g.batch == 1 && p.bm == 64 && g.n % 4 == 0) {
        int tiles = ((g.m + 63) / 64) * ((g.n + 63) / 64);
        int want = (256 + tiles - 1) / tiles, deep = g.k / (4 * BK);
        nsplit = want < deep ? want : deep;
        if (nsplit > 1) {
            k_per_split = ((g.k + nsplit - 1) / nsplit + BK - 1) / BK * BK;
            nsplit = (g.k + k_per_split - 1) / k_per_split;
        }
        if (nsplit < 2) nsplit = 1;
    }
    void* ws = nullptr;
    if (nsplit > 1 && rp_hip_malloc(&ws, (size_t)nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
    int rc = (p.bm == 128) ? launch_mfmaw_layout<T, 128, 128>(g, p, (float*)ws, nsplit, k_per_split)
                           : launch_mfmaw_layout<T, 64, 64>(g, p, (float*)ws, nsplit, k_per_split);
    if (rc == 0 && nsplit > 1) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, traits<T>::code);
    if (ws) rp_hip_free(ws);          // stream-ordered reuse: the pool hands it out again only to later work on this stream
    return rc;
}

int launch_mfmaw(const GemmArgs& g, const Plan& p, int dtype) {
    if (dtype == RP_DTYPE_FLOAT32) return launch_mfmaw_t<float>(g, p);
    if (dtype == RP_DTYPE_FLOAT64) return launch_mfmaw_t<double>(g, p);
    set_error("mfmaw GEMM: unsupported dtype %d", dtype);
    return -1;
}

}  // namespace rp
