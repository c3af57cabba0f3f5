// The two non-MFMA GEMM kernels: the generic strided kernel that takes any
// shape and stride, and the skinny split-k kernel for a few rows of A against a
// row-major B (bound by streaming B from HBM).
#include "rp_gemm.h"
#include "rp_gemm_splitk_finish.h"

#include <mutex>

namespace rp {

// ============================================================================
// generic: 64x64 output tile, 16-deep k slabs, 256 threads each owning 4x4.
// ============================================================================
// With SPLITK (one matrix, fp32 accumulation) the grid's z axis splits k instead of walking the batch: every
// block writes its fp32 partial tile [split][m][n] to a workspace and the combine kernel finishes.
template <typename T, bool SPLITK>
__global__ void __launch_bounds__(256) gemm_generic_kernel(GemmArgs g, float* partials, int k_per_split) {
    using Acc = typename traits<T>::acc;
    constexpr int TM = 64, TN = 64, TK = 16;
    __shared__ Acc As[TK][TM + 1];
    __shared__ Acc Bs[TK][TN + 1];

    const int z = SPLITK ? 0 : blockIdx.z;
    const int kbeg = SPLITK ? blockIdx.z * k_per_split : 0;
    const int kend = SPLITK ? (kbeg + k_per_split < g.k ? kbeg + k_per_split : g.k) : g.k;
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

    // slab k0 sits in registers while slab k0 - TK is being multiplied out of LDS, so the latency of
    // the strided element loads overlaps the FMAs instead of adding to every slab
    Acc ra[4], rb[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = t + 256 * i;
            int kk = a_kfast ? id % TK : id / TM;
            int r = a_kfast ? id / TK : id % TM;
            int gm = m0 + r, gk = k0 + kk;
            ra[i] = (gm < g.m && gk < kend) ? widen(A[(long long)gm * g.a_rs + (long long)gk * g.a_cs]) : (Acc)0;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = t + 256 * i;
            int kk = b_nfast ? id / TN : id % TK;
            int c = b_nfast ? id % TN : id / TK;
            int gn = n0 + c, gk = k0 + kk;
            rb[i] = (gn < g.n && gk < kend) ? widen(B[(long long)gk * g.b_rs + (long long)gn * g.b_cs]) : (Acc)0;
        }
    };
    fetch(kbeg);
    for (int k0 = kbeg; k0 < kend; k0 += TK) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = t + 256 * i;
            As[a_kfast ? id % TK : id / TM][a_kfast ? id / TK : id % TM] = ra[i];
            Bs[b_nfast ? id / TN : id % TK][b_nfast ? id % TN : id / TK] = rb[i];
        }
        __syncthreads();
        if (k0 + TK < kend) fetch(k0 + TK);
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
            if constexpr (SPLITK) {
                partials[((long long)blockIdx.z * g.m + gm) * g.n + gn] = (float)acc[i][j];
                continue;
            }
            T* p = C + (long long)gm * g.c_rs + (long long)gn * g.c_cs;
            T old = g.accumulate ? *p : T{};
            T bv = bias ? bias[gn] : T{};
            *p = finish<T>(acc[i][j], bias != nullptr, bv, g.accumulate != 0, old);
        }
    }
}

// ============================================================================
// skinny: m <= 8 rows of A against a row-major B (unit column stride).
// The cost is streaming B once from HBM.  Each lane owns VEC adjacent columns
// (one 16-byte load per k row) and a wave covers 64*VEC columns.  The 8 waves
// of a block share a column group and take interleaved k rows of the block's
// k range; they combine through LDS in a fixed tree.  The grid's second axis
// splits k further: split partials go to a workspace and a small second kernel
// adds them in split order (so the result does not depend on scheduling) and
// runs the epilogue.  (For these few-microsecond launches the second kernel
// is cheaper than the three device-scope round trips of a single-launch
// "last block reduces" finish; the long streaming kernel of the 16-bit
// few-row path uses that finish, see splitk_arrival_counters.)
// ============================================================================
constexpr int SK_THREADS = 512, SK_WAVES = SK_THREADS / 64;

template <typename T, int MROWS>
__global__ void __launch_bounds__(SK_THREADS) gemm_skinny_kernel(GemmArgs g, float* partials, int k_per_block) {
    constexpr int VEC = 16 / sizeof(T);
    extern __shared__ __attribute__((aligned(16))) float sk_lds[];   // first A's slice [k_per_block][MROWS], later the wave-combine buffer
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col0 = (blockIdx.x * 64 + lane) * VEC;
    const int split = blockIdx.y, nsplit = gridDim.y;
    const bool col_ok = col0 < g.n;          // n is a multiple of VEC, so a vector is wholly in or out
    const T* A = (const T*)g.A;
    const T* B = (const T*)g.B;

    float acc[MROWS][VEC];
#pragma unroll
    for (int r = 0; r < MROWS; r++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[r][e] = 0.f;

    const int kb = split * k_per_block;
    const int ke = kb + k_per_block < g.k ? kb + k_per_block : g.k;
    const int klen = ke - kb;
    // this block's slice of A, widened once, rows beyond m as zeros
    for (int i = threadIdx.x; i < MROWS * klen; i += SK_THREADS) {
        int r = i / klen, kl = i - r * klen;
        sk_lds[kl * MROWS + r] = (r < g.m) ? widen(A[(long long)r * g.a_rs + (long long)(kb + kl) * g.a_cs]) : 0.f;
    }
    __syncthreads();

    if (col_ok) {
        const T* bp = B + col0 + (long long)kb * g.b_rs;
        constexpr int U = 8;
        int kl = wave;
        for (; kl + SK_WAVES * (U - 1) < klen; kl += SK_WAVES * U) {
            u32x4_t raw[U];
#pragma unroll
            for (int u = 0; u < U; u++) raw[u] = __builtin_nontemporal_load((const u32x4_t*)(bp + (long long)(kl + SK_WAVES * u) * g.b_rs));
#pragma unroll
            for (int u = 0; u < U; u++) {
                T bv[VEC];
                memcpy(bv, &raw[u], 16);
                float bw[VEC];
#pragma unroll
                for (int e = 0; e < VEC; e++) bw[e] = widen(bv[e]);
#pragma unroll
                for (int r = 0; r < MROWS; r++) {
                    float a = sk_lds[(kl + SK_WAVES * u) * MROWS + r];
#pragma unroll
                    for (int e = 0; e < VEC; e++) acc[r][e] += a * bw[e];
                }
            }
        }
        for (; kl < klen; kl += SK_WAVES) {
            u32x4_t raw = *(const u32x4_t*)(bp + (long long)kl * g.b_rs);
            T bv[VEC];
            memcpy(bv, &raw, 16);
#pragma unroll
            for (int r = 0; r < MROWS; r++) {
                float a = sk_lds[kl * MROWS + r];
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[r][e] += a * widen(bv[e]);
            }
        }
    }
    __syncthreads();            // everyone is done with A's slice; the buffer now carries wave partials

    // fixed tree over the 8 waves: (4..7 -> 0..3), (2..3 -> 0..1), (1 -> 0)
    constexpr int WSZ = MROWS * VEC * 64;
#pragma unroll
    for (int half = SK_WAVES / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
            float* dst = sk_lds + (wave - half) * WSZ;
#pragma unroll
            for (int r = 0; r < MROWS; r++)
#pragma unroll
                for (int e = 0; e < VEC; e++) dst[(r * VEC + e) * 64 + lane] = acc[r][e];
        }
        __syncthreads();
        if (wave < half) {
            const float* src = sk_lds + wave * WSZ;
#pragma unroll
            for (int r = 0; r < MROWS; r++)
#pragma unroll
                for (int e = 0; e < VEC; e++) acc[r][e] += src[(r * VEC + e) * 64 + lane];
        }
        __syncthreads();
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

    // partial layout: [split][row][n] fp32; a second kernel adds the splits in order and runs the epilogue
    if (wave == 0 && col_ok) {
#pragma unroll
        for (int r = 0; r < MROWS; r++) {
            if (r >= g.m) break;
            float* q = partials + ((long long)split * g.m + r) * g.n + col0;
#pragma unroll
            for (int e = 0; e < VEC; e += 4) *(f32x4_t*)(q + e) = f32x4_t{acc[r][e], acc[r][e + 1], acc[r][e + 2], acc[r][e + 3]};
        }
    }
}

// Sum the k-split partials [nsplit][m][n] in split order (fixed, so results do not depend on scheduling),
// then bias / accumulate / narrow.  One thread per 4 adjacent columns of one row (n is a multiple of 4);
// loads are issued eight splits at a time so the sum is not a chain of dependent memory latencies.
template <typename T>
__global__ void __launch_bounds__(256) gemm_splitk_combine_kernel(GemmArgs g, const float* partials, int nsplit, int part_rows) {
    const int quads = g.n / 4;
    const int item = blockIdx.x * 256 + threadIdx.x;
    if (item >= g.m * quads) return;
    const int r = item / quads, c0 = (item - r * quads) * 4;
    f32x4_t sum = {0.f, 0.f, 0.f, 0.f};
    const long long split_stride = (long long)part_rows * g.n;
    const float* q = partials + (long long)blockIdx.y * nsplit * split_stride + (long long)r * g.n + c0;      // matrix blockIdx.y of the batch
    int s = 0;
    for (; s + 8 <= nsplit; s += 8) {
        f32x4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = *(const f32x4_t*)(q + (s + u) * split_stride);
#pragma unroll
        for (int u = 0; u < 8; u++) sum += v[u];
    }
    for (; s < nsplit; s++) sum += *(const f32x4_t*)(q + s * split_stride);
    if constexpr (sizeof(T) == 2) {                    // 16-bit outputs: one 8-byte store where the layout allows, no branch per value without bias and accumulation
        const SplitkOutput<T> out(g, (long long)blockIdx.y * g.c_bs);
        if (out.plain()) out.store_quad_plain(r, c0, sum);
        else out.store_quad(r, c0, sum);
    } else {
        T* C = (T*)g.C + (long long)blockIdx.y * g.c_bs;
        const T* bias = (const T*)g.bias;
        const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            T* p = C + (long long)r * g.c_rs + (long long)(c0 + e) * g.c_cs;
            T old = accum ? *p : T{};
            *p = finish<T>(sum[e], has_bias, has_bias ? bias[c0 + e] : T{}, accum, old);
        }
    }
}

int* splitk_arrival_counters(long long tiles, size_t partial_bytes, bool* failed) {
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static int* blocks[MAX_DEVICES] = {};
    *failed = false;
    if (path_disabled("one_launch_splitk") || tiles > SPLITK_MAX_TILES || partial_bytes >= (1ull << 31)) return nullptr;
    if (noalloc_active()) {                              // inside the entry point that allocates nothing: its fixed counters
        int* fixed = noalloc_arrival_counters();
        if (!fixed) *failed = true;
        return fixed;
    }
    int dev = 0;
    if (rp_hip_get_device(&dev) != 0) { *failed = true; return nullptr; }
    if (dev < 0 || dev >= MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (blocks[dev]) return blocks[dev];
    // First use on this device.  The counters must read zero for every stream that will ever use them, so they are
    // created outside any recording and cleared with a blocking fill; a first use that happens while a graph is being
    // recorded takes the two-launch path instead (the next eager call creates the block).
    if (stream_is_capturing()) return nullptr;
    void* p = nullptr;
    if (!check_hip(hipMalloc(&p, SPLITK_MAX_TILES * sizeof(int)), "hipMalloc (split-k counters)")) { *failed = true; return nullptr; }
    if (!check_hip(hipMemset(p, 0, SPLITK_MAX_TILES * sizeof(int)), "hipMemset (split-k counters)") ||
        !check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize (split-k counters)")) { (void)hipFree(p); *failed = true; return nullptr; }
    blocks[dev] = (int*)p;
    return blocks[dev];
}

// the same for any n: one thread per output element
template <typename T>
__global__ void __launch_bounds__(256) gemm_splitk_combine_scalar_kernel(GemmArgs g, const float* partials, int nsplit, int part_rows) {
    const int item = blockIdx.x * 256 + threadIdx.x;
    if (item >= g.m * g.n) return;
    const int r = item / g.n, c = item - r * g.n;
    const long long split_stride = (long long)part_rows * g.n;
    const float* q = partials + (long long)blockIdx.y * nsplit * split_stride + (long long)r * g.n + c;
    float sum = 0.f;
    int s = 0;
    for (; s + 8 <= nsplit; s += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = q[(s + u) * split_stride];
#pragma unroll
        for (int u = 0; u < 8; u++) sum += v[u];
    }
    for (; s < nsplit; s++) sum += q[s * split_stride];
    T* C = (T*)g.C + (long long)blockIdx.y * g.c_bs;
    const T* bias = (const T*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    T* p = C + (long long)r * g.c_rs + (long long)c * g.c_cs;
    T old = accum ? *p : T{};
    *p = finish<T>(sum, has_bias, has_bias ? bias[c] : T{}, accum, old);
}

int launch_splitk_combine(const GemmArgs& g, const float* partials, int nsplit, int part_rows, int dtype) {
    if (g.n % 4) {
        dim3 sgrid((g.m * g.n + 255) / 256, g.batch);
        switch (dtype) {
            case RP_DTYPE_FLOAT32:  hipLaunchKernelGGL(gemm_splitk_combine_scalar_kernel<float>, sgrid, dim3(256), 0, current_stream(), g, partials, nsplit, part_rows); break;
            case RP_DTYPE_FLOAT16:  hipLaunchKernelGGL(gemm_splitk_combine_scalar_kernel<f16_t>, sgrid, dim3(256), 0, current_stream(), g, partials, nsplit, part_rows); break;
            case RP_DTYPE_BFLOAT16: hipLaunchKernelGGL(gemm_splitk_combine_scalar_kernel<bf16_t>, sgrid, dim3(256), 0, current_stream(), g, partials, nsplit, part_rows); break;
            default: set_error("split-k combine: unsupported dtype %d", dtype); return -1;
        }
        return check_launch("gemm_splitk_combine_scalar_kernel") ? 0 : -1;
    }
    int items = g.m * (g.n / 4);
    dim3 grid((items + 255) / 256, g.batch);
    switch (dtype) {
        case RP_DTYPE_FLOAT32:  hipLaunchKernelGGL(gemm_splitk_combine_kernel<float>, grid, dim3(256), 0, current_stream(), g, partials, nsplit, part_rows); break;
        case RP_DTYPE_FLOAT16:  hipLaunchKernelGGL(gemm_splitk_combine_kernel<f16_t>, grid, dim3(256), 0, current_stream(), g, partials, nsplit, part_rows); break;
        case RP_DTYPE_BFLOAT16: hipLaunchKernelGGL(gemm_splitk_combine_kernel<bf16_t>, grid, dim3(256), 0, current_stream(), g, partials, nsplit, part_rows); break;
        default: set_error("split-k combine: unsupported dtype %d", dtype); return -1;
    }
    return check_launch("gemm_splitk_combine_kernel") ? 0 : -1;
}

template <typename T>
static int launch_generic_t(const GemmArgs& g) {
    const int tiles = ((g.n + 63) / 64) * ((g.m + 63) / 64);
    // A single small output with a deep k would run on a handful of CUs: split k across about 128 blocks, each
    // at least two 16-deep slabs, and add the partials in split order afterwards (fp32 accumulation only).
    if (sizeof(typename traits<T>::acc) == 4 && g.batch == 1 && tiles < 64 && g.k >= 64) {
        int nsplit = (128 + tiles - 1) / tiles;
        if (nsplit > g.k / 32) nsplit = g.k / 32;
        int k_per_split = ((g.k + nsplit - 1) / nsplit + 15) / 16 * 16;
        nsplit = (g.k + k_per_split - 1) / k_per_split;
        if (nsplit > 1) {
            void* ws = nullptr;
            if (gemm_workspace(&ws, (size_t)nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
            dim3 grid((g.n + 63) / 64, (g.m + 63) / 64, nsplit);
            hipLaunchKernelGGL((gemm_generic_kernel<T, true>), grid, dim3(256), 0, current_stream(), g, (float*)ws, k_per_split);
            int rc = check_launch("gemm_generic_kernel") ? 0 : -1;
            if (rc == 0) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, traits<T>::code);
            gemm_workspace_release(ws);      // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
            return rc;
        }
    }
    dim3 grid((g.n + 63) / 64, (g.m + 63) / 64, g.batch);
    hipLaunchKernelGGL((gemm_generic_kernel<T, false>), grid, dim3(256), 0, current_stream(), g, nullptr, 0);
    return check_launch("gemm_generic_kernel") ? 0 : -1;
}

template <typename T>
static int launch_skinny_t(const GemmArgs& g) {
    constexpr int VEC = 16 / sizeof(T);
    int groups = (g.n + 64 * VEC - 1) / (64 * VEC);
    // enough blocks to put two on every CU, each wave keeping at least 32 k rows
    const int want = (512 + groups - 1) / groups;
    int k_per_block = (g.k + want - 1) / want;
    if (k_per_block < 256) k_per_block = 256;
    if (k_per_block > 2048) k_per_block = 2048;            // bounds the LDS copy of A (2048 x 8 floats = 64 KB)
    k_per_block = (k_per_block + SK_WAVES - 1) / SK_WAVES * SK_WAVES;
    int nsplit = (g.k + k_per_block - 1) / k_per_block;
    if (nsplit > 65535) { set_error("gemm skinny: k too large"); return -1; }
    void* ws = nullptr;
    if (nsplit > 1 && gemm_workspace(&ws, (size_t)nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
    dim3 grid(groups, nsplit);
    auto smem = [&](int mrows) {
        size_t a_slice = (size_t)k_per_block * mrows * 4, combine = (size_t)(SK_WAVES / 2) * mrows * VEC * 64 * 4;
        return a_slice > combine ? a_slice : combine;
    };
    hipError_t attr = hipSuccess;
    if (g.m <= 1)      hipLaunchKernelGGL((gemm_skinny_kernel<T, 1>), grid, dim3(SK_THREADS), smem(1), current_stream(), g, (float*)ws, k_per_block);
    else if (g.m <= 2) hipLaunchKernelGGL((gemm_skinny_kernel<T, 2>), grid, dim3(SK_THREADS), smem(2), current_stream(), g, (float*)ws, k_per_block);
    else if (g.m <= 4) hipLaunchKernelGGL((gemm_skinny_kernel<T, 4>), grid, dim3(SK_THREADS), smem(4), current_stream(), g, (float*)ws, k_per_block);
    else {
        auto kern = gemm_skinny_kernel<T, 8>;
        if (smem(8) > 64 * 1024) attr = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem(8));
        if (attr == hipSuccess) hipLaunchKernelGGL(kern, grid, dim3(SK_THREADS), smem(8), current_stream(), g, (float*)ws, k_per_block);
    }
    bool ok = check_hip(attr, "hipFuncSetAttribute") && check_launch("gemm_skinny_kernel");
    if (ok && nsplit > 1) ok = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, traits<T>::code) == 0;
    if (ws) gemm_workspace_release(ws);      // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return ok ? 0 : -1;
}

int launch_generic(const GemmArgs& g, int dtype) {
    RP_DISPATCH_DTYPE(dtype, return launch_generic_t<T>(g));
    return -1;
}

int launch_skinny(const GemmArgs& g, int dtype) {
    switch (dtype) {
        case RP_DTYPE_FLOAT32:  return launch_skinny_t<float>(g);
        case RP_DTYPE_FLOAT16:  return launch_skinny_t<f16_t>(g);
        case RP_DTYPE_BFLOAT16: return launch_skinny_t<bf16_t>(g);
        default: set_error("skinny GEMM: unsupported dtype %d", dtype); return -1;
    }
}

}  // namespace rp
