// fp32 GEMM with a short reduction (k <= 64): every wave multiplies straight out of registers.
//
// With k this short a tile has no k loop to pipeline: a block of the LDS kernel loads its two slabs, waits,
// multiplies for a few microseconds and stores, and two such blocks per CU cannot hide each other's waiting.
// Here nothing goes through LDS and nothing is synchronised.  v_mfma_f32_32x32x2_f32 takes one float per lane
// and operand: lane (r, h) = (lane % 32, lane / 32) supplies free index r at the k of "slot" h.  Sums may run
// over k in any order as long as both operands use the same one, so MFMA step t pairs k = t (h = 0) with
// k = 32 + t (h = 1): a lane owns the 32 consecutive k values [32h, 32h + 32) of its row or column.  For an
// operand with unit stride along k those are 128 contiguous bytes, eight 16-byte loads; for an operand with
// unit stride along its free index, step t is one 4-byte load whose 32 lanes read 128 contiguous bytes.
// A wave computes a 64 x 64 patch (2 x 2 MFMA tiles, 128 MFMAs) from 64 rows of A and 64 columns of B held in
// 128 registers; a block is 2 x 2 waves, so neighbouring waves re-read each other's rows from the vector cache,
// and two blocks per CU overlap one's loads and stores with the other's MFMAs.  The accumulators go to memory
// as they lie: register v of a tile is one row's 32 adjacent columns across 32 lanes, 128 contiguous bytes.
#include "rp_gemm.h"

#include <type_traits>

namespace rp {

constexpr int D32_BM = 128, D32_BN = 128, D32_MAXK = 64;
constexpr uint32_t D32_OOB = 0x80000000u;

// One operand's 2 tiles x 32 k values per lane.  KC: unit stride along k; MC: unit stride along the free index.
// fs / ks: strides of the free index and of k in elements; first: first free index of the wave's patch; extent: free extent.
template <bool MC>
struct D32Operand {
    float v[2][32];
    __device__ __forceinline__ void load(const float* base, long long span_bytes, long long fs, long long ks, int first, int extent, int k, int r, int h) {
        const int n = span_bytes <= 0 ? 0 : (span_bytes > 0x7fffffffll ? 0x7fffffff : (int)span_bytes);
        __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, n, 0x00020000);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int f = first + 32 * i + r;
            if constexpr (!MC) {
                // rows past the extent lie past the descriptor's end and read zero; k past the end is masked here
                const uint32_t off = (uint32_t)(((long long)f * fs + 32 * h) * 4);
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    const bool in = f < extent && 32 * h + 4 * q < k;
                    const u32x4_t raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, in ? (int)(off + 16 * q) : (int)D32_OOB, 0, 0);
                    const f32x4_t w = __builtin_bit_cast(f32x4_t, raw);      // (cast the whole vector: a bit cast of one element of it reads element 0 every time)
                    v[i][4 * q + 0] = w[0]; v[i][4 * q + 1] = w[1]; v[i][4 * q + 2] = w[2]; v[i][4 * q + 3] = w[3];
                }
            } else {
                // k past the end lies past the descriptor's end; free indices past the extent are masked here
                const uint32_t off = (f < extent) ? (uint32_t)(((long long)(32 * h) * ks + f) * 4) : D32_OOB;
#pragma unroll
                for (int t = 0; t < 32; t++) {
                    const bool in = f < extent && 32 * h + t < k;
                    v[i][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, in ? (int)off : (int)D32_OOB, (int)(t * ks * 4), 0));
                }
            }
        }
    }
};

template <bool A_MC, bool B_MC>
__global__ void __launch_bounds__(256, 2) gemm_direct32_kernel(GemmArgs g, int tiles_m, int tiles_n) {
    TileCoord tc = schedule_tile(blockIdx.x, tiles_m, tiles_n);
    if (!tc.valid) return;
    const int z = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int m0 = tc.tm * D32_BM + (wave >> 1) * 64, n0 = tc.tn * D32_BN + (wave & 1) * 64;      // the wave's patch
    if (m0 >= g.m || n0 >= g.n) return;               // a patch wholly outside the output (no barriers in this kernel)
    const float* A = (const float*)g.A + (long long)z * g.a_bs;
    const float* B = (const float*)g.B + (long long)z * g.b_bs;
    const long long a_span = ((long long)(g.m - 1) * g.a_rs + (long long)(g.k - 1) * g.a_cs + 1) * 4;
    const long long b_span = ((long long)(g.n - 1) * g.b_cs + (long long)(g.k - 1) * g.b_rs + 1) * 4;

    D32Operand<A_MC> a;
    D32Operand<B_MC> b;
    a.load(A, a_span, g.a_rs, g.a_cs, m0, g.m, g.k, r, h);
    b.load(B, b_span, g.b_cs, g.b_rs, n0, g.n, g.k, r, h);

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
    // every load above is in flight before the first MFMA waits for its operands (the steps are straight-line code:
    // behind a branch the compiler would issue each group of loads only where it is consumed)
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, 32>([&](auto tc_) {
        constexpr int t = decltype(tc_)::value;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i][t], b.v[j][t], acc[i][j], 0, 0, 0);
    });

    // epilogue: accumulator register v of tile (i, j) is row 32i + 8(v / 4) + 4h + v % 4, column 32j + r
    float* C = (float*)g.C + (long long)z * g.c_bs;
    const float* bias = (const float*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    if (m0 + 64 <= g.m && n0 + 64 <= g.n && !accum) {
        // a whole patch that overwrites C: 64 stores, nothing to test per element
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int gn = n0 + 32 * j + r;
            const float bv = has_bias ? bias[gn] : 0.f;
            float* pcol = C + (long long)(m0 + 4 * h) * g.c_rs + (long long)gn * g.c_cs;
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    pcol[(long long)(32 * i + 8 * (v / 4) + (v % 4)) * g.c_rs] = finish<float>(acc[i][j][v], has_bias, bv, false, 0.f);
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int gn = n0 + 32 * j + r;
        if (gn >= g.n) continue;
        const float bv = has_bias ? bias[gn] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int gm = m0 + 32 * i + 8 * (v / 4) + 4 * h + (v % 4);
                if (gm >= g.m) continue;
                float* pc = C + (long long)gm * g.c_rs + (long long)gn * g.c_cs;
                const float old = accum ? *pc : 0.f;
                *pc = finish<float>(acc[i][j][v], has_bias, bv, accum, old);
            }
    }
}

// Whether this kernel takes the product: fp32, 32 < k <= 64 (all 32 steps are always issued), both operands with a unit stride and 16-byte rows where k is
// the unit-stride axis, offsets that fit the 32-bit addressing of buffer loads, none of the segment / fold options.
bool direct32_takes(const GemmArgs& g) {
    if (g.k > D32_MAXK || g.k <= 32 || g.seg_k || g.seg_n || g.c_fold_from || g.bias_by_row) return false;
    const bool a_kc = g.a_cs == 1, a_mc = g.a_rs == 1, b_kc = g.b_rs == 1, b_mc = g.b_cs == 1;
    if (!(a_kc || a_mc) || !(b_kc || b_mc)) return false;
    if (a_kc && !(g.k % 4 == 0 && g.a_rs % 4 == 0 && g.a_bs % 4 == 0 && ((uintptr_t)g.A & 15) == 0)) return false;
    if (!a_kc && ((uintptr_t)g.A & 3)) return false;
    if (b_kc && !(g.k % 4 == 0 && g.b_cs % 4 == 0 && g.b_bs % 4 == 0 && ((uintptr_t)g.B & 15) == 0)) return false;
    if (!b_kc && ((uintptr_t)g.B & 3)) return false;
    const long long a_span = ((long long)(g.m - 1) * g.a_rs + (long long)(g.k - 1) * g.a_cs + 1) * 4;
    const long long b_span = ((long long)(g.n - 1) * g.b_cs + (long long)(g.k - 1) * g.b_rs + 1) * 4;
    return a_span < (1ll << 31) && b_span < (1ll << 31) && g.batch <= 65535;
}

int launch_direct32(const GemmArgs& g) {
    const int tiles_m = (g.m + D32_BM - 1) / D32_BM, tiles_n = (g.n + D32_BN - 1) / D32_BN;
    dim3 grid(scheduled_grid(tiles_m, tiles_n), g.batch);
    const bool a_mc = g.a_cs != 1, b_mc = g.b_rs != 1;          // KC wins when both strides are 1 (extent-1 corner cases)
    if (!a_mc && !b_mc) hipLaunchKernelGGL((gemm_direct32_kernel<false, false>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n);
    else if (!a_mc && b_mc) hipLaunchKernelGGL((gemm_direct32_kernel<false, true>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n);
    else if (a_mc && !b_mc) hipLaunchKernelGGL((gemm_direct32_kernel<true, false>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n);
    else hipLaunchKernelGGL((gemm_direct32_kernel<true, true>), grid, dim3(256), 0, current_stream(), g, tiles_m, tiles_n);
    return check_launch("gemm_direct32_kernel") ? 0 : -1;
}

}  // namespace rp
