// fp32 GEMMs whose whole output is a few hundred 16 x 16 tiles (the layers of a small MLP: 256 x 784 by 784 x 256 and
// smaller).  Such a product is over in microseconds, so what it costs is latency: a 64 x 64 tile leaves 240 CUs
// idle unless k is split over blocks, and a split needs a second launch (or a device-scope exchange) to add the
// partial tiles, which costs as much again as the multiplication.  Here a workgroup owns one 16 x 16 tile of C, its four
// waves each take a quarter of k with v_mfma_f32_16x16x4_f32, and the four partial tiles meet in LDS: one launch, a
// fixed order of additions, up to about a thousand workgroups in flight.  Operands are read straight from global
// memory with any strides (16-byte loads along k where k is the unit-stride axis); nothing is staged, every value is
// used once per workgroup.
#include "rp_gemm.h"

namespace rp {

typedef __attribute__((ext_vector_type(4))) float f32x4t_t;

// MFMA step j of a 16-deep chunk uses k = chunk + 4*(lane / 16) + j for the four k slots: a permutation of k that both
// operands share, chosen so that a lane's four values are consecutive in k.
template <bool VEC>
__device__ __forceinline__ void tiny_load4(float (&v)[4], const float* p, long long k_stride, int k0, int k_end) {
    if (VEC && k0 + 4 <= k_end) {
        const f32x4t_t x = *(const f32x4t_t*)(p + k0);
        v[0] = x[0]; v[1] = x[1]; v[2] = x[2]; v[3] = x[3];
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = (k0 + j < k_end) ? p[(long long)(k0 + j) * k_stride] : 0.f;
    }
}

// One 16 x 16 tile of C_z (tile row tm, tile column tn) by the 256 threads of a workgroup; red: 3 x 256 floats of LDS.
template <bool A_VEC, bool B_VEC>
__device__ __forceinline__ void tiny_tile(const GemmArgs& g, int z, int tm, int tn, float (*red)[256]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int m0 = tm * 16, n0 = tn * 16;
    // rows past m and columns past n read the last valid row / column: their products land in output elements that
    // are never written
    const int row = m0 + r16 < g.m ? m0 + r16 : g.m - 1;
    const int col = n0 + r16 < g.n ? n0 + r16 : g.n - 1;
    const float* ap = (const float*)g.A + (long long)z * g.a_bs + (long long)row * g.a_rs;
    const float* bp = (const float*)g.B + (long long)z * g.b_bs + (long long)col * g.b_cs;

    // chunks of 16 k, a contiguous quarter of them per wave
    const int chunks = (g.k + 15) / 16, per_wave = (chunks + 3) / 4;
    const int c_begin = wave * per_wave, c_end = c_begin + per_wave < chunks ? c_begin + per_wave : chunks;
    f32x4t_t acc = {0.f, 0.f, 0.f, 0.f};
    int c = c_begin;
    for (; c + 2 <= c_end; c += 2) {                 // two chunks at a time: sixteen values in flight per lane
        float a0[4], b0[4], a1[4], b1[4];
        const int k0 = 16 * c + 4 * kq, k1 = k0 + 16;
        tiny_load4<A_VEC>(a0, ap, g.a_cs, k0, g.k);
        tiny_load4<B_VEC>(b0, bp, g.b_rs, k0, g.k);
        tiny_load4<A_VEC>(a1, ap, g.a_cs, k1, g.k);
        tiny_load4<B_VEC>(b1, bp, g.b_rs, k1, g.k);
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[j], b0[j], acc, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[j], b1[j], acc, 0, 0, 0);
    }
    if (c < c_end) {
        float a0[4], b0[4];
        const int k0 = 16 * c + 4 * kq;
        tiny_load4<A_VEC>(a0, ap, g.a_cs, k0, g.k);
        tiny_load4<B_VEC>(b0, bp, g.b_rs, k0, g.k);
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[j], b0[j], acc, 0, 0, 0);
    }

    // the four partial tiles meet in LDS and are added in wave order
    if (wave > 0) *(f32x4t_t*)&red[wave - 1][lane * 4] = acc;
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 0; w < 3; w++) {
        const f32x4t_t part = *(const f32x4t_t*)&red[w][lane * 4];
        acc += part;
    }
    // accumulator register v of lane (kq, r16) is C[m0 + 4*kq + v][n0 + r16]
    const int gc = n0 + r16;
    if (gc >= g.n) return;
    const float* bias = (const float*)g.bias;
    const bool has_bias = bias != nullptr, accum = g.accumulate != 0;
    const float bv = has_bias ? bias[gc] : 0.f;
    float* cp = (float*)g.C + (long long)z * g.c_bs + (long long)gc * g.c_cs;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int gr = m0 + 4 * kq + v;
        if (gr >= g.m) break;
        float* p = cp + (long long)gr * g.c_rs;
        *p = finish<float>(acc[v], has_bias, bv, accum, accum ? *p : 0.f);
    }
}

template <bool A_VEC, bool B_VEC>
__global__ void __launch_bounds__(256) gemm_tiny32_kernel(GemmArgs g) {
    __shared__ float red[3][256];
    tiny_tile<A_VEC, B_VEC>(g, blockIdx.z, blockIdx.y, blockIdx.x, red);
}

// 16-byte loads along k need k to be the unit-stride axis, rows a whole number of vectors apart and an aligned base
static bool tiny_a_vec(const GemmArgs& g) { return g.a_cs == 1 && g.a_rs % 4 == 0 && g.a_bs % 4 == 0 && ((uintptr_t)g.A & 15) == 0; }
static bool tiny_b_vec(const GemmArgs& g) { return g.b_rs == 1 && g.b_cs % 4 == 0 && g.b_bs % 4 == 0 && ((uintptr_t)g.B & 15) == 0; }

// The backward of a small Linear layer in one launch: the tiles of dX = dY . W^T, then the tiles of dW = X^T . dY, then
// the column sums of dY for db (one thread per column, rows added top to bottom as reduce_rows does).  Every block
// does what it would have done in three separate launches, so the bits are the same; what goes away is two launch
// latencies, which is most of the time of such a layer.  Either GEMM or the sums may be absent (zero tiles / blocks).
struct ColumnSums {
    float* out;
    const float* grad;       // [rows, cols], dense
    int rows, cols, accumulate;
};

template <bool A_VEC, bool B_VEC>
__device__ __forceinline__ void tiny_tile_of(const GemmArgs& g, int tile, float (*red)[256]) {
    const int tiles_n = (g.n + 15) / 16;
    tiny_tile<A_VEC, B_VEC>(g, 0, tile / tiles_n, tile % tiles_n, red);
}

__device__ __forceinline__ void tiny_tile_any(const GemmArgs& g, bool a_vec, bool b_vec, int tile, float (*red)[256]) {
    if (a_vec && b_vec) tiny_tile_of<true, true>(g, tile, red);
    else if (a_vec) tiny_tile_of<true, false>(g, tile, red);
    else if (b_vec) tiny_tile_of<false, true>(g, tile, red);
    else tiny_tile_of<false, false>(g, tile, red);
}

__global__ void __launch_bounds__(256) linear_backward_tiny32_kernel(GemmArgs gx, GemmArgs gw, ColumnSums db, int tiles_x, int tiles_w, int vec_flags) {
    __shared__ float red[3][256];
    const int b = blockIdx.x;
    if (b < tiles_x) { tiny_tile_any(gx, vec_flags & 1, vec_flags & 2, b, red); return; }
    if (b < tiles_x + tiles_w) { tiny_tile_any(gw, vec_flags & 4, vec_flags & 8, b - tiles_x, red); return; }
    const int j = (b - tiles_x - tiles_w) * 256 + threadIdx.x;
    if (j >= db.cols) return;
    float s = 0.f;
    const float* p = db.grad + j;
    int i = 0;
    constexpr int U = 16;                       // independent loads in flight; the adds stay in row order
    for (; i + U <= db.rows; i += U) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = p[(size_t)(i + u) * db.cols];
#pragma unroll
        for (int u = 0; u < U; u++) s += v[u];
    }
    for (; i < db.rows; i++) s += p[(size_t)i * db.cols];
    db.out[j] = db.accumulate ? db.out[j] + s : s;
}

// gx / gw: batch 1, fp32, each taken by the tiny kernel on its own (the caller checks); m == 0 marks an absent GEMM,
// cols == 0 absent sums.
int launch_linear_backward_tiny(const GemmArgs& gx, const GemmArgs& gw, void* db, const void* dy, int rows, int cols, int accumulate_db) {
    const int tiles_x = gx.m > 0 ? ((gx.m + 15) / 16) * ((gx.n + 15) / 16) : 0;
    const int tiles_w = gw.m > 0 ? ((gw.m + 15) / 16) * ((gw.n + 15) / 16) : 0;
    const int blocks_db = db ? (cols + 255) / 256 : 0;
    if (tiles_x + tiles_w + blocks_db == 0) return 0;
    ColumnSums cs{(float*)db, (const float*)dy, rows, db ? cols : 0, accumulate_db};
    const int flags = (gx.m > 0 && tiny_a_vec(gx) ? 1 : 0) | (gx.m > 0 && tiny_b_vec(gx) ? 2 : 0) | (gw.m > 0 && tiny_a_vec(gw) ? 4 : 0) | (gw.m > 0 && tiny_b_vec(gw) ? 8 : 0);
    hipLaunchKernelGGL(linear_backward_tiny32_kernel, dim3(tiles_x + tiles_w + blocks_db), dim3(256), 0, current_stream(), gx, gw, cs, tiles_x, tiles_w, flags);
    return check_launch("linear_backward_tiny32_kernel") ? 0 : -1;
}

int launch_tiny(const GemmArgs& g, int dtype) {
    if (dtype != RP_DTYPE_FLOAT32) { set_error("tiny GEMM: float32 only (dtype %d)", dtype); return -1; }
    const dim3 grid((g.n + 15) / 16, (g.m + 15) / 16, g.batch);
    if (grid.y > 65535 || grid.z > 65535) { set_error("tiny GEMM: output too large for the grid"); return -1; }
    const bool a_vec = tiny_a_vec(g), b_vec = tiny_b_vec(g);
    if (a_vec && b_vec) hipLaunchKernelGGL((gemm_tiny32_kernel<true, true>), grid, dim3(256), 0, current_stream(), g);
    else if (a_vec) hipLaunchKernelGGL((gemm_tiny32_kernel<true, false>), grid, dim3(256), 0, current_stream(), g);
    else if (b_vec) hipLaunchKernelGGL((gemm_tiny32_kernel<false, true>), grid, dim3(256), 0, current_stream(), g);
    else hipLaunchKernelGGL((gemm_tiny32_kernel<false, false>), grid, dim3(256), 0, current_stream(), g);
    return check_launch("gemm_tiny32_kernel") ? 0 : -1;
}

}  // namespace rp
