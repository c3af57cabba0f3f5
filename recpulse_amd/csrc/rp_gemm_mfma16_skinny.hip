// bf16 / fp16 GEMMs with few rows and deep k: the cost is streaming B once from HBM.
//
// Row-major A times row-major B with at most 32 rows takes the streaming kernel (rp_gemm_mfma16_stream128.hip), in
// which B never touches LDS and the k splits are added inside the same launch by the last block to arrive.  Other
// operand layouts, more rows, and the shapes that kernel declines take the tiled kernel with a 32 x 128 block tile
// below, whose fp32 partials a second kernel combines.  Both split k across the grid so that enough waves stream B to
// saturate HBM, and both add the splits in split order.
#include "rp_gemm_mfma16_kernel.h"


namespace rp {

template <typename T>
static int launch_skinny16_t(const GemmArgs& g, const Plan& p, float* partials, int nsplit, int k_per_split) {
    constexpr int BM = 32, BN = 128, WGM = 1;
    if (!p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, false, true, true, true>(g, partials, nsplit, k_per_split);
    if (!p.a_mc && !p.b_mc) return m16_launch<T, BM, BN, WGM, false, false, true, true>(g, partials, nsplit, k_per_split);
    if (p.a_mc && p.b_mc) return m16_launch<T, BM, BN, WGM, true, true, true, true>(g, partials, nsplit, k_per_split);
    return m16_launch<T, BM, BN, WGM, true, false, true, true>(g, partials, nsplit, k_per_split);
}

int launch_mfma16_skinny(const GemmArgs& g, const Plan& p, int dtype) {
    if (dtype != RP_DTYPE_BFLOAT16 && dtype != RP_DTYPE_FLOAT16) { set_error("mfma16 skinny GEMM: unsupported dtype %d", dtype); return -1; }
    if (!p.a_mc && p.b_mc && stream128_takes(g)) return launch_stream128(g, dtype);
    constexpr int BN = 128;
    const int tiles = ((g.n + BN - 1) / BN) * ((g.m + 31) / 32) * g.batch;
    // about three blocks per CU in flight, each split at least four slabs deep
    int nsplit = (768 + tiles - 1) / tiles;
    int max_split = g.k / (4 * M16_BK) > 0 ? g.k / (4 * M16_BK) : 1;
    if (nsplit > max_split) nsplit = max_split;
    int k_per_split = ((g.k + nsplit - 1) / nsplit + M16_BK - 1) / M16_BK * M16_BK;
    nsplit = (g.k + k_per_split - 1) / k_per_split;
    void* ws = nullptr;
    if (gemm_workspace(&ws, (size_t)g.batch * nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
    int rc;
    if (dtype == RP_DTYPE_BFLOAT16) rc = launch_skinny16_t<bf16_t>(g, p, (float*)ws, nsplit, k_per_split);
    else rc = launch_skinny16_t<f16_t>(g, p, (float*)ws, nsplit, k_per_split);
    if (rc == 0) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, dtype);
    gemm_workspace_release(ws);          // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

}  // namespace rp
