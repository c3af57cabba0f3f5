// bf16 / fp16 MFMA GEMM for few rows (m <= 32) and deep k: a 32 x 128 block tile with the 4 waves side by
// side along n, k split across the grid's z axis so that enough blocks stream B to saturate HBM, fp32 partials
// combined by a second kernel.
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
    constexpr int BN = 128;
    const int tiles_n = (g.n + BN - 1) / BN;
    // about three blocks per CU in flight, each split at least four slabs deep
    int nsplit = (768 + tiles_n - 1) / tiles_n;
    int max_split = g.k / (4 * M16_BK) > 0 ? g.k / (4 * M16_BK) : 1;
    if (nsplit > max_split) nsplit = max_split;
    int k_per_split = ((g.k + nsplit - 1) / nsplit + M16_BK - 1) / M16_BK * M16_BK;
    nsplit = (g.k + k_per_split - 1) / k_per_split;
    void* ws = nullptr;
    if (rp_hip_malloc(&ws, (size_t)nsplit * g.m * g.n * sizeof(float)) != 0) return -1;
    int rc;
    if (dtype == RP_DTYPE_BFLOAT16) rc = launch_skinny16_t<bf16_t>(g, p, (float*)ws, nsplit, k_per_split);
    else if (dtype == RP_DTYPE_FLOAT16) rc = launch_skinny16_t<f16_t>(g, p, (float*)ws, nsplit, k_per_split);
    else { set_error("mfma16 skinny GEMM: unsupported dtype %d", dtype); rc = -1; }
    if (rc == 0) rc = launch_splitk_combine(g, (const float*)ws, nsplit, g.m, dtype);
    rp_hip_free(ws);          // stream-ordered reuse: the pool hands it out again only to later work on this stream
    return rc;
}

}  // namespace rp
