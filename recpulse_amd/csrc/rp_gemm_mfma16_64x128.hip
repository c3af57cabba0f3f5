// bf16 / fp16 MFMA GEMM, 64 x 128 block tile (1 x 4 waves of 64 x 32).
#include "rp_gemm_mfma16_kernel.h"

namespace rp {

int launch_mfma16_64x128(const GemmArgs& g, const Plan& p, int dtype) { return m16_launch_tile_dtype<64, 128, 1>(g, p, dtype); }

}  // namespace rp
