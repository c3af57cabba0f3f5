// bf16 / fp16 MFMA GEMM, 64 x 64 block tile (2 x 2 waves).
#include "rp_gemm_mfma16_kernel.h"

namespace rp {

int launch_mfma16_64(const GemmArgs& g, const Plan& p, int dtype) { return m16_launch_tile_dtype<64, 64, 2>(g, p, dtype); }

}  // namespace rp
