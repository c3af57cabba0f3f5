// bf16 / fp16 MFMA GEMM, 128 x 128 block tile (2 x 2 waves).
#include "rp_gemm_mfma16_kernel.h"

namespace rp {

int launch_mfma16_128(const GemmArgs& g, const Plan& p, int dtype) { return m16_launch_tile_dtype<128, 128, 2>(g, p, dtype); }

}  // namespace rp
