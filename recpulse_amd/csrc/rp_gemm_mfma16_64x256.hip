// bf16 / fp16 MFMA GEMM, 64 x 256 block tile (1 x 4 waves of 64 x 64): outputs of at most 64 rows, where a
// 128 x 128 tile would spend half of its MFMAs on rows that do not exist.
#include "rp_gemm_mfma16_kernel.h"

namespace rp {

int launch_mfma16_64x256(const GemmArgs& g, const Plan& p, int dtype) { return m16_launch_tile_dtype<64, 256, 1>(g, p, dtype); }

}  // namespace rp
