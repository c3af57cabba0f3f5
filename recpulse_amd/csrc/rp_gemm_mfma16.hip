// bf16 / fp16 MFMA GEMM: tile selection across the per-tile translation units.
#include "rp_gemm.h"

namespace rp {

int launch_mfma16_256(const GemmArgs& g, const Plan& p, int dtype);
int launch_mfma16_128(const GemmArgs& g, const Plan& p, int dtype);
int launch_mfma16_64(const GemmArgs& g, const Plan& p, int dtype);
int launch_mfma16_64x256(const GemmArgs& g, const Plan& p, int dtype);
int launch_mfma16_64x128(const GemmArgs& g, const Plan& p, int dtype);
int launch_mfma16_skinny(const GemmArgs& g, const Plan& p, int dtype);

int launch_mfma16(const GemmArgs& g, const Plan& p, int dtype) {
    if (p.fam == FAM_MFMA16_SKINNY) return launch_mfma16_skinny(g, p, dtype);
    if (p.bm == 256) return launch_mfma16_256(g, p, dtype);
    if (p.bm == 128) return launch_mfma16_128(g, p, dtype);
    if (p.bn == 256) return launch_mfma16_64x256(g, p, dtype);
    if (p.bn == 128) return launch_mfma16_64x128(g, p, dtype);
    return launch_mfma16_64(g, p, dtype);
}

}  // namespace rp
