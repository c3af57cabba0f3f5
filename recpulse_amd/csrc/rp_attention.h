// Argument blocks and launch entry points shared by the attention kernels of the 16-bit types (rp_attention.hip)
// and of float32 (rp_attention_f32.hip).
#pragma once
#include "rp_common.h"

namespace rp {

struct AttnArgs {
    void* O;
    const void* Q;
    const void* K;
    const void* V;
    float* L;                   // optional [batch, sq] row-wise log-sum-exp of the scaled scores
    int batch, sq, sk;
    long long q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs;      // in elements; the head dimension is contiguous
    float scale;
};

constexpr int AT_KEYS = 32;                 // keys per step
constexpr int AT_QROWS = 128;               // query rows per workgroup (32 per wave)

struct AttnBwdArgs {
    void* dQ; void* dK; void* dV;           // dense [batch, s, d]
    const void* Q; const void* K; const void* V; const void* O; const void* dO;
    const float* L;                         // [batch, sq] log-sum-exp rows from the forward
    float* Dq;                              // [batch, sq] row dots of dO and O: written by the dQ kernel, read by the dK/dV kernel
    int batch, sq, sk;
    long long q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs, do_bs, do_rs;
    float scale;
};

// Which (row tile, batch entry) this workgroup takes.  Workgroups are dealt to the 8 XCDs round robin in launch order, so
// with the plain (blockIdx.x, blockIdx.y) the row tiles of one batch entry land on different XCDs and each of their L2s
// fetches that entry's K and V (Q and dO in the dK/dV kernel) for itself: the fused forward at [192, 512, 64] read 113 MB
// where 38 MB are its inputs.  Here XCD x takes a contiguous eighth of the (tile, entry) pairs, in launch order: the tiles
// of a batch entry run at the same time on one XCD.
#ifdef __HIPCC__
__device__ __forceinline__ void attn_block(int& tile, int& z) {
    const unsigned nx = gridDim.x, total = nx * gridDim.y, linear = blockIdx.x + nx * blockIdx.y;
    unsigned id = linear;
    if (total % 8 == 0) id = (linear % 8) * (total / 8) + linear / 8;
    tile = (int)(id % nx);
    z = (int)(id / nx);
}
#endif

// float32 kernels (v_mfma_f32_32x32x2_f32), head dimension 32, 64 or 128
int launch_attention_f32(const AttnArgs& g, int d);
int launch_attention_bwd_f32(const AttnBwdArgs& g, int d);

}  // namespace rp
