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

// float32 kernels (v_mfma_f32_32x32x2_f32), head dimension 32 or 64
int launch_attention_f32(const AttnArgs& g, int d);
int launch_attention_bwd_f32(const AttnBwdArgs& g, int d);

}  // namespace rp
