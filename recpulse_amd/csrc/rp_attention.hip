// Fused attention forward for bf16 / fp16: O = softmax(scale * Q * K^T) * V without ever writing the score matrix.
//
// The reference composes attention from op_matmul, op_mul_scalar, op_softmax and op_matmul
// (ops/ops.c:6816-6884, 6022-6086, 5721-5788), which streams the [S, S] score and probability matrices through
// memory four times; at 512 x 512 per head they outweigh Q, K, V and O eight to one.  Here a workgroup owns 128 query
// rows of one head (a wave 32 of them) and walks the keys 32 at a time:
//
//   S^T tile   = K_blk (32 keys x D) * Q_w^T (D x 32 queries)        MFMA 32x32x16, fp32 accumulate
//   online softmax on S^T: in this orientation a lane owns ONE query (its column) and 16 keys (its registers), so the
//                running maximum and sum are per-lane scalars; the two lanes that share a query exchange one value
//   O^T tile  += V_blk^T (D x 32 keys) * P^T (32 keys x 32 queries)
//
// Both products are written transposed on purpose: the accumulator layout of S^T (lane = query column, registers =
// key rows 8*(v/4) + 4*(lane/32) + v%4) is, after narrowing to 16 bits, exactly a B operand of the second product whose
// k slots are those same keys, so the probabilities go from one MFMA to the next without leaving the lane; and O^T has
// the same lane = query mapping, so the rescaling factor of the online softmax is a per-lane scalar too.
// Q and K fragments are 16-byte global loads straight into MFMA operand registers (rows are d-contiguous); V is the one
// operand that needs a transpose (k slots = keys, rows = d) and goes through LDS with ds_read_tr16_b64.
// Probabilities are narrowed to the tensor dtype before the second product (as the reference's P is), accumulation is
// fp32 throughout, and the scores themselves are never rounded to 16 bits (the reference rounds S and S*scale).
#include "rp_gemm_mfma16_kernel.h"

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

template <typename T, int D>
__global__ void __launch_bounds__(256) attention_fwd16_kernel(AttnArgs g) {
    static_assert(D % 32 == 0 && D <= 128, "head dimension: a multiple of 32 up to 128");
    constexpr int KS = D / 16;              // k-steps of the first product
    constexpr int DT = D / 32;              // 32-row tiles of O^T
    constexpr int VP = m16_mc_pitch(D);     // LDS pitch of a V row in elements, the GEMM kernels' conflict-free one for this read pattern
    constexpr int VPIECES = AT_KEYS * D / 8 / 256 > 0 ? AT_KEYS * D / 8 / 256 : 1;      // 16-byte pieces of a V block per thread
    __shared__ __attribute__((aligned(16))) uint16_t vlds[2][AT_KEYS * VP];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, c = lane & 31;
    const int z = blockIdx.y;
    const int q0 = blockIdx.x * AT_QROWS + wave * 32;               // this wave's first query row
    const uint16_t* Q = (const uint16_t*)g.Q + (long long)z * g.q_bs;
    const uint16_t* K = (const uint16_t*)g.K + (long long)z * g.k_bs;
    const uint16_t* V = (const uint16_t*)g.V + (long long)z * g.v_bs;
    const float sc = g.scale * 1.44269504088896341f;                // scores are kept in units of log2 e

    // Q^T as a B operand: lane (h, c) holds d = 16*ks + 8h .. +7 of query row q0 + c (zero beyond sq)
    const char* q_end = (const char*)(Q + ((long long)(g.sq - 1) * g.q_rs + D));
    const char* q_base = (const char*)(Q + (long long)q0 * g.q_rs);
    const __amdgpu_buffer_rsrc_t q_rsrc = m16_rsrc(q_base, q0 < g.sq ? (long long)(q_end - q_base) : 0);
    s16x8_t qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
        qf[ks] = __builtin_bit_cast(s16x8_t, __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, (int)(((long long)c * g.q_rs + 16 * ks + 8 * h) * 2), 0, 0));

    // K as an A operand: lane (h, c) holds d = 16*ks + 8h .. +7 of key kb + c; rows past sk read zeros and are masked below
    const char* k_end = (const char*)(K + ((long long)(g.sk - 1) * g.k_rs + D));
    const uint32_t k_voff = (uint32_t)(((long long)c * g.k_rs + 8 * h) * 2);
    auto load_k = [&](s16x8_t (&kf)[KS], int kb) {
        const char* kp = (const char*)(K + (long long)kb * g.k_rs);
        const __amdgpu_buffer_rsrc_t k_rsrc = m16_rsrc(kp, kb < g.sk ? (long long)(k_end - kp) : 0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kf[ks] = __builtin_bit_cast(s16x8_t, __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, (int)k_voff, 32 * ks, 0));
    };

    // V block [32 keys][D] into LDS, 16 bytes per thread and piece
    const char* v_end = (const char*)(V + ((long long)(g.sk - 1) * g.v_rs + D));
    auto load_v = [&](u32x4_t (&vr)[VPIECES], int kb) {
        const char* vp = (const char*)(V + (long long)kb * g.v_rs);
        const __amdgpu_buffer_rsrc_t v_rsrc = m16_rsrc(vp, kb < g.sk ? (long long)(v_end - vp) : 0);
#pragma unroll
        for (int i = 0; i < VPIECES; i++) {
            const int id = threadIdx.x + 256 * i, key = id / (D / 8), d8 = (id % (D / 8)) * 8;
            const bool live = AT_KEYS * D / 8 >= 256 || id < AT_KEYS * D / 8;
            vr[i] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, live ? (int)(((long long)key * g.v_rs + d8) * 2) : (int)M16_OOB, 0, 0);
        }
    };
    auto store_v = [&](const u32x4_t (&vr)[VPIECES], uint16_t* stage) {
#pragma unroll
        for (int i = 0; i < VPIECES; i++) {
            const int id = threadIdx.x + 256 * i, key = id / (D / 8), d8 = (id % (D / 8)) * 8;
            if (AT_KEYS * D / 8 >= 256 || id < AT_KEYS * D / 8) *(u32x4_t*)(stage + key * VP + d8) = vr[i];
        }
    };
    // V^T as an A operand of the second product: lane row d = 32*dt + c, k slot e of MFMA t <-> key 16t + 8*(e/4) + 4h + e%4.
    // ds_read_tr16_b64: in each 16-lane group, source lane s points at 4 consecutive d of key row s/4 and destination lane
    // j receives d index j of key rows 0..3: read H of MFMA t therefore starts at key 16t + 8H + 4h.
    const int grp = lane >> 4, s16 = lane & 15;
    const int v_fr0 = (4 * (grp >> 1) + (s16 >> 2)) * VP + 16 * (grp & 1) + 4 * (s16 & 3);
    auto read_v = [&](const uint16_t* stage, int dt, int t) {
        s16x8_t f;
#pragma unroll
        for (int H = 0; H < 2; H++) {
            s16x4_t q4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(lds_u16*)(stage + v_fr0 + (16 * t + 8 * H) * VP + 32 * dt));
            f[4 * H + 0] = q4[0]; f[4 * H + 1] = q4[1]; f[4 * H + 2] = q4[2]; f[4 * H + 3] = q4[3];
        }
        return f;
    };

    f32x16_t ot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) ot[dt][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;            // running maximum (log2 units) and this lane's share of the running sum

    const int nblocks = (g.sk + AT_KEYS - 1) / AT_KEYS;
    s16x8_t kf[2][KS];
    u32x4_t vr[VPIECES];
    load_k(kf[0], 0);
    load_v(vr, 0);
    store_v(vr, vlds[0]);
    load_k(kf[1], AT_KEYS);
    load_v(vr, AT_KEYS);
    __syncthreads();

    auto step = [&](int blk, auto slotc) {
        constexpr int SLOT = decltype(slotc)::value;
        const int kb = blk * AT_KEYS;
        const uint16_t* stage = vlds[blk & 1];
        // scores of 32 keys x 32 queries
        f32x16_t st;
#pragma unroll
        for (int v = 0; v < 16; v++) st[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) st = mfma16_ops<T>::mma(kf[SLOT][ks], qf[ks], st);
        load_k(kf[SLOT], kb + 2 * AT_KEYS);                 // this slot's next use is two blocks on
        // V of the next block goes to the other stage (everyone left it at the previous barrier); then request the one after
        store_v(vr, vlds[(blk & 1) ^ 1]);
        load_v(vr, kb + 2 * AT_KEYS);

        float mx = m_run;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int key = kb + 8 * (v / 4) + 4 * h + (v % 4);
            st[v] = key < g.sk ? st[v] * sc : -INFINITY;
            mx = st[v] > mx ? st[v] : mx;
        }
        const float other = __shfl_xor(mx, 32, 64);         // the lane that holds this query's other 16 keys
        mx = other > mx ? other : mx;
        // a query row beyond sq (or a block of masked keys met first) keeps mx = -inf: exp2(-inf - -inf) must not produce NaN
        const float m_use = mx == -INFINITY ? 0.f : mx;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        float psum = 0.f;
        T p[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float e = __builtin_amdgcn_exp2f(st[v] - m_use);
            p[v] = narrow<T>(e);
            psum += widen(p[v]);                            // the sum counts the probabilities the second product sees
        }
        l_run = l_run * alpha + psum;
        m_run = mx;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++) ot[dt][v] *= alpha;
        // O^T += V^T * P^T, 16 keys per MFMA
#pragma unroll
        for (int t = 0; t < 2; t++) {
            s16x8_t pb;
#pragma unroll
            for (int e = 0; e < 8; e++) pb[e] = (short)p[8 * t + e].bits;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) ot[dt] = mfma16_ops<T>::mma(read_v(stage, dt, t), pb, ot[dt]);
        }
        __syncthreads();                                    // next stage is written, this one is free
    };
    for (int blk = 0; blk < nblocks; blk += 2) {
        step(blk, std::integral_constant<int, 0>{});
        if (blk + 1 < nblocks) step(blk + 1, std::integral_constant<int, 1>{});
    }

    // finish: the two lanes of a query add their sums; O[q][d] = O^T[d][q] / l
    const float l_all = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
    const int q = q0 + c;
    if (q < g.sq) {
        T* orow = (T*)g.O + (long long)z * g.o_bs + (long long)q * g.o_rs;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                // registers 4*v4 .. 4*v4+3 are four consecutive d: 32*dt + 8*v4 + 4h + (0..3)
                T out[4];
#pragma unroll
                for (int e = 0; e < 4; e++) out[e] = narrow<T>(ot[dt][4 * v4 + e] * inv);
                uint2 w;
                memcpy(&w, out, 8);
                *(uint2*)(orow + 32 * dt + 8 * v4 + 4 * h) = w;
            }
        if (g.L && h == 0) g.L[(long long)z * g.sq + q] = (m_run + __builtin_amdgcn_logf(l_all)) * 0.693147180559945309f;   // natural log of the row sum of exp(scale * s)
    }
}

template <typename T>
static int launch_attention_t(const AttnArgs& g, int d) {
    dim3 grid((g.sq + AT_QROWS - 1) / AT_QROWS, g.batch);
    switch (d) {
        case 32:  hipLaunchKernelGGL((attention_fwd16_kernel<T, 32>), grid, dim3(256), 0, current_stream(), g); break;
        case 64:  hipLaunchKernelGGL((attention_fwd16_kernel<T, 64>), grid, dim3(256), 0, current_stream(), g); break;
        case 128: hipLaunchKernelGGL((attention_fwd16_kernel<T, 128>), grid, dim3(256), 0, current_stream(), g); break;
        default: set_error("rp_hip_attention_forward: head dimension %d (supported: 32, 64, 128)", d); return -1;
    }
    return check_launch("attention_fwd16_kernel") ? 0 : -1;
}

}  // namespace rp

using namespace rp;

extern "C" int rp_hip_attention_forward(void* O, const void* Q, const void* K, const void* V, float* lse,
                                        int batch, int sq, int sk, int d,
                                        long long q_bs, long long q_rs, long long k_bs, long long k_rs,
                                        long long v_bs, long long v_rs, long long o_bs, long long o_rs,
                                        double scale, int dtype) {
    if (!O || !Q || !K || !V || batch <= 0 || sq <= 0 || sk <= 0 || d <= 0) {
        set_error("rp_hip_attention_forward: null operand or non-positive extent (batch=%d sq=%d sk=%d d=%d)", batch, sq, sk, d);
        return -1;
    }
    if (dtype != RP_DTYPE_BFLOAT16 && dtype != RP_DTYPE_FLOAT16) { set_error("rp_hip_attention_forward: bfloat16 / float16 only (dtype %d)", dtype); return -1; }
    const long long strides[] = {q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs};
    for (long long s : strides)
        if (s < 0 || s % 8) { set_error("rp_hip_attention_forward: strides must be non-negative multiples of 8 elements"); return -1; }
    if (q_rs >= (1ll << 22) || k_rs >= (1ll << 22) || v_rs >= (1ll << 22)) { set_error("rp_hip_attention_forward: row stride too large"); return -1; }
    if (((uintptr_t)O | (uintptr_t)Q | (uintptr_t)K | (uintptr_t)V) & 15) { set_error("rp_hip_attention_forward: operands must be 16-byte aligned"); return -1; }
    constexpr int MAX_BATCH = 65535;
    for (int b0 = 0; b0 < batch; b0 += MAX_BATCH) {
        const int nb = batch - b0 < MAX_BATCH ? batch - b0 : MAX_BATCH;
        AttnArgs g{(char*)O + b0 * o_bs * 2, (const char*)Q + b0 * q_bs * 2, (const char*)K + b0 * k_bs * 2, (const char*)V + b0 * v_bs * 2,
                   lse ? lse + (long long)b0 * sq : nullptr, nb, sq, sk, q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs, (float)scale};
        int rc = dtype == RP_DTYPE_BFLOAT16 ? launch_attention_t<bf16_t>(g, d) : launch_attention_t<f16_t>(g, d);
        if (rc != 0) return -1;
    }
    return 0;
}
