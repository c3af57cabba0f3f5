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
// Q fragments are 16-byte global loads straight into MFMA operand registers, once per wave (rows are d-contiguous).
// K and V blocks are staged in LDS by the whole workgroup with row-contiguous loads: K fragments are read back with
// ds_read_b128, V, the one operand that needs a transpose (k slots = keys, rows = d), with ds_read_tr16_b64.
// Probabilities are narrowed to the tensor dtype before the second product (as the reference's P is), accumulation is
// fp32 throughout, and the scores themselves are never rounded to 16 bits (the reference rounds S and S*scale).
#include "rp_gemm_mfma16_kernel.h"
#include "rp_attention.h"

namespace rp {

// Two fp32 values to a pair of T with the hardware's packed round-to-nearest-even conversion (one instruction for
// two values).  The probabilities and the score gradients packed with it exist only inside the fused kernels, as MFMA
// operands; tensors that leave a kernel are narrowed with the reference's rule (narrow<T>).
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) __bf16 v2;
    const v2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, v);
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) _Float16 v2;
    const v2 v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, v);
}
// slots 8t .. 8t+7 of sixteen fp32 values as one MFMA B operand
template <typename T> __device__ __forceinline__ s16x8_t pack8(const float* x) {
    u32x4_t w = {pack2<T>(x[0], x[1]), pack2<T>(x[2], x[3]), pack2<T>(x[4], x[5]), pack2<T>(x[6], x[7])};
    return __builtin_bit_cast(s16x8_t, w);
}

template <typename T, int D>
__global__ void __launch_bounds__(256, D <= 64 ? 3 : 1) attention_fwd16_kernel(AttnArgs g) {
    static_assert(D % 32 == 0 && D <= 128, "head dimension: a multiple of 32 up to 128");
    constexpr int KS = D / 16;              // k-steps of the first product
    constexpr int DT = D / 32;              // 32-row tiles of O^T
    constexpr int VP = m16_mc_pitch(D);     // LDS pitch of a V row in elements, the GEMM kernels' conflict-free one for this read pattern
    constexpr int VPIECES = AT_KEYS * D / 8 / 256 > 0 ? AT_KEYS * D / 8 / 256 : 1;      // 16-byte pieces of a V block per thread
    constexpr int RP = D + 8;               // LDS pitch of a K row in elements: 16 bytes past a multiple of 128, so that ds_read_b128 of 16 rows is conflict-free
    __shared__ __attribute__((aligned(16))) uint16_t vlds[2][AT_KEYS * VP];
    __shared__ __attribute__((aligned(16))) uint16_t klds[2][AT_KEYS * RP];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, c = lane & 31;
    int row_tile, z;
    attn_block(row_tile, z);
    const int q0 = row_tile * AT_QROWS + wave * 32;               // this wave's first query row
    const uint16_t* Q = (const uint16_t*)g.Q + (long long)z * g.q_bs;
    const uint16_t* K = (const uint16_t*)g.K + (long long)z * g.k_bs;
    const uint16_t* V = (const uint16_t*)g.V + (long long)z * g.v_bs;
    // exp(scale * s - max) = exp2(s * sc - max * sc) with sc = |scale| log2 e: one fused multiply-add per score; a
    // negative scale flips the sign of the scores first, so that the running maximum can be kept on the raw scores
    const float sc = fabsf(g.scale) * 1.44269504088896341f;
    const bool flip = g.scale < 0.f;

    // Q^T as a B operand: lane (h, c) holds d = 16*ks + 8h .. +7 of query row q0 + c (zero beyond sq)
    const char* q_end = (const char*)(Q + ((long long)(g.sq - 1) * g.q_rs + D));
    const char* q_base = (const char*)(Q + (long long)q0 * g.q_rs);
    const __amdgpu_buffer_rsrc_t q_rsrc = buffer_rsrc(q_base, q0 < g.sq ? (long long)(q_end - q_base) : 0);
    s16x8_t qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
        qf[ks] = __builtin_bit_cast(s16x8_t, __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, (int)(((long long)c * g.q_rs + 16 * ks + 8 * h) * 2), 0, 0));

    // K and V blocks [32 keys][D] go to LDS, 16 bytes per thread and piece, in whole rows (every cache line is
    // requested once per workgroup; fragment loads straight from global memory would touch 32 lines per instruction
    // and per wave, which the vector cache's tag pipeline cannot keep up with).  Rows past sk read zeros.
    const char* k_end = (const char*)(K + ((long long)(g.sk - 1) * g.k_rs + D));
    const char* v_end = (const char*)(V + ((long long)(g.sk - 1) * g.v_rs + D));
    auto load_blk = [&](u32x4_t (&r)[VPIECES], const uint16_t* M, long long rs, const char* end, int kb) {
        const char* mp = (const char*)(M + (long long)kb * rs);
        const __amdgpu_buffer_rsrc_t rsrc = buffer_rsrc(mp, kb < g.sk ? (long long)(end - mp) : 0);
#pragma unroll
        for (int i = 0; i < VPIECES; i++) {
            const int id = threadIdx.x + 256 * i, key = id / (D / 8), d8 = (id % (D / 8)) * 8;
            const bool live = AT_KEYS * D / 8 >= 256 || id < AT_KEYS * D / 8;
            r[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, live ? (int)(((long long)key * rs + d8) * 2) : (int)BUFFER_OOB, 0, 0);
        }
    };
    auto load_v = [&](u32x4_t (&vr)[VPIECES], int kb) { load_blk(vr, V, g.v_rs, v_end, kb); };
    auto load_k = [&](u32x4_t (&kr)[VPIECES], int kb) { load_blk(kr, K, g.k_rs, k_end, kb); };
    // K as an A operand of the first product: lane (h, c) reads d = 16*ks + 8h .. +7 of key row c
    auto store_k = [&](const u32x4_t (&kr)[VPIECES], uint16_t* stage) {
#pragma unroll
        for (int i = 0; i < VPIECES; i++) {
            const int id = threadIdx.x + 256 * i, key = id / (D / 8), d8 = (id % (D / 8)) * 8;
            if (AT_KEYS * D / 8 >= 256 || id < AT_KEYS * D / 8) *(u32x4_t*)(stage + key * RP + d8) = kr[i];
        }
    };
    const int k_fr0 = c * RP + 8 * h;
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
    float m_run = -INFINITY, l_run = 0.f;            // running maximum (of the raw, sign-adjusted scores) and this lane's share of the running sum

    const int nblocks = (g.sk + AT_KEYS - 1) / AT_KEYS;
    u32x4_t kr[VPIECES], vr[VPIECES];
    load_k(kr, 0);
    load_v(vr, 0);
    store_k(kr, klds[0]);
    store_v(vr, vlds[0]);
    load_k(kr, AT_KEYS);
    load_v(vr, AT_KEYS);
    __syncthreads();

    auto step = [&](int blk) {
        const int kb = blk * AT_KEYS;
        const uint16_t* stage = vlds[blk & 1];
        const uint16_t* kstage = klds[blk & 1];
        // scores of 32 keys x 32 queries
        f32x16_t st;
#pragma unroll
        for (int v = 0; v < 16; v++) st[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) st = mfma16_ops<T>::mma(*(const s16x8_t*)(kstage + k_fr0 + 16 * ks), qf[ks], st);
        // the next block goes to the other stage (everyone left it at the previous barrier); then request the one after
        store_k(kr, klds[(blk & 1) ^ 1]);
        store_v(vr, vlds[(blk & 1) ^ 1]);
        load_k(kr, kb + 2 * AT_KEYS);
        load_v(vr, kb + 2 * AT_KEYS);

        // this step's V^T fragments, requested before the softmax arithmetic that hides their latency
        s16x8_t vfr[2][DT];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) vfr[t][dt] = read_v(stage, dt, t);

        if (flip) {
#pragma unroll
            for (int v = 0; v < 16; v++) st[v] = -st[v];
        }
        const bool ragged = kb + AT_KEYS > g.sk;            // the last block of a ragged sk
        if (ragged) {
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (kb + 8 * (v / 4) + 4 * h + (v % 4) >= g.sk) st[v] = -INFINITY;
        }
        float mx = m_run;
#pragma unroll
        for (int v = 0; v < 16; v++) mx = fmaxf(st[v], mx);
        const float other = __shfl_xor(mx, 32, 64);         // the lane that holds this query's other 16 keys
        mx = fmaxf(other, mx);
        // a query row beyond sq (or a block of masked keys met first) keeps mx = -inf: exp2(-inf - -inf) must not produce NaN
        const float m_use = mx == -INFINITY ? 0.f : mx;
        const float msc = m_use * sc;
        const float alpha = __builtin_amdgcn_exp2f(m_run == -INFINITY ? -INFINITY : m_run * sc - msc);
        float psum = 0.f;
        float e[16];
#pragma unroll
        for (int v = 0; v < 16; v++) e[v] = __builtin_amdgcn_exp2f(fmaf(st[v], sc, -msc));
        if (ragged) {                                       // a masked score times a zero scale would be NaN, not 0
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (kb + 8 * (v / 4) + 4 * h + (v % 4) >= g.sk) e[v] = 0.f;
        }
#pragma unroll
        for (int v = 0; v < 16; v++) psum += e[v];
        l_run = l_run * alpha + psum;
        m_run = mx;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {   // once the running maxima have settled there is nothing to rescale
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int v = 0; v < 16; v++) ot[dt][v] *= alpha;
        }
        // O^T += V^T * P^T, 16 keys per MFMA
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const s16x8_t pb = pack8<T>(e + 8 * t);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) ot[dt] = mfma16_ops<T>::mma(vfr[t][dt], pb, ot[dt]);
        }
        __syncthreads();                                    // next stage is written, this one is free
    };
    for (int blk = 0; blk < nblocks; blk++) step(blk);

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
        if (g.L && h == 0) g.L[(long long)z * g.sq + q] = (m_run * sc + __builtin_amdgcn_logf(l_all)) * 0.693147180559945309f;   // natural log of the row sum of exp(scale * s)
    }
}

// ============================================================================
// Backward, two kernels.  With P = softmax(scale * Q K^T), O = P V and upstream dO:
//   Dq[q] = sum_d dO[q,d] O[q,d]
//   dV = P^T dO          dP = dO V^T          dS = P o (dP - Dq) * scale          dQ = dS K          dK = dS^T Q
// P is recomputed from the saved row-wise log-sum-exp: P = exp(scale * s - L[q]); nothing of size S x S is stored.
// Every product is arranged so that the fp32 accumulator of one MFMA, narrowed to 16 bits, is the B operand of the
// next without leaving the lane (see the forward kernel): the dQ kernel works on S^T tiles (lane = query), the
// dK/dV kernel on S tiles (lane = key).  Operands whose rows are d-contiguous in memory load straight into MFMA
// registers; the ones that must be read transposed (K^T for dQ; dO^T and Q^T for dV and dK) go through LDS and
// ds_read_tr16_b64.
// ============================================================================
// A [32 rows][D] block of a d-contiguous matrix, staged in LDS for transposed MFMA operand reads.
template <int D>
struct AttnBlock {
    static constexpr int VP = m16_mc_pitch(D);
    static constexpr int ELEMS = AT_KEYS * VP;
    static constexpr int PIECES = AT_KEYS * D / 8 / 256 > 0 ? AT_KEYS * D / 8 / 256 : 1;
    static __device__ __forceinline__ void load(u32x4_t (&r)[PIECES], const uint16_t* M, long long rs, int row0, int rows, const char* end) {
        const char* p = (const char*)(M + (long long)row0 * rs);
        const __amdgpu_buffer_rsrc_t rsrc = buffer_rsrc(p, row0 < rows ? (long long)(end - p) : 0);
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int id = threadIdx.x + 256 * i, row = id / (D / 8), d8 = (id % (D / 8)) * 8;
            const bool live = AT_KEYS * D / 8 >= 256 || id < AT_KEYS * D / 8;
            r[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, live ? (int)(((long long)row * rs + d8) * 2) : (int)BUFFER_OOB, 0, 0);
        }
    }
    static __device__ __forceinline__ void store(const u32x4_t (&r)[PIECES], uint16_t* stage) {
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int id = threadIdx.x + 256 * i, row = id / (D / 8), d8 = (id % (D / 8)) * 8;
            if (AT_KEYS * D / 8 >= 256 || id < AT_KEYS * D / 8) *(u32x4_t*)(stage + row * VP + d8) = r[i];
        }
    }
    // the same block kept a second way, for operands whose fragments are 8 consecutive d of one row (ds_read_b128):
    // the pitch is 16 bytes past a multiple of 128, which spreads 16 rows over all banks
    static constexpr int RP = D + 8;
    static constexpr int ROW_ELEMS = AT_KEYS * RP;
    static __device__ __forceinline__ void store_rows(const u32x4_t (&r)[PIECES], uint16_t* stage) {
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int id = threadIdx.x + 256 * i, row = id / (D / 8), d8 = (id % (D / 8)) * 8;
            if (AT_KEYS * D / 8 >= 256 || id < AT_KEYS * D / 8) *(u32x4_t*)(stage + row * RP + d8) = r[i];
        }
    }
    // fragment ks of block row c: d = 16*ks + 8h .. +7 (an A operand with row = lane % 32)
    static __device__ __forceinline__ s16x8_t frag(const uint16_t* stage, int c, int h, int ks) {
        return *(const s16x8_t*)(stage + c * RP + 16 * ks + 8 * h);
    }
    // lane's base offset for transposed reads: k slot e of MFMA t <-> block row 16t + 8*(e/4) + 4*(lane/32) + e%4
    static __device__ __forceinline__ int tr_base(int lane) {
        const int grp = lane >> 4, s16 = lane & 15;
        return (4 * (grp >> 1) + (s16 >> 2)) * VP + 16 * (grp & 1) + 4 * (s16 & 3);
    }
    static __device__ __forceinline__ s16x8_t read_tr(const uint16_t* stage, int base, int dt, int t) {
        s16x8_t f;
#pragma unroll
        for (int H = 0; H < 2; H++) {
            s16x4_t q4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(lds_u16*)(stage + base + (16 * t + 8 * H) * VP + 32 * dt));
            f[4 * H + 0] = q4[0]; f[4 * H + 1] = q4[1]; f[4 * H + 2] = q4[2]; f[4 * H + 3] = q4[3];
        }
        return f;
    }
};

// rows row0 + c of a d-contiguous matrix as MFMA operand fragments (A: row = lane % 32; B: column = lane % 32), zero past `rows`
template <int KS>
__device__ __forceinline__ void attn_load_rows(s16x8_t (&f)[KS], const uint16_t* M, long long rs, int row0, int rows, const char* end, int c, int h) {
    const char* p = (const char*)(M + (long long)row0 * rs);
    const __amdgpu_buffer_rsrc_t rsrc = buffer_rsrc(p, row0 < rows ? (long long)(end - p) : 0);
    const int voff = (int)(((long long)c * rs + 8 * h) * 2);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) f[ks] = __builtin_bit_cast(s16x8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 32 * ks, 0));
}

// dQ: a wave owns 32 queries and walks the keys.
template <typename T, int D>
__global__ void __launch_bounds__(256, D <= 64 ? 3 : 1) attention_bwd_dq16_kernel(AttnBwdArgs g) {
    constexpr int KS = D / 16, DT = D / 32;
    using Blk = AttnBlock<D>;
    __shared__ __attribute__((aligned(16))) uint16_t klds[2][Blk::ELEMS];           // K for transposed reads (K^T of the dQ product)
    __shared__ __attribute__((aligned(16))) uint16_t krows[2][Blk::ROW_ELEMS];       // K and V for row fragments (S^T and dP^T)
    __shared__ __attribute__((aligned(16))) uint16_t vrows[2][Blk::ROW_ELEMS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, c = lane & 31;
    int row_tile, z;
    attn_block(row_tile, z);
    const int q0 = row_tile * AT_QROWS + wave * 32;
    const uint16_t* Q = (const uint16_t*)g.Q + (long long)z * g.q_bs;
    const uint16_t* K = (const uint16_t*)g.K + (long long)z * g.k_bs;
    const uint16_t* V = (const uint16_t*)g.V + (long long)z * g.v_bs;
    const uint16_t* dO = (const uint16_t*)g.dO + (long long)z * g.do_bs;
    const char* q_end = (const char*)(Q + ((long long)(g.sq - 1) * g.q_rs + D));
    const char* k_end = (const char*)(K + ((long long)(g.sk - 1) * g.k_rs + D));
    const char* v_end = (const char*)(V + ((long long)(g.sk - 1) * g.v_rs + D));
    const char* do_end = (const char*)(dO + ((long long)(g.sq - 1) * g.do_rs + D));
    const float sc = g.scale * 1.44269504088896341f;

    s16x8_t qf[KS], dof[KS];                 // B operands: column = query q0 + c
    attn_load_rows<KS>(qf, Q, g.q_rs, q0, g.sq, q_end, c, h);
    attn_load_rows<KS>(dof, dO, g.do_rs, q0, g.sq, do_end, c, h);
    const int q = q0 + c;
    const float lq = q < g.sq ? g.L[(long long)z * g.sq + q] * 1.44269504088896341f : 0.f;
    // Dq[q] = sum_d dO[q, d] * O[q, d]: the lane holds 8 of every 16 d of its query, the lane 32 away the rest
    float dq_dot = 0.f;
    {
        const uint16_t* O = (const uint16_t*)g.O + (long long)z * g.o_bs;
        s16x8_t of[KS];
        attn_load_rows<KS>(of, O, g.o_rs, q0, g.sq, (const char*)(O + ((long long)(g.sq - 1) * g.o_rs + D)), c, h);
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                T a, b;
                a.bits = (uint16_t)dof[ks][e]; b.bits = (uint16_t)of[ks][e];
                dq_dot += widen(a) * widen(b);
            }
        dq_dot += __shfl_xor(dq_dot, 32, 64);
        if (q < g.sq && h == 0) g.Dq[(long long)z * g.sq + q] = dq_dot;
    }
    const float dq_dot_scaled = dq_dot * g.scale;

    f32x16_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[dt][v] = 0.f;

    const int tr0 = Blk::tr_base(lane);
    const int nblocks = (g.sk + AT_KEYS - 1) / AT_KEYS;
    // K and V blocks are staged by the whole workgroup with row-contiguous loads (fragment loads straight from
    // global memory touch 32 cache lines per instruction and wave, more than the vector cache's tag pipeline sustains)
    u32x4_t kr[Blk::PIECES], vr[Blk::PIECES];
    Blk::load(kr, K, g.k_rs, 0, g.sk, k_end);
    Blk::load(vr, V, g.v_rs, 0, g.sk, v_end);
    Blk::store(kr, klds[0]); Blk::store_rows(kr, krows[0]); Blk::store_rows(vr, vrows[0]);
    Blk::load(kr, K, g.k_rs, AT_KEYS, g.sk, k_end);
    Blk::load(vr, V, g.v_rs, AT_KEYS, g.sk, v_end);
    __syncthreads();

    auto step = [&](int blk) {
        const int kb = blk * AT_KEYS;
        const uint16_t* stage = klds[blk & 1];
        f32x16_t st, dp;
#pragma unroll
        for (int v = 0; v < 16; v++) { st[v] = 0.f; dp[v] = 0.f; }
        const int cur = blk & 1;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) st = mfma16_ops<T>::mma(Blk::frag(krows[cur], c, h, ks), qf[ks], st);        // S^T: keys x queries
#pragma unroll
        for (int ks = 0; ks < KS; ks++) dp = mfma16_ops<T>::mma(Blk::frag(vrows[cur], c, h, ks), dof[ks], dp);       // dP^T
        // this step's K^T fragments, requested before the arithmetic that hides their latency
        s16x8_t ktf[2][DT];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) ktf[t][dt] = Blk::read_tr(stage, tr0, dt, t);
        Blk::store(kr, klds[cur ^ 1]); Blk::store_rows(kr, krows[cur ^ 1]); Blk::store_rows(vr, vrows[cur ^ 1]);
        Blk::load(kr, K, g.k_rs, kb + 2 * AT_KEYS, g.sk, k_end);
        Blk::load(vr, V, g.v_rs, kb + 2 * AT_KEYS, g.sk, v_end);
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float p = __builtin_amdgcn_exp2f(fmaf(st[v], sc, -lq));
            ds[v] = p * fmaf(dp[v], g.scale, -dq_dot_scaled);                  // P o (dP - Dq) * scale
        }
        if (kb + AT_KEYS > g.sk) {                          // the last block of a ragged sk: keys past the end count for nothing
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (kb + 8 * (v / 4) + 4 * h + (v % 4) >= g.sk) ds[v] = 0.f;
        }
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const s16x8_t dsb = pack8<T>(ds + 8 * t);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) acc[dt] = mfma16_ops<T>::mma(ktf[t][dt], dsb, acc[dt]);      // dQ^T += K^T dS^T
        }
        __syncthreads();
    };
    for (int blk = 0; blk < nblocks; blk++) step(blk);
    if (q < g.sq) {
        T* row = (T*)g.dQ + ((long long)z * g.sq + q) * D;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                T out[4];
#pragma unroll
                for (int e = 0; e < 4; e++) out[e] = narrow<T>(acc[dt][4 * v4 + e]);
                uint2 w;
                memcpy(&w, out, 8);
                *(uint2*)(row + 32 * dt + 8 * v4 + 4 * h) = w;
            }
    }
}

// dK and dV: a wave owns 32 keys and walks the queries.
template <typename T, int D>
__global__ void __launch_bounds__(256, D <= 64 ? 2 : 1) attention_bwd_dkv16_kernel(AttnBwdArgs g) {
    constexpr int KS = D / 16, DT = D / 32;
    using Blk = AttnBlock<D>;
    // dynamic LDS (above 64 KB for d = 128): Q and dO blocks, each kept for transposed reads (Q^T, dO^T of the dK and
    // dV products) and for row fragments (S and dP), two stages; then L and Dq of the block's queries
    extern __shared__ __attribute__((aligned(16))) uint16_t dkv_lds[];
    uint16_t (*qlds)[Blk::ELEMS] = (uint16_t (*)[Blk::ELEMS])dkv_lds;
    uint16_t (*dolds)[Blk::ELEMS] = (uint16_t (*)[Blk::ELEMS])(dkv_lds + 2 * Blk::ELEMS);
    uint16_t (*qrows)[Blk::ROW_ELEMS] = (uint16_t (*)[Blk::ROW_ELEMS])(dkv_lds + 4 * Blk::ELEMS);
    uint16_t (*dorows)[Blk::ROW_ELEMS] = (uint16_t (*)[Blk::ROW_ELEMS])(dkv_lds + 4 * Blk::ELEMS + 2 * Blk::ROW_ELEMS);
    float (*rowlds)[2][AT_KEYS] = (float (*)[2][AT_KEYS])(dkv_lds + 4 * Blk::ELEMS + 4 * Blk::ROW_ELEMS);        // [stage][L, Dq][query of the block]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, c = lane & 31;
    int row_tile, z;
    attn_block(row_tile, z);
    const int k0 = row_tile * AT_QROWS + wave * 32;               // this wave's first key
    const uint16_t* Q = (const uint16_t*)g.Q + (long long)z * g.q_bs;
    const uint16_t* K = (const uint16_t*)g.K + (long long)z * g.k_bs;
    const uint16_t* V = (const uint16_t*)g.V + (long long)z * g.v_bs;
    const uint16_t* dO = (const uint16_t*)g.dO + (long long)z * g.do_bs;
    const char* q_end = (const char*)(Q + ((long long)(g.sq - 1) * g.q_rs + D));
    const char* k_end = (const char*)(K + ((long long)(g.sk - 1) * g.k_rs + D));
    const char* v_end = (const char*)(V + ((long long)(g.sk - 1) * g.v_rs + D));
    const char* do_end = (const char*)(dO + ((long long)(g.sq - 1) * g.do_rs + D));
    const float sc = g.scale * 1.44269504088896341f;
    const float* Lz = g.L + (long long)z * g.sq;
    const float* Dz = g.Dq + (long long)z * g.sq;

    s16x8_t kf[KS], vf[KS];                  // B operands: column = key k0 + c
    attn_load_rows<KS>(kf, K, g.k_rs, k0, g.sk, k_end, c, h);
    attn_load_rows<KS>(vf, V, g.v_rs, k0, g.sk, v_end, c, h);

    f32x16_t dkt[DT], dvt[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) { dkt[dt][v] = 0.f; dvt[dt][v] = 0.f; }

    const int tr0 = Blk::tr_base(lane);
    const int nblocks = (g.sq + AT_KEYS - 1) / AT_KEYS;
    u32x4_t qr[Blk::PIECES], dor[Blk::PIECES];
    // L and Dq of the block's 32 queries: every lane requests query qb + lane % 32 (buffer loads, zero past sq, so
    // that no branch surrounds them and the wait for them can be counted); wave 0 puts them in LDS: its lower half
    // the L (in log2 units, +inf past sq, which makes those rows' probabilities exactly 0), its upper half Dq * scale
    const __amdgpu_buffer_rsrc_t l_rsrc = buffer_rsrc(Lz, (long long)g.sq * 4), d_rsrc = buffer_rsrc(Dz, (long long)g.sq * 4);
    float row_l = 0.f, row_d = 0.f;
    auto load_rowv = [&](int qb) {
        row_l = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(l_rsrc, (qb + c) * 4, 0, 0));
        row_d = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(d_rsrc, (qb + c) * 4, 0, 0));
    };
    auto store_rowv = [&](int stage, int qb) {
        if (wave == 0) rowlds[stage][h][c] = h ? row_d * g.scale : (qb + c < g.sq ? row_l * 1.44269504088896341f : INFINITY);
    };
    Blk::load(qr, Q, g.q_rs, 0, g.sq, q_end);
    Blk::load(dor, dO, g.do_rs, 0, g.sq, do_end);
    load_rowv(0);
    Blk::store(qr, qlds[0]); Blk::store_rows(qr, qrows[0]);
    Blk::store(dor, dolds[0]); Blk::store_rows(dor, dorows[0]);
    store_rowv(0, 0);
    Blk::load(qr, Q, g.q_rs, AT_KEYS, g.sq, q_end);
    Blk::load(dor, dO, g.do_rs, AT_KEYS, g.sq, do_end);
    load_rowv(AT_KEYS);
    __syncthreads();

    auto step = [&](int blk) {
        const int qb = blk * AT_KEYS;
        const int cur = blk & 1;
        f32x16_t st, dp;
#pragma unroll
        for (int v = 0; v < 16; v++) { st[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) st = mfma16_ops<T>::mma(Blk::frag(qrows[cur], c, h, ks), kf[ks], st);        // S: queries x keys
#pragma unroll
        for (int ks = 0; ks < KS; ks++) dp = mfma16_ops<T>::mma(Blk::frag(dorows[cur], c, h, ks), vf[ks], dp);       // dP
        Blk::store(qr, qlds[cur ^ 1]); Blk::store_rows(qr, qrows[cur ^ 1]);
        Blk::store(dor, dolds[cur ^ 1]); Blk::store_rows(dor, dorows[cur ^ 1]);
        store_rowv(cur ^ 1, qb + AT_KEYS);
        Blk::load(qr, Q, g.q_rs, qb + 2 * AT_KEYS, g.sq, q_end);
        Blk::load(dor, dO, g.do_rs, qb + 2 * AT_KEYS, g.sq, do_end);
        load_rowv(qb + 2 * AT_KEYS);
        float p[16], ds[16];
#pragma unroll
        for (int v4 = 0; v4 < 4; v4++) {
            // registers 4*v4 .. 4*v4+3 are queries qb + 8*v4 + 4h + (0..3): their L and scaled Dq are 16 contiguous bytes each
            const f32x4_t l4 = *(const f32x4_t*)&rowlds[cur][0][8 * v4 + 4 * h];
            const f32x4_t d4 = *(const f32x4_t*)&rowlds[cur][1][8 * v4 + 4 * h];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int v = 4 * v4 + e;
                p[v] = __builtin_amdgcn_exp2f(fmaf(st[v], sc, -l4[e]));          // 0 for a query past sq: its L is +inf
                ds[v] = p[v] * fmaf(dp[v], g.scale, -d4[e]);                      // P o (dP - Dq) * scale
            }
        }
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const s16x8_t pb = pack8<T>(p + 8 * t), dsb = pack8<T>(ds + 8 * t);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                dvt[dt] = mfma16_ops<T>::mma(Blk::read_tr(dolds[cur], tr0, dt, t), pb, dvt[dt]);      // dV^T += dO^T P
                dkt[dt] = mfma16_ops<T>::mma(Blk::read_tr(qlds[cur], tr0, dt, t), dsb, dkt[dt]);      // dK^T += Q^T dS
            }
        }
        __syncthreads();
    };
    for (int blk = 0; blk < nblocks; blk++) step(blk);
    const int key = k0 + c;
    if (key < g.sk) {
        T* krow = (T*)g.dK + ((long long)z * g.sk + key) * D;
        T* vrow = (T*)g.dV + ((long long)z * g.sk + key) * D;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v4 = 0; v4 < 4; v4++) {
                T ok[4], ov[4];
#pragma unroll
                for (int e = 0; e < 4; e++) { ok[e] = narrow<T>(dkt[dt][4 * v4 + e]); ov[e] = narrow<T>(dvt[dt][4 * v4 + e]); }
                uint2 wk, wv;
                memcpy(&wk, ok, 8); memcpy(&wv, ov, 8);
                *(uint2*)(krow + 32 * dt + 8 * v4 + 4 * h) = wk;
                *(uint2*)(vrow + 32 * dt + 8 * v4 + 4 * h) = wv;
            }
    }
}

template <int D>
constexpr size_t attn_dkv_lds_bytes() { return (size_t)(4 * AttnBlock<D>::ELEMS + 4 * AttnBlock<D>::ROW_ELEMS) * 2 + 2 * 2 * AT_KEYS * sizeof(float); }

template <typename T, int D>
static int launch_attention_bwd_d(const AttnBwdArgs& g) {
    dim3 gq((g.sq + AT_QROWS - 1) / AT_QROWS, g.batch), gk((g.sk + AT_QROWS - 1) / AT_QROWS, g.batch);
    constexpr size_t smem = attn_dkv_lds_bytes<D>();
    auto dkv = attention_bwd_dkv16_kernel<T, D>;
    if (smem > 64 * 1024 && !check_hip(hipFuncSetAttribute((const void*)dkv, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem), "hipFuncSetAttribute")) return -1;
    hipLaunchKernelGGL((attention_bwd_dq16_kernel<T, D>), gq, dim3(256), 0, current_stream(), g);
    hipLaunchKernelGGL(dkv, gk, dim3(256), smem, current_stream(), g);
    return check_launch("attention backward kernels") ? 0 : -1;
}

template <typename T>
static int launch_attention_bwd_t(const AttnBwdArgs& g, int d) {
    switch (d) {
        case 32: return launch_attention_bwd_d<T, 32>(g);
        case 64: return launch_attention_bwd_d<T, 64>(g);
        case 128: return launch_attention_bwd_d<T, 128>(g);
        default: set_error("rp_hip_attention_backward: head dimension %d (supported: 32, 64, 128)", d); return -1;
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
    if (dtype != RP_DTYPE_BFLOAT16 && dtype != RP_DTYPE_FLOAT16 && dtype != RP_DTYPE_FLOAT32) { set_error("rp_hip_attention_forward: bfloat16, float16 or float32 (dtype %d)", dtype); return -1; }
    const bool f32 = dtype == RP_DTYPE_FLOAT32;
    const long long esz = f32 ? 4 : 2, vec = 16 / esz;
    if (d != 32 && d != 64 && d != 128) { set_error("rp_hip_attention_forward: head dimension %d (supported: 32, 64, 128)", d); return -1; }
    const long long strides[] = {q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs};
    for (long long s : strides)
        if (s < 0 || s % vec) { set_error("rp_hip_attention_forward: strides must be non-negative multiples of 16 bytes"); return -1; }
    if (q_rs >= (1ll << 22) || k_rs >= (1ll << 22) || v_rs >= (1ll << 22)) { set_error("rp_hip_attention_forward: row stride too large"); return -1; }
    if (((uintptr_t)O | (uintptr_t)Q | (uintptr_t)K | (uintptr_t)V) & 15) { set_error("rp_hip_attention_forward: operands must be 16-byte aligned"); return -1; }
    constexpr int MAX_BATCH = 65535;
    for (int b0 = 0; b0 < batch; b0 += MAX_BATCH) {
        const int nb = batch - b0 < MAX_BATCH ? batch - b0 : MAX_BATCH;
        AttnArgs g{(char*)O + b0 * o_bs * esz, (const char*)Q + b0 * q_bs * esz, (const char*)K + b0 * k_bs * esz, (const char*)V + b0 * v_bs * esz,
                   lse ? lse + (long long)b0 * sq : nullptr, nb, sq, sk, q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs, (float)scale};
        int rc = f32 ? launch_attention_f32(g, d) : dtype == RP_DTYPE_BFLOAT16 ? launch_attention_t<bf16_t>(g, d) : launch_attention_t<f16_t>(g, d);
        if (rc != 0) return -1;
    }
    return 0;
}

extern "C" int rp_hip_attention_backward(void* dQ, void* dK, void* dV, const void* Q, const void* K, const void* V,
                                         const void* O, const void* dO, const float* lse,
                                         int batch, int sq, int sk, int d,
                                         long long q_bs, long long q_rs, long long k_bs, long long k_rs,
                                         long long v_bs, long long v_rs, long long o_bs, long long o_rs,
                                         long long do_bs, long long do_rs, double scale, int dtype) {
    if (!dQ || !dK || !dV || !Q || !K || !V || !O || !dO || !lse || batch <= 0 || sq <= 0 || sk <= 0 || d <= 0) {
        set_error("rp_hip_attention_backward: null operand or non-positive extent (batch=%d sq=%d sk=%d d=%d)", batch, sq, sk, d);
        return -1;
    }
    if (dtype != RP_DTYPE_BFLOAT16 && dtype != RP_DTYPE_FLOAT16 && dtype != RP_DTYPE_FLOAT32) { set_error("rp_hip_attention_backward: bfloat16, float16 or float32 (dtype %d)", dtype); return -1; }
    const bool f32 = dtype == RP_DTYPE_FLOAT32;
    const long long esz = f32 ? 4 : 2, vec = 16 / esz;
    if (d != 32 && d != 64 && d != 128) { set_error("rp_hip_attention_backward: head dimension %d (supported: 32, 64, 128)", d); return -1; }
    const long long strides[] = {q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs, do_bs, do_rs};
    for (long long s : strides)
        if (s < 0 || s % vec) { set_error("rp_hip_attention_backward: strides must be non-negative multiples of 16 bytes"); return -1; }
    if (q_rs >= (1ll << 22) || k_rs >= (1ll << 22) || v_rs >= (1ll << 22) || o_rs >= (1ll << 22) || do_rs >= (1ll << 22)) { set_error("rp_hip_attention_backward: row stride too large"); return -1; }
    if (((uintptr_t)dQ | (uintptr_t)dK | (uintptr_t)dV | (uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)O | (uintptr_t)dO) & 15) {
        set_error("rp_hip_attention_backward: operands must be 16-byte aligned");
        return -1;
    }
    void* dots = nullptr;
    if (rp_hip_malloc(&dots, (size_t)batch * sq * sizeof(float)) != 0) return -1;
    // the batch rides on a grid axis that holds at most 65535 blocks: longer batches go in chunks
    constexpr int MAX_BATCH = 65535;
    int rc = 0;
    for (int b0 = 0; rc == 0 && b0 < batch; b0 += MAX_BATCH) {
        const int nb = batch - b0 < MAX_BATCH ? batch - b0 : MAX_BATCH;
        const long long q_off = (long long)b0 * sq * d * esz, k_off = (long long)b0 * sk * d * esz;        // the gradients are dense
        AttnBwdArgs g{(char*)dQ + q_off, (char*)dK + k_off, (char*)dV + k_off, (const char*)Q + b0 * q_bs * esz, (const char*)K + b0 * k_bs * esz,
                      (const char*)V + b0 * v_bs * esz, (const char*)O + b0 * o_bs * esz, (const char*)dO + b0 * do_bs * esz, lse + (long long)b0 * sq,
                      (float*)dots + (long long)b0 * sq, nb, sq, sk, q_bs, q_rs, k_bs, k_rs, v_bs, v_rs, o_bs, o_rs, do_bs, do_rs, (float)scale};
        rc = f32 ? launch_attention_bwd_f32(g, d) : dtype == RP_DTYPE_BFLOAT16 ? launch_attention_bwd_t<bf16_t>(g, d) : launch_attention_bwd_t<f16_t>(g, d);
    }
    rp_hip_free(dots);        // back to the pool while the kernels are still queued: safe for later work on this stream; held with the graph while one is being recorded
    return rc;
}

