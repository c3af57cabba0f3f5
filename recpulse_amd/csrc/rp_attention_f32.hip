// Fused attention for float32 (head dimension 32, 64 or 128): forward, and the dQ and dK/dV kernels of the backward.
//
// Same decomposition as the 16-bit kernels (a workgroup owns 128 queries or keys, a wave 32 of them; S^T, P^T, O^T are
// kept transposed so that a lane owns one query of the forward and of the dQ kernel, one key of the dK/dV kernel), on
// v_mfma_f32_32x32x2_f32.  That instruction multiplies a 32 x 2 by a 2 x 32 panel: a lane holds ONE scalar of each
// operand (row or column lane % 32, k slot lane / 32), so
//   * for the products over d (S^T = K Q^T and the like) MFMA j pairs d = j (lanes 0..31) with d = j + D/2 (lanes
//     32..63): a lane's operand values are D/2 consecutive floats of its row, read with 16-byte loads;
//   * for the products over keys or queries (O^T += V^T P^T and the like) MFMA v uses accumulator register v of the
//     preceding product as its B operand as it stands: its two k slots are the rows 8*(v/4) + v%4 and
//     8*(v/4) + 4 + v%4 that register v holds in the two half-waves.  Nothing is converted or moved; the matching A
//     operand is one float per lane from LDS, read along d (consecutive lanes, consecutive banks).
// Probabilities and score gradients stay float32 throughout.  All three kernels are bound by the float32 MFMA rate
// (a 32 x 32 score tile costs 64, 96 or 128 MFMAs of 64 cycles), which is why the blocks of K, V, Q and dO simply go
// through LDS with a row pitch of D + 8 floats: conflict-free for the one-float reads, two-way for the 16-byte reads.
#include "rp_gemm_mfma16_kernel.h"
#include "rp_attention.h"

namespace rp {

typedef __attribute__((ext_vector_type(4))) float f32x4v_t;

__device__ __forceinline__ f32x16_t mma32(float a, float b, f32x16_t c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }

// A [32 rows][D] block of a d-contiguous float matrix in LDS.
template <int D>
struct Blk32 {
    static constexpr int RP = D + 8;                                 // floats
    static constexpr int ELEMS = AT_KEYS * RP;
    static constexpr int PIECES = AT_KEYS * D / 4 / 256;             // 16-byte pieces per thread
    static_assert(PIECES >= 1, "a block is at least one piece per thread");
    static __device__ __forceinline__ void load(u32x4_t (&r)[PIECES], const float* M, long long rs, int row0, int rows, const char* end) {
        const char* p = (const char*)(M + (long long)row0 * rs);
        const __amdgpu_buffer_rsrc_t rsrc = buffer_rsrc(p, row0 < rows ? (long long)(end - p) : 0);      // rows past the end read zeros
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int id = threadIdx.x + 256 * i, row = id / (D / 4), d4 = (id % (D / 4)) * 4;
            r[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(((long long)row * rs + d4) * 4), 0, 0);
        }
    }
    static __device__ __forceinline__ void store(const u32x4_t (&r)[PIECES], float* stage) {
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const int id = threadIdx.x + 256 * i, row = id / (D / 4), d4 = (id % (D / 4)) * 4;
            *(u32x4_t*)(stage + row * RP + d4) = r[i];
        }
    }
};

// D/2 consecutive floats of row row0 + c from d = (D/2) * h: the lane's operand values for the products over d
template <int KJ>
__device__ __forceinline__ void load_half_row(float (&f)[KJ], const float* M, long long rs, int row0, int rows, const char* end, int c, int h) {
    const char* p = (const char*)(M + (long long)row0 * rs);
    const __amdgpu_buffer_rsrc_t rsrc = buffer_rsrc(p, row0 < rows ? (long long)(end - p) : 0);
    const int voff = (int)(((long long)c * rs + KJ * h) * 4);
#pragma unroll
    for (int i = 0; i < KJ / 4; i++) {
        const f32x4v_t v = __builtin_bit_cast(f32x4v_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, 16 * i, 0));
        f[4 * i] = v[0]; f[4 * i + 1] = v[1]; f[4 * i + 2] = v[2]; f[4 * i + 3] = v[3];
    }
}

// acc += (block rows as A, over d) x (the lane's held half row as B): S^T, dP^T, S, dP
template <int D>
__device__ __forceinline__ f32x16_t product_over_d(const float* stage, const float (&held)[D / 2], int c, int h, f32x16_t acc) {
    constexpr int KJ = D / 2;
    const float* row = stage + c * Blk32<D>::RP + KJ * h;
#pragma unroll
    for (int i = 0; i < KJ / 4; i++) {
        const f32x4v_t a = *(const f32x4v_t*)(row + 4 * i);
#pragma unroll
        for (int e = 0; e < 4; e++) acc = mma32(a[e], held[4 * i + e], acc);
    }
    return acc;
}

// acc[dt] += (block^T as A, over the block's rows) x (sixteen accumulator registers as B): O^T, dQ^T, dV^T, dK^T
template <int D>
__device__ __forceinline__ void product_over_rows(f32x16_t (&acc)[D / 32], const float* stage, const float (&b)[16], int c, int h) {
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const float* src = stage + (8 * (v / 4) + 4 * h + (v % 4)) * Blk32<D>::RP + c;
#pragma unroll
        for (int dt = 0; dt < D / 32; dt++) acc[dt] = mma32(src[32 * dt], b[v], acc[dt]);
    }
}

template <int D>
__device__ __forceinline__ void write_rows_t(float* row, const f32x16_t (&acc)[D / 32], int h, float mul) {
    // the lane's column of the transposed accumulators is a row of the output: registers 4*v4 .. +3 are d = 32*dt + 8*v4 + 4h + (0..3)
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
        for (int v4 = 0; v4 < 4; v4++) {
            f32x4v_t o = {acc[dt][4 * v4] * mul, acc[dt][4 * v4 + 1] * mul, acc[dt][4 * v4 + 2] * mul, acc[dt][4 * v4 + 3] * mul};
            *(f32x4v_t*)(row + 32 * dt + 8 * v4 + 4 * h) = o;
        }
}

template <int D>
__global__ void __launch_bounds__(256, D <= 64 ? 2 : 1) attention_fwd32_kernel(AttnArgs g) {
    constexpr int KJ = D / 2, DT = D / 32;
    using Blk = Blk32<D>;
    __shared__ __attribute__((aligned(16))) float klds[2][Blk::ELEMS];
    __shared__ __attribute__((aligned(16))) float vlds[2][Blk::ELEMS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, c = lane & 31;
    int row_tile, z;
    attn_block(row_tile, z);
    const int q0 = row_tile * AT_QROWS + wave * 32;
    const float* Q = (const float*)g.Q + (long long)z * g.q_bs;
    const float* K = (const float*)g.K + (long long)z * g.k_bs;
    const float* V = (const float*)g.V + (long long)z * g.v_bs;
    const char* q_end = (const char*)(Q + ((long long)(g.sq - 1) * g.q_rs + D));
    const char* k_end = (const char*)(K + ((long long)(g.sk - 1) * g.k_rs + D));
    const char* v_end = (const char*)(V + ((long long)(g.sk - 1) * g.v_rs + D));
    // exp(scale * s - max) = exp2(s * sc - max * sc), sc = |scale| log2 e; a negative scale flips the scores' sign first
    const float sc = fabsf(g.scale) * 1.44269504088896341f;
    const bool flip = g.scale < 0.f;

    float qf[KJ];                                    // Q^T as a B operand: query q0 + c, d = j + KJ*h
    load_half_row<KJ>(qf, Q, g.q_rs, q0, g.sq, q_end, c, h);

    f32x16_t ot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) ot[dt][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const int nblocks = (g.sk + AT_KEYS - 1) / AT_KEYS;
    u32x4_t kr[Blk::PIECES], vr[Blk::PIECES];
    Blk::load(kr, K, g.k_rs, 0, g.sk, k_end);
    Blk::load(vr, V, g.v_rs, 0, g.sk, v_end);
    Blk::store(kr, klds[0]); Blk::store(vr, vlds[0]);
    Blk::load(kr, K, g.k_rs, AT_KEYS, g.sk, k_end);
    Blk::load(vr, V, g.v_rs, AT_KEYS, g.sk, v_end);
    __syncthreads();

    for (int blk = 0; blk < nblocks; blk++) {
        const int kb = blk * AT_KEYS, cur = blk & 1;
        f32x16_t st;
#pragma unroll
        for (int v = 0; v < 16; v++) st[v] = 0.f;
        st = product_over_d<D>(klds[cur], qf, c, h, st);                    // S^T: 32 keys x 32 queries
        Blk::store(kr, klds[cur ^ 1]); Blk::store(vr, vlds[cur ^ 1]);       // everyone left that stage at the previous barrier
        Blk::load(kr, K, g.k_rs, kb + 2 * AT_KEYS, g.sk, k_end);
        Blk::load(vr, V, g.v_rs, kb + 2 * AT_KEYS, g.sk, v_end);
        if (flip) {
#pragma unroll
            for (int v = 0; v < 16; v++) st[v] = -st[v];
        }
        const bool ragged = kb + AT_KEYS > g.sk;
        if (ragged) {
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (kb + 8 * (v / 4) + 4 * h + (v % 4) >= g.sk) st[v] = -INFINITY;
        }
        float mx = m_run;
#pragma unroll
        for (int v = 0; v < 16; v++) mx = fmaxf(st[v], mx);
        mx = fmaxf(__shfl_xor(mx, 32, 64), mx);             // the lane that holds this query's other 16 keys
        const float m_use = mx == -INFINITY ? 0.f : mx;     // a query past sq, or only masked keys so far: avoid exp2(-inf + inf)
        const float msc = m_use * sc;
        const float alpha = __builtin_amdgcn_exp2f(m_run == -INFINITY ? -INFINITY : m_run * sc - msc);
        float e[16];
#pragma unroll
        for (int v = 0; v < 16; v++) e[v] = __builtin_amdgcn_exp2f(fmaf(st[v], sc, -msc));
        if (ragged) {
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (kb + 8 * (v / 4) + 4 * h + (v % 4) >= g.sk) e[v] = 0.f;
        }
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) psum += e[v];
        l_run = l_run * alpha + psum;
        m_run = mx;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int v = 0; v < 16; v++) ot[dt][v] *= alpha;
        }
        product_over_rows<D>(ot, vlds[cur], e, c, h);       // O^T += V^T P^T
        __syncthreads();
    }

    const float l_all = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
    const int q = q0 + c;
    if (q < g.sq) {
        write_rows_t<D>((float*)g.O + (long long)z * g.o_bs + (long long)q * g.o_rs, ot, h, inv);
        if (g.L && h == 0) g.L[(long long)z * g.sq + q] = (m_run * sc + __builtin_amdgcn_logf(l_all)) * 0.693147180559945309f;
    }
}

// dQ: a wave owns 32 queries and walks the keys.
template <int D>
__global__ void __launch_bounds__(256, D <= 64 ? 2 : 1) attention_bwd_dq32_kernel(AttnBwdArgs g) {
    constexpr int KJ = D / 2, DT = D / 32;
    using Blk = Blk32<D>;
    __shared__ __attribute__((aligned(16))) float klds[2][Blk::ELEMS];
    __shared__ __attribute__((aligned(16))) float vlds[2][Blk::ELEMS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, c = lane & 31;
    int row_tile, z;
    attn_block(row_tile, z);
    const int q0 = row_tile * AT_QROWS + wave * 32;
    const float* Q = (const float*)g.Q + (long long)z * g.q_bs;
    const float* K = (const float*)g.K + (long long)z * g.k_bs;
    const float* V = (const float*)g.V + (long long)z * g.v_bs;
    const float* O = (const float*)g.O + (long long)z * g.o_bs;
    const float* dO = (const float*)g.dO + (long long)z * g.do_bs;
    const char* q_end = (const char*)(Q + ((long long)(g.sq - 1) * g.q_rs + D));
    const char* k_end = (const char*)(K + ((long long)(g.sk - 1) * g.k_rs + D));
    const char* v_end = (const char*)(V + ((long long)(g.sk - 1) * g.v_rs + D));
    const char* o_end = (const char*)(O + ((long long)(g.sq - 1) * g.o_rs + D));
    const char* do_end = (const char*)(dO + ((long long)(g.sq - 1) * g.do_rs + D));
    const float sc = g.scale * 1.44269504088896341f;

    float qf[KJ], dof[KJ];                           // B operands: query q0 + c, d = j + KJ*h
    load_half_row<KJ>(qf, Q, g.q_rs, q0, g.sq, q_end, c, h);
    load_half_row<KJ>(dof, dO, g.do_rs, q0, g.sq, do_end, c, h);
    const int q = q0 + c;
    const float lq = q < g.sq ? g.L[(long long)z * g.sq + q] * 1.44269504088896341f : 0.f;
    // Dq[q] = sum_d dO[q, d] * O[q, d]: the lane holds half of its query's d, the lane 32 away the rest
    float dq_dot = 0.f;
    {
        float of[KJ];
        load_half_row<KJ>(of, O, g.o_rs, q0, g.sq, o_end, c, h);
#pragma unroll
        for (int j = 0; j < KJ; j++) dq_dot += dof[j] * of[j];
        dq_dot += __shfl_xor(dq_dot, 32, 64);
        if (q < g.sq && h == 0) g.Dq[(long long)z * g.sq + q] = dq_dot;
    }
    const float dq_dot_scaled = dq_dot * g.scale;

    f32x16_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[dt][v] = 0.f;

    const int nblocks = (g.sk + AT_KEYS - 1) / AT_KEYS;
    u32x4_t kr[Blk::PIECES], vr[Blk::PIECES];
    Blk::load(kr, K, g.k_rs, 0, g.sk, k_end);
    Blk::load(vr, V, g.v_rs, 0, g.sk, v_end);
    Blk::store(kr, klds[0]); Blk::store(vr, vlds[0]);
    Blk::load(kr, K, g.k_rs, AT_KEYS, g.sk, k_end);
    Blk::load(vr, V, g.v_rs, AT_KEYS, g.sk, v_end);
    __syncthreads();

    for (int blk = 0; blk < nblocks; blk++) {
        const int kb = blk * AT_KEYS, cur = blk & 1;
        f32x16_t st, dp;
#pragma unroll
        for (int v = 0; v < 16; v++) { st[v] = 0.f; dp[v] = 0.f; }
        st = product_over_d<D>(klds[cur], qf, c, h, st);                    // S^T
        dp = product_over_d<D>(vlds[cur], dof, c, h, dp);                   // dP^T
        Blk::store(kr, klds[cur ^ 1]); Blk::store(vr, vlds[cur ^ 1]);
        Blk::load(kr, K, g.k_rs, kb + 2 * AT_KEYS, g.sk, k_end);
        Blk::load(vr, V, g.v_rs, kb + 2 * AT_KEYS, g.sk, v_end);
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const float p = __builtin_amdgcn_exp2f(fmaf(st[v], sc, -lq));
            ds[v] = p * fmaf(dp[v], g.scale, -dq_dot_scaled);               // P o (dP - Dq) * scale
        }
        if (kb + AT_KEYS > g.sk) {
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (kb + 8 * (v / 4) + 4 * h + (v % 4) >= g.sk) ds[v] = 0.f;
        }
        product_over_rows<D>(acc, klds[cur], ds, c, h);                     // dQ^T += K^T dS^T
        __syncthreads();
    }
    if (q < g.sq) write_rows_t<D>((float*)g.dQ + ((long long)z * g.sq + q) * D, acc, h, 1.f);
}

// dK and dV: a wave owns 32 keys and walks the queries.
template <int D>
__global__ void __launch_bounds__(256, D <= 32 ? 2 : 1) attention_bwd_dkv32_kernel(AttnBwdArgs g) {
    constexpr int KJ = D / 2, DT = D / 32;
    using Blk = Blk32<D>;
    __shared__ __attribute__((aligned(16))) float qlds[2][Blk::ELEMS];
    __shared__ __attribute__((aligned(16))) float dolds[2][Blk::ELEMS];
    __shared__ __attribute__((aligned(16))) float rowlds[2][2][AT_KEYS];        // [stage][L, Dq * scale][query of the block]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, c = lane & 31;
    int row_tile, z;
    attn_block(row_tile, z);
    const int k0 = row_tile * AT_QROWS + wave * 32;
    const float* Q = (const float*)g.Q + (long long)z * g.q_bs;
    const float* K = (const float*)g.K + (long long)z * g.k_bs;
    const float* V = (const float*)g.V + (long long)z * g.v_bs;
    const float* dO = (const float*)g.dO + (long long)z * g.do_bs;
    const char* q_end = (const char*)(Q + ((long long)(g.sq - 1) * g.q_rs + D));
    const char* k_end = (const char*)(K + ((long long)(g.sk - 1) * g.k_rs + D));
    const char* v_end = (const char*)(V + ((long long)(g.sk - 1) * g.v_rs + D));
    const char* do_end = (const char*)(dO + ((long long)(g.sq - 1) * g.do_rs + D));
    const float sc = g.scale * 1.44269504088896341f;
    const float* Lz = g.L + (long long)z * g.sq;
    const float* Dz = g.Dq + (long long)z * g.sq;

    float kf[KJ], vf[KJ];                            // B operands: key k0 + c, d = j + KJ*h
    load_half_row<KJ>(kf, K, g.k_rs, k0, g.sk, k_end, c, h);
    load_half_row<KJ>(vf, V, g.v_rs, k0, g.sk, v_end, c, h);

    f32x16_t dkt[DT], dvt[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) { dkt[dt][v] = 0.f; dvt[dt][v] = 0.f; }

    const int nblocks = (g.sq + AT_KEYS - 1) / AT_KEYS;
    u32x4_t qr[Blk::PIECES], dor[Blk::PIECES];
    // L and Dq of the block's queries: every lane requests query qb + lane % 32 with unconditional buffer loads (zero
    // past sq); wave 0 puts them in LDS, L in log2 units and +inf past sq (those rows' probabilities become exactly 0)
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
    Blk::store(qr, qlds[0]); Blk::store(dor, dolds[0]);
    store_rowv(0, 0);
    Blk::load(qr, Q, g.q_rs, AT_KEYS, g.sq, q_end);
    Blk::load(dor, dO, g.do_rs, AT_KEYS, g.sq, do_end);
    load_rowv(AT_KEYS);
    __syncthreads();

    for (int blk = 0; blk < nblocks; blk++) {
        const int qb = blk * AT_KEYS, cur = blk & 1;
        f32x16_t st, dp;
#pragma unroll
        for (int v = 0; v < 16; v++) { st[v] = 0.f; dp[v] = 0.f; }
        st = product_over_d<D>(qlds[cur], kf, c, h, st);                    // S: queries x keys
        dp = product_over_d<D>(dolds[cur], vf, c, h, dp);                   // dP
        Blk::store(qr, qlds[cur ^ 1]); Blk::store(dor, dolds[cur ^ 1]);
        store_rowv(cur ^ 1, qb + AT_KEYS);
        Blk::load(qr, Q, g.q_rs, qb + 2 * AT_KEYS, g.sq, q_end);
        Blk::load(dor, dO, g.do_rs, qb + 2 * AT_KEYS, g.sq, do_end);
        load_rowv(qb + 2 * AT_KEYS);
        float p[16], ds[16];
#pragma unroll
        for (int v4 = 0; v4 < 4; v4++) {
            // registers 4*v4 .. +3 are queries qb + 8*v4 + 4h + (0..3)
            const f32x4v_t l4 = *(const f32x4v_t*)&rowlds[cur][0][8 * v4 + 4 * h];
            const f32x4v_t d4 = *(const f32x4v_t*)&rowlds[cur][1][8 * v4 + 4 * h];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int v = 4 * v4 + e;
                p[v] = __builtin_amdgcn_exp2f(fmaf(st[v], sc, -l4[e]));
                ds[v] = p[v] * fmaf(dp[v], g.scale, -d4[e]);
            }
        }
        product_over_rows<D>(dvt, dolds[cur], p, c, h);                     // dV^T += dO^T P
        product_over_rows<D>(dkt, qlds[cur], ds, c, h);                     // dK^T += Q^T dS
        __syncthreads();
    }
    const int key = k0 + c;
    if (key < g.sk) {
        write_rows_t<D>((float*)g.dK + ((long long)z * g.sk + key) * D, dkt, h, 1.f);
        write_rows_t<D>((float*)g.dV + ((long long)z * g.sk + key) * D, dvt, h, 1.f);
    }
}

int launch_attention_f32(const AttnArgs& g, int d) {
    dim3 grid((g.sq + AT_QROWS - 1) / AT_QROWS, g.batch);
    switch (d) {
        case 32: hipLaunchKernelGGL((attention_fwd32_kernel<32>), grid, dim3(256), 0, current_stream(), g); break;
        case 64: hipLaunchKernelGGL((attention_fwd32_kernel<64>), grid, dim3(256), 0, current_stream(), g); break;
        case 128: hipLaunchKernelGGL((attention_fwd32_kernel<128>), grid, dim3(256), 0, current_stream(), g); break;      // (68 KB of static LDS: one workgroup per CU)
        default: set_error("rp_hip_attention_forward: float32 head dimension %d (supported: 32, 64, 128)", d); return -1;
    }
    return check_launch("attention_fwd32_kernel") ? 0 : -1;
}

int launch_attention_bwd_f32(const AttnBwdArgs& g, int d) {
    dim3 gq((g.sq + AT_QROWS - 1) / AT_QROWS, g.batch), gk((g.sk + AT_QROWS - 1) / AT_QROWS, g.batch);
    switch (d) {
        case 32:
            hipLaunchKernelGGL((attention_bwd_dq32_kernel<32>), gq, dim3(256), 0, current_stream(), g);
            hipLaunchKernelGGL((attention_bwd_dkv32_kernel<32>), gk, dim3(256), 0, current_stream(), g);
            break;
        case 64:
            hipLaunchKernelGGL((attention_bwd_dq32_kernel<64>), gq, dim3(256), 0, current_stream(), g);
            hipLaunchKernelGGL((attention_bwd_dkv32_kernel<64>), gk, dim3(256), 0, current_stream(), g);
            break;
        case 128:
            hipLaunchKernelGGL((attention_bwd_dq32_kernel<128>), gq, dim3(256), 0, current_stream(), g);
            hipLaunchKernelGGL((attention_bwd_dkv32_kernel<128>), gk, dim3(256), 0, current_stream(), g);
            break;
        default: set_error("rp_hip_attention_backward: float32 head dimension %d (supported: 32, 64, 128)", d); return -1;
    }
    return check_launch("attention backward kernels (float32)") ? 0 : -1;
}

}  // namespace rp
