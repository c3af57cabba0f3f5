// The finish of a k split inside one launch, shared by the kernels that use it.
#pragma once
#include "rp_gemm.h"

namespace rp {

// ---- the finish of a k split, shared by the kernels that split k inside one launch ----
// The epilogue of four adjacent outputs of one row, stored as one 8-byte vector where the layout allows (c_vec).
template <typename T>
struct SplitkOutput {
    T* C;
    const T* bias;
    long long c_rs, c_cs;
    bool has_bias, accum, c_vec;
    // (c_offset: elements from g.C to the matrix of a batch that is written)
    __device__ __forceinline__ explicit SplitkOutput(const GemmArgs& g, long long c_offset = 0)
        : C((T*)g.C + c_offset), bias((const T*)g.bias), c_rs(g.c_rs), c_cs(g.c_cs), has_bias(g.bias != nullptr), accum(g.accumulate != 0),
          c_vec(g.c_cs == 1 && g.c_rs % 4 == 0 && ((uintptr_t)((T*)g.C + c_offset) & 7) == 0) {}
    // True when an output needs nothing but the rounding and can be stored as one vector: callers then take
    // store_quad_plain, which has no branch per value (the general form below decides bias, accumulation and layout
    // for every value again, some sixty scalar branches for four quads).
    __device__ __forceinline__ bool plain() const { return !has_bias && !accum && c_vec; }
    __device__ __forceinline__ void store_quad_plain(int row, int col, f32x4_t sum) const {
        T y[4];
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = finish<T>(sum[e], false, T{}, false, T{});
        u32x2_t w = {(uint32_t)y[0].bits | ((uint32_t)y[1].bits << 16), (uint32_t)y[2].bits | ((uint32_t)y[3].bits << 16)};
        *(u32x2_t*)(C + (long long)row * c_rs + col) = w;
    }
    __device__ __forceinline__ void store_quad(int row, int col, f32x4_t sum) const {
        T y[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            T* pc = C + (long long)row * c_rs + (long long)(col + e) * c_cs;
            T old = accum ? *pc : T{};
            y[e] = finish<T>(sum[e], has_bias, has_bias ? bias[col + e] : T{}, accum, old);
        }
        if (c_vec) {
            u32x2_t w = {(uint32_t)y[0].bits | ((uint32_t)y[1].bits << 16), (uint32_t)y[2].bits | ((uint32_t)y[3].bits << 16)};
            *(u32x2_t*)(C + (long long)row * c_rs + col) = w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) C[(long long)row * c_rs + (long long)(col + e) * c_cs] = y[e];
        }
    }
    // N quads of one thread (dead ones skipped), with the choice between the two forms made once
    template <int N>
    __device__ __forceinline__ void store_quads(const int (&row)[N], const int (&col)[N], const bool (&live)[N], const f32x4_t (&sum)[N]) const {
        if (plain()) {
#pragma unroll
            for (int q = 0; q < N; q++)
                if (live[q]) store_quad_plain(row[q], col[q], sum[q]);
        } else {
#pragma unroll
            for (int q = 0; q < N; q++)
                if (live[q]) store_quad(row[q], col[q], sum[q]);
        }
    }
};

// A block's arrival at its tile's counter after its partial stores.  Every thread first waits until its own stores are
// acknowledged (by the XCD's L2 when all blocks of the tile run on that XCD: `local`; by memory for device-scope
// stores otherwise), so no cache-wide write-back is needed.  True in every thread of the block that arrived last.
__device__ __forceinline__ bool splitk_arrive(int* counter, int nsplit, bool local, bool* flag) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        int before;
        if (local) before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);    // executed by this XCD's L2
        else before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = before == nsplit - 1;
    }
    __syncthreads();
    return *flag;
}

// The block that arrived last adds the fp32 partials [split][g.m][g.n] of rows m0 .. m_end-1 and COLS columns from n0 in
// split order (so the result does not depend on which block that is), runs the epilogue and leaves the counter at
// zero for the next launch.  QN quads per thread and pass; the loads of U splits of all of a thread's quads are in
// flight together (QN * U * 4 registers, which count against the calling kernel's occupancy): their offsets are all
// computed first and the kind of load is a template parameter, so that the loads are issued back to back (with a
// branch per load the compiler puts waits between them, and the finish takes a memory round trip per load).  (Plain
// loads of the partials cannot hit stale lines of this CU's vector cache: it fills on the CU's own loads only and
// starts every launch empty, and the one block of a launch that reads a tile's partials reads them here for the first
// time.)
template <typename T, int COLS, int QN, int U_SPLITS, bool LOCAL>
__device__ __forceinline__ void splitk_finish_window_scope(const GemmArgs& g, const SplitkOutput<T>& out, __amdgpu_buffer_rsrc_t part_rsrc, int nsplit,
                                                           int m0, int m_end, int n0, int* counter) {
    const long long split_stride = (long long)g.m * g.n;
    constexpr int QPR = COLS / 4;                        // quads per row of the window
    constexpr int RPP = 256 * QN / QPR;                  // rows per pass
    for (int r0 = m0; r0 < m_end; r0 += RPP) {
        long long at[QN];
        bool live[QN];
        int row[QN], col[QN];
#pragma unroll
        for (int q = 0; q < QN; q++) {
            const int idx = threadIdx.x + 256 * q;
            row[q] = r0 + idx / QPR; col[q] = n0 + (idx % QPR) * 4;
            live[q] = row[q] < m_end && col[q] < g.n;    // n is a multiple of 4 here, so a quad is wholly in or out
            at[q] = live[q] ? ((long long)row[q] * g.n + col[q]) * 4 : (long long)BUFFER_OOB;      // bytes; dead quads read zeros
        }
        f32x4_t sum[QN];
#pragma unroll
        for (int q = 0; q < QN; q++) sum[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < nsplit; sp += U_SPLITS) {
            int off[U_SPLITS][QN];
#pragma unroll
            for (int u = 0; u < U_SPLITS; u++)
#pragma unroll
                for (int q = 0; q < QN; q++) off[u][q] = (live[q] && sp + u < nsplit) ? (int)(at[q] + (sp + u) * split_stride * 4) : (int)BUFFER_OOB;
#pragma unroll
            for (int u = 0; u < U_SPLITS; u++)
#pragma unroll
                for (int q = 0; q < QN; q++) asm volatile("" : "+v"(off[u][q]));
            __builtin_amdgcn_sched_barrier(0);
            u32x4_t v[U_SPLITS][QN];
#pragma unroll
            for (int u = 0; u < U_SPLITS; u++)
#pragma unroll
                for (int q = 0; q < QN; q++) v[u][q] = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, off[u][q], 0, LOCAL ? 0 : SPLITK_DEVICE_SCOPE);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U_SPLITS; u++)
#pragma unroll
                for (int q = 0; q < QN; q++) sum[q] += __builtin_bit_cast(f32x4_t, v[u][q]);       // split order; absent splits add +0
        }
        out.store_quads(row, col, live, sum);
    }
    if (threadIdx.x == 0) {
        if (LOCAL) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename T, int COLS, int QN, int U_SPLITS = 8>
__device__ __forceinline__ void splitk_finish_window(const GemmArgs& g, const SplitkOutput<T>& out, __amdgpu_buffer_rsrc_t part_rsrc, int nsplit,
                                                     int m0, int m_end, int n0, bool local, int* counter) {
    if (local) splitk_finish_window_scope<T, COLS, QN, U_SPLITS, true>(g, out, part_rsrc, nsplit, m0, m_end, n0, counter);
    else splitk_finish_window_scope<T, COLS, QN, U_SPLITS, false>(g, out, part_rsrc, nsplit, m0, m_end, n0, counter);
}

}  // namespace rp
