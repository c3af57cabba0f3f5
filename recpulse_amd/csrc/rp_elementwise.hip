// Element-wise, row-wise and reduction entry points that the benchmark
// configurations run around the GEMMs: add / broadcasting add, scalar multiply, relu and softmax
// with their VJPs, strided gather, reductions, fill / convert, and the
// on-device bias gradient and cross-entropy.  16-bit dtypes compute in fp32
// and narrow once with the reference's rounding, like the reference's host
// path (functional/functional.c:10-56).
#include "rp_common.h"

#include <cfloat>

namespace rp {

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;      // one 16-byte memory access

static constexpr int kThreads = 256;
static constexpr int kMaxDims = 8;

static inline unsigned grid_for(size_t n, int threads = kThreads, size_t cap = 1u << 20) {
    size_t b = (n + threads - 1) / threads;
    if (b < 1) b = 1;
    if (b > cap) b = cap;
    return (unsigned)b;
}

// ---- flat maps ----------------------------------------------------------------
// out[i] = op(x1[i], x2[i]) in the accumulate type, narrowed once.  When every pointer is 16-byte aligned each
// thread moves whole 16-byte vectors, four per pass with all four loads in flight; a scalar loop takes the rest.
template <typename A> struct AddOp { __device__ __forceinline__ A operator()(A a, A b) const { return a + b; } };
template <typename A> struct MulScalarOp { A s; __device__ __forceinline__ A operator()(A a, A) const { return a * s; } };
template <typename A> struct ReluOp { __device__ __forceinline__ A operator()(A a, A) const { return a > (A)0 ? a : (A)0; } };
template <typename A> struct BackReluOp { __device__ __forceinline__ A operator()(A g, A x) const { return x > (A)0 ? g : (A)0; } };   // (grad, input)

template <typename T, bool TWO, typename Op>
__global__ void map_scalar_kernel(T* out, const T* x1, const T* x2, Op op, size_t begin, size_t n) {
    using A = typename traits<T>::acc;
    for (size_t i = begin + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        out[i] = narrow<T>(op(widen(x1[i]), TWO ? widen(x2[i]) : (A)0));
}

template <typename T, bool TWO, typename Op>
__global__ void __launch_bounds__(kThreads) map_vec_kernel(T* out, const T* x1, const T* x2, Op op, size_t nvec) {
    using A = typename traits<T>::acc;
    constexpr int VEC = 16 / sizeof(T), U = 4;
    const u32x4_t* p1 = (const u32x4_t*)x1;
    const u32x4_t* p2 = (const u32x4_t*)x2;
    u32x4_t* po = (u32x4_t*)out;
    for (size_t base = (size_t)blockIdx.x * (kThreads * U); base < nvec; base += (size_t)gridDim.x * (kThreads * U)) {
        u32x4_t r1[U], r2[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            size_t i = base + u * kThreads + threadIdx.x;
            if (i < nvec) {
                r1[u] = __builtin_nontemporal_load(p1 + i);
                if (TWO) r2[u] = __builtin_nontemporal_load(p2 + i);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            size_t i = base + u * kThreads + threadIdx.x;
            if (i >= nvec) continue;
            T a[VEC], b[VEC], o[VEC];
            memcpy(a, &r1[u], 16);
            if (TWO) memcpy(b, &r2[u], 16);
#pragma unroll
            for (int e = 0; e < VEC; e++) o[e] = narrow<T>(op(widen(a[e]), TWO ? widen(b[e]) : (A)0));
            u32x4_t w;
            memcpy(&w, o, 16);
            __builtin_nontemporal_store(w, po + i);
        }
    }
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

template <typename T, bool TWO, typename Op>
static void launch_map(T* out, const T* x1, const T* x2, Op op, size_t n) {
    constexpr int VEC = 16 / sizeof(T);
    size_t nvec = (aligned16(out) && aligned16(x1) && (!TWO || aligned16(x2))) ? n / VEC : 0;
    if (nvec) {
        size_t blocks = (nvec + kThreads * 4 - 1) / (kThreads * 4);
        if (blocks > (1u << 20)) blocks = 1u << 20;
        hipLaunchKernelGGL((map_vec_kernel<T, TWO, Op>), dim3((unsigned)blocks), dim3(kThreads), 0, current_stream(), out, x1, x2, op, nvec);
    }
    size_t done = nvec * VEC;
    if (done < n)
        hipLaunchKernelGGL((map_scalar_kernel<T, TWO, Op>), dim3(grid_for(n - done)), dim3(kThreads), 0, current_stream(), out, x1, x2, op, done, n);
}

// p[0 .. n) = v with 16-byte stores over the aligned middle (a store of one element per lane fills half a cache line
// per wave and runs at a third of the bandwidth); the elements before and after it go one by one.
template <typename T>
__device__ __forceinline__ void fill_span(T* p, T v, size_t n) {
    constexpr int VEC = 16 / (int)sizeof(T);
    typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
    size_t head = ((16 - ((uintptr_t)p & 15)) & 15) / sizeof(T);
    head = head < n ? head : n;
    const size_t nvec = (n - head) / VEC, tail0 = head + nvec * VEC;
    T lanes[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) lanes[e] = v;
    u32x4 pattern;
    __builtin_memcpy(&pattern, lanes, 16);
    u32x4* body = (u32x4*)(p + head);
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = tid; i < nvec; i += stride) body[i] = pattern;
    if (tid < head) p[tid] = v;
    if (tid < n - tail0) p[tail0 + tid] = v;
}

template <typename T>
__global__ void fill_kernel(T* p, T v, size_t n) {
    fill_span(p, v, n);
}

// out[i] = scalar[0] * scale, the product taken in double and narrowed once (what the host computes when it reads
// the scalar back first)
template <typename T>
__global__ void fill_scaled_kernel(T* out, const T* scalar, double scale, size_t n) {
    const T v = narrow<T>((typename traits<T>::acc)((double)widen(scalar[0]) * scale));
    fill_span(out, v, n);
}

// dtype conversion pivots through fp32 like the reference (core/tensor_host.c:130-207),
// except float64 <-> float64 / float32 which are direct.
// GROUP elements per thread (the whole groups of the array; the rest go one by one), read and written as one
// vector each when `vectors` says both arrays are aligned for that.
template <typename D, typename S>
__global__ void convert_kernel(D* dst, const S* src, size_t n, int vectors) {
    constexpr int GROUP = 16 / (int)(sizeof(D) < sizeof(S) ? sizeof(D) : sizeof(S));      // the narrower side moves 16 bytes
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    const size_t groups = vectors ? n / GROUP : 0;
    for (size_t i = tid; i < groups; i += stride) {
        S in[GROUP];
        D out[GROUP];
        __builtin_memcpy(in, __builtin_assume_aligned(src + i * GROUP, 16), sizeof(in));
#pragma unroll
        for (int e = 0; e < GROUP; e++) out[e] = narrow<D>((typename traits<D>::acc)widen(in[e]));
        __builtin_memcpy(__builtin_assume_aligned(dst + i * GROUP, 16), out, sizeof(out));
    }
    for (size_t i = groups * GROUP + tid; i < n; i += stride) dst[i] = narrow<D>((typename traits<D>::acc)widen(src[i]));
}

// ---- broadcasting add ------------------------------------------------------------
struct StridedArgs {
    int ndim;
    int shape[kMaxDims];
    long long s1[kMaxDims];
    long long s2[kMaxDims];
};

template <typename T>
__global__ void add_strided_kernel(T* out, const T* x1, const T* x2, StridedArgs a, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        size_t rem = i;
        long long i1 = 0, i2 = 0;
        for (int d = a.ndim - 1; d >= 0; d--) {
            size_t c = rem % (size_t)a.shape[d];
            rem /= (size_t)a.shape[d];
            i1 += (long long)c * a.s1[d];
            i2 += (long long)c * a.s2[d];
        }
        out[i] = narrow<T>(widen(x1[i1]) + widen(x2[i2]));
    }
}

// the Linear case: [rows, cols] dense + [cols]
template <typename T>
__global__ void add_row_vector_kernel(T* out, const T* x, const T* v, size_t n, int cols) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        out[i] = narrow<T>(widen(x[i]) + widen(v[i % (size_t)cols]));
}

struct GatherArgs {
    int ndim;
    int shape[kMaxDims];
    long long strides[kMaxDims];
};

template <typename T>
__global__ void gather_kernel(T* out, const T* in, GatherArgs a, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        size_t rem = i;
        long long off = 0;
        for (int d = a.ndim - 1; d >= 0; d--) {
            off += (long long)(rem % (size_t)a.shape[d]) * a.strides[d];
            rem /= (size_t)a.shape[d];
        }
        out[i] = in[off];
    }
}

// ---- softmax family ----------------------------------------------------------------
// inner == 1: one 64-lane wave per row, lanes stride the row, wave reductions
// by DPP-free shuffles.  Otherwise one thread per (outer, inner) pair walks
// its row serially (the reference device kernel's shape,
// functional/functional_device.cu:1486-1508).
template <typename A>
__device__ __forceinline__ A wave_max(A v) {
    for (int o = 32; o > 0; o >>= 1) { A t = __shfl_xor(v, o, 64); v = t > v ? t : v; }
    return v;
}
template <typename A>
__device__ __forceinline__ A wave_sum(A v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float rp_exp(float x) { return expf(x); }
__device__ __forceinline__ double rp_exp(double x) { return exp(x); }
__device__ __forceinline__ float rp_log(float x) { return logf(x); }
__device__ __forceinline__ double rp_log(double x) { return log(x); }
template <typename A> __device__ __forceinline__ A lowest();
template <> __device__ __forceinline__ float lowest<float>() { return -FLT_MAX; }
template <> __device__ __forceinline__ double lowest<double>() { return -DBL_MAX; }

template <typename T, bool LOG>
__global__ void softmax_rows_kernel(T* out, const T* x, size_t rows, size_t dim) {
    using A = typename traits<T>::acc;
    int lane = threadIdx.x & 63;
    size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    size_t nwaves = ((size_t)gridDim.x * blockDim.x) >> 6;
    for (size_t r = wave; r < rows; r += nwaves) {
        const T* xr = x + r * dim;
        T* orow = out + r * dim;
        A mx = lowest<A>();
        for (size_t d = lane; d < dim; d += 64) { A v = widen(xr[d]); mx = v > mx ? v : mx; }
        mx = wave_max(mx);
        A sum = 0;
        for (size_t d = lane; d < dim; d += 64) sum += rp_exp(widen(xr[d]) - mx);
        sum = wave_sum(sum);
        if (LOG) {
            A lse = rp_log(sum);
            for (size_t d = lane; d < dim; d += 64) orow[d] = narrow<T>(widen(xr[d]) - mx - lse);
        } else {
            for (size_t d = lane; d < dim; d += 64) orow[d] = narrow<T>(rp_exp(widen(xr[d]) - mx) / sum);
        }
    }
}

// Rows that fit a wave's registers (dim <= 64 lanes * CH chunks * 16 bytes, dim a whole number of 16-byte
// vectors, aligned rows): each lane loads CH 16-byte pieces of the row once, everything else happens in
// registers, and the result leaves as 16-byte stores.  One wave per row, four rows per block.
// With has_scale the input is first multiplied by the scalar and rounded to T, which is what a separate scalar multiply
// in front of the softmax leaves in memory (reference ops/ops.c:6022-6086 then 5721-5788): one pass instead of two, same bits.
template <typename T, bool LOG, int CH>
__global__ void __launch_bounds__(kThreads) softmax_rows_reg_kernel(T* out, const T* x, size_t rows, int dim, bool has_scale, typename traits<T>::acc scale) {
    using A = typename traits<T>::acc;
    constexpr int VEC = 16 / sizeof(T);
    const int lane = threadIdx.x & 63;
    const size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const size_t nwaves = ((size_t)gridDim.x * blockDim.x) >> 6;
    for (size_t r = wave; r < rows; r += nwaves) {
        const T* xr = x + r * (size_t)dim;
        T* orow = out + r * (size_t)dim;
        u32x4_t raw[CH];
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int e0 = (c * 64 + lane) * VEC;
            if (e0 < dim) raw[c] = __builtin_nontemporal_load((const u32x4_t*)(xr + e0));
        }
        A v[CH][VEC];
        A mx = lowest<A>();
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const bool in = (c * 64 + lane) * VEC < dim;
            T t[VEC];
            memcpy(t, &raw[c], 16);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                A xv = widen(t[e]);
                if (has_scale) xv = widen(narrow<T>(xv * scale));
                v[c][e] = in ? xv : lowest<A>();
                mx = v[c][e] > mx ? v[c][e] : mx;
            }
        }
        mx = wave_max(mx);
        A sum = 0;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const bool in = (c * 64 + lane) * VEC < dim;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                // 16-bit outputs keep 8 or 11 significant bits: the hardware exp2 (1 ulp of fp32) is ample there
                A ex;
                if constexpr (sizeof(T) == 2) ex = __builtin_amdgcn_exp2f((v[c][e] - mx) * 1.44269504088896341f);
                else ex = rp_exp(v[c][e] - mx);
                sum += in ? ex : (A)0;
                if (!LOG) v[c][e] = ex;
            }
        }
        sum = wave_sum(sum);
        const A lse = LOG ? rp_log(sum) : (A)0;
        const A inv = (A)1 / sum;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int e0 = (c * 64 + lane) * VEC;
            if (e0 >= dim) continue;
            T o[VEC];
#pragma unroll
            for (int e = 0; e < VEC; e++) o[e] = narrow<T>(LOG ? v[c][e] - mx - lse : (sizeof(T) == 2 ? v[c][e] * inv : v[c][e] / sum));
            u32x4_t w;
            memcpy(&w, o, 16);
            __builtin_nontemporal_store(w, (u32x4_t*)(orow + e0));
        }
    }
}

// With has_scale the gradient is rounded to T and then multiplied by the scalar and rounded again: the softmax's own
// gradient followed by that of a scalar multiply in front of it (reference ops/grad_host.c:1387-1398, ops/ops.c:6022-6086).
template <typename T, int CH>
__global__ void __launch_bounds__(kThreads) backwards_softmax_rows_reg_kernel(const T* gc, const T* y, T* gx, size_t rows, int dim, bool has_scale, typename traits<T>::acc scale) {
    using A = typename traits<T>::acc;
    constexpr int VEC = 16 / sizeof(T);
    const int lane = threadIdx.x & 63;
    const size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const size_t nwaves = ((size_t)gridDim.x * blockDim.x) >> 6;
    for (size_t r = wave; r < rows; r += nwaves) {
        const size_t row0 = r * (size_t)dim;
        u32x4_t rg[CH], ry[CH];
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int e0 = (c * 64 + lane) * VEC;
            if (e0 < dim) {
                rg[c] = __builtin_nontemporal_load((const u32x4_t*)(gc + row0 + e0));
                ry[c] = __builtin_nontemporal_load((const u32x4_t*)(y + row0 + e0));
            }
        }
        A g[CH][VEC], s[CH][VEC];
        A dot = 0;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const bool in = (c * 64 + lane) * VEC < dim;
            T tg[VEC], ty[VEC];
            memcpy(tg, &rg[c], 16);
            memcpy(ty, &ry[c], 16);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                g[c][e] = in ? widen(tg[e]) : (A)0;
                s[c][e] = in ? widen(ty[e]) : (A)0;
                dot += g[c][e] * s[c][e];
            }
        }
        dot = wave_sum(dot);
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int e0 = (c * 64 + lane) * VEC;
            if (e0 >= dim) continue;
            T o[VEC];
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                o[e] = narrow<T>(s[c][e] * (g[c][e] - dot));
                if (has_scale) o[e] = narrow<T>(widen(o[e]) * scale);
            }
            u32x4_t w;
            memcpy(&w, o, 16);
            __builtin_nontemporal_store(w, (u32x4_t*)(gx + row0 + e0));
        }
    }
}

// chunks per lane the register kernels need for this row length, or 0 when the row does not qualify
template <typename T>
static int reg_row_chunks(size_t dim, const void* p0, const void* p1, const void* p2) {
    constexpr size_t VEC = 16 / sizeof(T);
    if (dim % VEC || dim > 64 * VEC * 8 || !aligned16(p0) || !aligned16(p1) || (p2 && !aligned16(p2))) return 0;
    size_t ch = (dim + 64 * VEC - 1) / (64 * VEC);
    return ch <= 1 ? 1 : ch <= 2 ? 2 : ch <= 4 ? 4 : 8;
}

template <typename T, int CH>
static void launch_softmax_reg_ch(T* out, const T* x, size_t rows, size_t dim, unsigned blocks, bool take_log, bool has_scale, typename traits<T>::acc scale) {
    if (take_log) hipLaunchKernelGGL((softmax_rows_reg_kernel<T, true, CH>), dim3(blocks), dim3(kThreads), 0, current_stream(), out, x, rows, (int)dim, has_scale, scale);
    else          hipLaunchKernelGGL((softmax_rows_reg_kernel<T, false, CH>), dim3(blocks), dim3(kThreads), 0, current_stream(), out, x, rows, (int)dim, has_scale, scale);
}
// launch the register kernel when the rows qualify; false means the caller takes the general one
template <typename T>
static bool launch_softmax_reg(T* out, const T* x, size_t rows, size_t dim, unsigned blocks, bool take_log, bool has_scale = false, typename traits<T>::acc scale = 1) {
    switch (reg_row_chunks<T>(dim, out, x, nullptr)) {
        case 1: launch_softmax_reg_ch<T, 1>(out, x, rows, dim, blocks, take_log, has_scale, scale); return true;
        case 2: launch_softmax_reg_ch<T, 2>(out, x, rows, dim, blocks, take_log, has_scale, scale); return true;
        case 4: launch_softmax_reg_ch<T, 4>(out, x, rows, dim, blocks, take_log, has_scale, scale); return true;
        case 8: launch_softmax_reg_ch<T, 8>(out, x, rows, dim, blocks, take_log, has_scale, scale); return true;
        default: return false;
    }
}
template <typename T>
static bool launch_bsoftmax_reg(const T* gc, const T* y, T* gx, size_t rows, size_t dim, unsigned blocks, bool has_scale = false, typename traits<T>::acc scale = 1) {
#define RP_BSOFTMAX_REG(CH) hipLaunchKernelGGL((backwards_softmax_rows_reg_kernel<T, CH>), dim3(blocks), dim3(kThreads), 0, current_stream(), gc, y, gx, rows, (int)dim, has_scale, scale)
    switch (reg_row_chunks<T>(dim, gc, y, gx)) {
        case 1: RP_BSOFTMAX_REG(1); return true;
        case 2: RP_BSOFTMAX_REG(2); return true;
        case 4: RP_BSOFTMAX_REG(4); return true;
        case 8: RP_BSOFTMAX_REG(8); return true;
        default: return false;
    }
#undef RP_BSOFTMAX_REG
}

template <typename T, bool LOG>
__global__ void softmax_strided_kernel(T* out, const T* x, size_t outer, size_t dim, size_t inner) {
    using A = typename traits<T>::acc;
    size_t n = outer * inner;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (size_t)gridDim.x * blockDim.x) {
        size_t base = (t / inner) * dim * inner + (t % inner);
        A mx = lowest<A>();
        for (size_t d = 0; d < dim; d++) { A v = widen(x[base + d * inner]); mx = v > mx ? v : mx; }
        A sum = 0;
        for (size_t d = 0; d < dim; d++) sum += rp_exp(widen(x[base + d * inner]) - mx);
        if (LOG) {
            A lse = rp_log(sum);
            for (size_t d = 0; d < dim; d++) out[base + d * inner] = narrow<T>(widen(x[base + d * inner]) - mx - lse);
        } else {
            for (size_t d = 0; d < dim; d++) out[base + d * inner] = narrow<T>(rp_exp(widen(x[base + d * inner]) - mx) / sum);
        }
    }
}

template <typename T>
__global__ void backwards_softmax_rows_kernel(const T* gc, const T* y, T* gx, size_t rows, size_t dim) {
    using A = typename traits<T>::acc;
    int lane = threadIdx.x & 63;
    size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    size_t nwaves = ((size_t)gridDim.x * blockDim.x) >> 6;
    for (size_t r = wave; r < rows; r += nwaves) {
        const T* g = gc + r * dim;
        const T* s = y + r * dim;
        A dot = 0;
        for (size_t d = lane; d < dim; d += 64) dot += widen(g[d]) * widen(s[d]);
        dot = wave_sum(dot);
        for (size_t d = lane; d < dim; d += 64) gx[r * dim + d] = narrow<T>(widen(s[d]) * (widen(g[d]) - dot));
    }
}

template <typename T>
__global__ void backwards_softmax_strided_kernel(const T* gc, const T* y, T* gx, size_t outer, size_t dim, size_t inner) {
    using A = typename traits<T>::acc;
    size_t n = outer * inner;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (size_t)gridDim.x * blockDim.x) {
        size_t base = (t / inner) * dim * inner + (t % inner);
        A dot = 0;
        for (size_t d = 0; d < dim; d++) dot += widen(gc[base + d * inner]) * widen(y[base + d * inner]);
        for (size_t d = 0; d < dim; d++)
            gx[base + d * inner] = narrow<T>(widen(y[base + d * inner]) * (widen(gc[base + d * inner]) - dot));
    }
}

// gradient of log_softmax (reference ops/grad_host.c:1428-1500): gx = g - exp(y) * sum_d g, with y the op's output.
// One thread per (outer, inner) pair, the sum in index order as the reference's host loop runs it; for rows that
// are contiguous (inner == 1) a wave per row with the partial sums of the lanes added by wave_sum.
template <typename T>
__global__ void backwards_log_softmax_rows_kernel(const T* gc, const T* y, T* gx, size_t rows, size_t dim) {
    using A = typename traits<T>::acc;
    int lane = threadIdx.x & 63;
    size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    size_t nwaves = ((size_t)gridDim.x * blockDim.x) >> 6;
    for (size_t r = wave; r < rows; r += nwaves) {
        const T* g = gc + r * dim;
        const T* l = y + r * dim;
        A sum = 0;
        for (size_t d = lane; d < dim; d += 64) sum += widen(g[d]);
        sum = wave_sum(sum);
        for (size_t d = lane; d < dim; d += 64) gx[r * dim + d] = narrow<T>(widen(g[d]) - rp_exp(widen(l[d])) * sum);
    }
}

template <typename T>
__global__ void backwards_log_softmax_strided_kernel(const T* gc, const T* y, T* gx, size_t outer, size_t dim, size_t inner) {
    using A = typename traits<T>::acc;
    size_t n = outer * inner;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (size_t)gridDim.x * blockDim.x) {
        size_t base = (t / inner) * dim * inner + (t % inner);
        A sum = 0;
        for (size_t d = 0; d < dim; d++) sum += widen(gc[base + d * inner]);
        for (size_t d = 0; d < dim; d++)
            gx[base + d * inner] = narrow<T>(widen(gc[base + d * inner]) - rp_exp(widen(y[base + d * inner])) * sum);
    }
}

// ---- reductions ----------------------------------------------------------------------
// Deterministic two-level sum in two launches: each block sums a contiguous slab
// (threads stride it, then a fixed-order LDS tree) into a file-scope partials
// array; a one-thread second kernel adds the partials in index order.  Calls that
// overlap on one device would share the array: the library's single-stream
// ordering keeps them apart.
static constexpr int kMaxPartials = 1024;
__device__ double g_partials[kMaxPartials];

template <typename T>
__global__ void sum_partials_kernel(const T* x, size_t n) {
    using A = typename traits<T>::acc;
    __shared__ A red[kThreads];
    size_t per_block = (n + gridDim.x - 1) / gridDim.x;
    size_t lo = (size_t)blockIdx.x * per_block;
    size_t hi = lo + per_block < n ? lo + per_block : n;
    A s = 0;
    for (size_t i = lo + threadIdx.x; i < hi; i += blockDim.x) s += widen(x[i]);
    red[threadIdx.x] = s;
    __syncthreads();
    for (int o = kThreads / 2; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) g_partials[blockIdx.x] = (double)red[0];
}

template <typename T>
__global__ void sum_finish_kernel(T* out, int nparts, double scale) {
    using A = typename traits<T>::acc;
    A total = 0;
    for (int b = 0; b < nparts; b++) total += (A)g_partials[b];
    if (scale != 1.0) total = (A)(total / (A)scale);
    out[0] = narrow<T>(total);
}

// reduce the middle axis of [outer, dim, inner]; one thread per output, serial in dim
template <typename T>
__global__ void sum_dim_kernel(T* out, const T* x, size_t outer, size_t dim, size_t inner) {
    using A = typename traits<T>::acc;
    size_t n = outer * inner;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (size_t)gridDim.x * blockDim.x) {
        size_t base = (t / inner) * dim * inner + (t % inner);
        A s = 0;
        for (size_t d = 0; d < dim; d++) s += widen(x[base + d * inner]);
        out[t] = narrow<T>(s);
    }
}

// Linear's bias gradient: out[j] = sum_i grad[i, j], rows added top to bottom
// in the accumulate type — the order the reference's host loop produces
// (ops/ops.c:7048-7061).  Threads of a block own adjacent columns, so every
// row read is one coalesced segment.
template <typename T>
__global__ void reduce_rows_kernel(T* out, const T* g, int rows, int cols, int accumulate) {
    using A = typename traits<T>::acc;
    int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= cols) return;
    A s = 0;
    const T* p = g + j;
    int i = 0;
    constexpr int U = 16;                       // independent loads in flight; the adds stay in row order
    for (; i + U <= rows; i += U) {
        A v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = widen(p[(size_t)(i + u) * cols]);
#pragma unroll
        for (int u = 0; u < U; u++) s += v[u];
    }
    for (; i < rows; i++) s += widen(p[(size_t)i * cols]);
    T r = narrow<T>(s);
    if (accumulate) r = narrow<T>(widen(out[j]) + widen(r));
    out[j] = r;
}

// ---- cross-entropy ----------------------------------------------------------------------
// One block.  Threads stride the batch in chunks of blockDim rows; each computes its row's
// log-softmax and softmax serially (class counts are small), writes the scaled gradient and
// leaves -logp[target] in LDS; thread 0 adds every chunk's losses in batch order in fp64, as
// the reference's host loop does (ops/ops.c:5342-5352).
template <typename T>
__global__ void cross_entropy_kernel(T* loss, T* grad, const T* logits, const int* targets,
                                     int batch, int classes, T upstream, const T* upstream_dev) {
    __shared__ double nll[kThreads];
    double total = 0.0;
    if (upstream_dev) upstream *= upstream_dev[0];           // the upstream gradient where it lives: no host round trip
    for (int b0 = 0; b0 < batch; b0 += blockDim.x) {
        int b = b0 + threadIdx.x;
        if (b < batch) {
            const T* row = logits + (size_t)b * classes;
            T mx = lowest<T>();
            for (int c = 0; c < classes; c++) mx = row[c] > mx ? row[c] : mx;
            T sum = 0;
            for (int c = 0; c < classes; c++) sum += rp_exp(row[c] - mx);
            T lse = rp_log(sum);
            int t = targets[b];
            bool valid = (t >= 0 && t < classes);      // callers validate; a bad index poisons the loss instead of reading out of bounds
            nll[threadIdx.x] = valid ? -(double)(row[t] - mx - lse) : (double)NAN;
            if (grad) {
                T sc = (T)1 / (T)batch;
                for (int c = 0; c < classes; c++) {
                    T p = rp_exp(row[c] - mx) / sum;
                    if (c == t) p -= (T)1;
                    p *= sc;
                    grad[(size_t)b * classes + c] = p * upstream;
                }
            }
        }
        if (!loss) continue;                           // gradient only: nobody needs the sum (uniform: no thread reaches the barriers)
        __syncthreads();
        if (threadIdx.x == 0) {
            const int lim = batch - b0 < (int)blockDim.x ? batch - b0 : (int)blockDim.x;
            int i = 0;
            for (; i + 16 <= lim; i += 16) {             // sixteen LDS reads in flight, the adds still one by one in batch order
                double v[16];
#pragma unroll
                for (int u = 0; u < 16; u++) v[u] = nll[i + u];
#pragma unroll
                for (int u = 0; u < 16; u++) total += v[u];
            }
            for (; i < lim; i++) total += nll[i];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0 && loss) {
        if (sizeof(T) == 8) loss[0] = (T)(total / (double)batch);
        else { float f = (float)total; f /= (float)batch; loss[0] = (T)f; }
    }
}

// The same with every reduction (0 none, 1 mean, 2 sum: reference ops/ops.h:109-111) and on probabilities as well as on
// logits (reference ops/ops.c:5545-5643, 5412-5543).  loss: batch elements for 'none', one otherwise.  upstream_dev: the
// gradient of the loss on the device, batch elements for 'none', one otherwise (grad only).
template <typename T>
__global__ void cross_entropy_any_kernel(T* loss, T* grad, const T* x, const int* targets, int batch, int classes,
                                         int reduction, int from_logits, const T* upstream_dev) {
    __shared__ double nll[kThreads];
    double total = 0.0;
    for (int b0 = 0; b0 < batch; b0 += blockDim.x) {
        int b = b0 + threadIdx.x;
        if (b < batch) {
            const T* row = x + (size_t)b * classes;
            int t = targets[b];
            bool valid = (t >= 0 && t < classes);      // callers validate; a bad index poisons the loss instead of reading out of bounds
            T mx = 0, sum = 1, logp = 0;
            if (from_logits) {
                mx = lowest<T>();
                for (int c = 0; c < classes; c++) mx = row[c] > mx ? row[c] : mx;
                sum = 0;
                for (int c = 0; c < classes; c++) sum += rp_exp(row[c] - mx);
                if (valid) logp = row[t] - mx - rp_log(sum);
            } else if (valid) {
                logp = rp_log(row[t]);
            }
            nll[threadIdx.x] = valid ? -(double)logp : (double)NAN;
            if (loss && reduction == 0) loss[b] = valid ? -logp : (T)NAN;
            if (grad) {
                const T up = upstream_dev[reduction == 0 ? b : 0];
                const T sc = (T)1 / (T)batch;
                for (int c = 0; c < classes; c++) {
                    T g;
                    if (from_logits) { g = rp_exp(row[c] - mx) / sum; if (c == t) g -= (T)1; }
                    else g = (c == t) ? (T)-1 / row[c] : (T)0;
                    if (reduction == 1) g *= sc;
                    grad[(size_t)b * classes + c] = g * up;
                }
            }
        }
        if (!loss || reduction == 0) continue;         // uniform: no thread reaches the barriers
        __syncthreads();
        if (threadIdx.x == 0) {
            const int lim = batch - b0 < (int)blockDim.x ? batch - b0 : (int)blockDim.x;
            int i = 0;
            for (; i + 16 <= lim; i += 16) {             // sixteen LDS reads in flight, the adds one by one in batch order, in double (reference ops/ops.c:5342-5352)
                double v[16];
#pragma unroll
                for (int u = 0; u < 16; u++) v[u] = nll[i + u];
#pragma unroll
                for (int u = 0; u < 16; u++) total += v[u];
            }
            for (; i < lim; i++) total += nll[i];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0 && loss && reduction != 0) {
        if (sizeof(T) == 8) loss[0] = (T)(reduction == 1 ? total / (double)batch : total);
        else { float f = (float)total; if (reduction == 1) f /= (float)batch; loss[0] = (T)f; }
    }
}

}  // namespace rp

using namespace rp;

#define RP_REQUIRE(cond, name)                                              \
    do { if (!(cond)) { set_error("%s: invalid argument", name); return -1; } } while (0)

// Host-side narrowing of a fill value with the same bit rules as the device.
template <typename T> static T host_narrow(double value);
template <> double host_narrow<double>(double value) { return value; }
template <> float host_narrow<float>(double value) { return (float)value; }
template <> bf16_t host_narrow<bf16_t>(double value) {
    float f = (float)value;
    uint32_t w;
    __builtin_memcpy(&w, &f, 4);
    bf16_t r;
    r.bits = (uint16_t)((w >> 16) + ((w >> 15) & 1u));
    return r;
}
template <> f16_t host_narrow<f16_t>(double value) {
    float f = (float)value;
    uint32_t w;
    __builtin_memcpy(&w, &f, 4);
    uint32_t s = (w >> 16) & 0x8000u, e32 = (w >> 23) & 0xFFu, f23 = w & 0x7FFFFFu;
    int e = (int)e32 - 112;
    f16_t r;
    if (e32 == 0xFFu) r.bits = (uint16_t)(f23 ? (s | 0x7C00u | (f23 >> 13) | 1u) : (s | 0x7C00u));
    else if (e <= 0) {
        if (e < -10) r.bits = (uint16_t)s;
        else { f23 |= 0x800000u; int sh = 14 - e; r.bits = (uint16_t)((s | (f23 >> sh)) + ((f23 >> (sh - 1)) & 1u)); }
    } else if (e >= 0x1F) r.bits = (uint16_t)(s | 0x7C00u);
    else r.bits = (uint16_t)((s | ((uint32_t)e << 10) | (f23 >> 13)) + ((f23 >> 12) & 1u));
    return r;
}

template <typename D>
static int convert_from(void* dst, const void* src, int src_dtype, size_t size) {
    // every group of elements is at least 16 bytes on either side, so 16-byte aligned bases keep every group aligned
    const int vectors = (((uintptr_t)dst | (uintptr_t)src) & 15) == 0 ? 1 : 0;
    unsigned blocks = grid_for(vectors ? size / 2 + 1 : size);
    switch (src_dtype) {
        case RP_DTYPE_FLOAT32:  hipLaunchKernelGGL((convert_kernel<D, float>), dim3(blocks), dim3(kThreads), 0, current_stream(), (D*)dst, (const float*)src, size, vectors); break;
        case RP_DTYPE_FLOAT64:  hipLaunchKernelGGL((convert_kernel<D, double>), dim3(blocks), dim3(kThreads), 0, current_stream(), (D*)dst, (const double*)src, size, vectors); break;
        case RP_DTYPE_FLOAT16:  hipLaunchKernelGGL((convert_kernel<D, f16_t>), dim3(blocks), dim3(kThreads), 0, current_stream(), (D*)dst, (const f16_t*)src, size, vectors); break;
        case RP_DTYPE_BFLOAT16: hipLaunchKernelGGL((convert_kernel<D, bf16_t>), dim3(blocks), dim3(kThreads), 0, current_stream(), (D*)dst, (const bf16_t*)src, size, vectors); break;
        default: set_error("rp_hip_convert: unsupported source dtype %d", src_dtype); return -1;
    }
    return check_launch("convert_kernel") ? 0 : -1;
}

// ---- a scalar multiply whose launch is postponed -----------------------------------
// rp_hip_mul_scalar_deferred records the multiply instead of launching it.  Everything the calling thread does next in
// this library passes flush_deferred() first (current_stream() calls it, so does every entry point that touches the
// device without asking for the stream), which launches the recorded kernel: later work sees the product exactly as if
// it had been launched at once.  The one exception is a caller that knows the product will never be read and takes the
// record back with rp_hip_take_deferred, to hand source and scalar to rp_hip_scaled_softmax: the product is then
// never written.  One record per thread; recording a second multiply launches the first.
namespace rp {

struct DeferredScale { bool active; void* out; const void* x; double sd; float sf; size_t size; int dtype; };
static thread_local DeferredScale g_deferred = {false, nullptr, nullptr, 0.0, 0.f, 0, 0};

void flush_deferred() {
    if (!g_deferred.active) return;
    const DeferredScale d = g_deferred;
    g_deferred.active = false;                          // (the launch below asks for the stream again)
    const void* scalar = d.dtype == RP_DTYPE_FLOAT64 ? (const void*)&d.sd : (const void*)&d.sf;
    (void)mul_scalar_kernel_device(d.out, d.x, scalar, d.size, d.dtype);
}

bool deferred_touches(const void* ptr) { return g_deferred.active && (ptr == g_deferred.out || ptr == g_deferred.x); }

}  // namespace rp

extern "C" {

int add_kernel_device(void* out, const void* x1, const void* x2, size_t size, int dtype) {
    RP_REQUIRE(out && x1 && x2 && size, "add_kernel_device");
    RP_DISPATCH_DTYPE(dtype, launch_map<T, true>((T*)out, (const T*)x1, (const T*)x2, AddOp<typename traits<T>::acc>{}, size));
    return check_launch("add_kernel") ? 0 : -1;
}

int add_strided_kernel_device(void* out, const void* x1, const void* x2, int ndim, const int* out_shape,
                              const int* x1_strides, const int* x2_strides, size_t out_size, int dtype) {
    RP_REQUIRE(out && x1 && x2 && out_shape && x1_strides && x2_strides && out_size && ndim > 0, "add_strided_kernel_device");
    if (ndim > kMaxDims) { set_error("add_strided_kernel_device: more than %d dimensions", kMaxDims); return -1; }
    // [rows, cols] dense + row vector: the Linear bias add
    if (ndim == 2 && x1_strides[0] == out_shape[1] && x1_strides[1] == 1 && x2_strides[0] == 0 && x2_strides[1] == 1) {
        RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(add_row_vector_kernel<T>, dim3(grid_for(out_size)), dim3(kThreads), 0,
                                                   current_stream(), (T*)out, (const T*)x1, (const T*)x2, out_size, out_shape[1]));
        return check_launch("add_row_vector_kernel") ? 0 : -1;
    }
    StridedArgs a;
    a.ndim = ndim;
    for (int d = 0; d < ndim; d++) { a.shape[d] = out_shape[d]; a.s1[d] = x1_strides[d]; a.s2[d] = x2_strides[d]; }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(add_strided_kernel<T>, dim3(grid_for(out_size)), dim3(kThreads), 0, current_stream(),
                                               (T*)out, (const T*)x1, (const T*)x2, a, out_size));
    return check_launch("add_strided_kernel") ? 0 : -1;
}

int mul_scalar_kernel_device(void* out, const void* x, const void* scalar, size_t size, int dtype) {
    RP_REQUIRE(out && x && scalar && size, "mul_scalar_kernel_device");
    RP_DISPATCH_DTYPE(dtype, {
        using A = typename traits<T>::acc;
        A s = *(const A*)scalar;
        launch_map<T, false>((T*)out, (const T*)x, (const T*)nullptr, MulScalarOp<A>{s}, size);
    });
    return check_launch("mul_scalar_kernel") ? 0 : -1;
}

int relu_kernel_device(void* out, const void* x, size_t size, int dtype) {
    RP_REQUIRE(out && x && size, "relu_kernel_device");
    RP_DISPATCH_DTYPE(dtype, launch_map<T, false>((T*)out, (const T*)x, (const T*)nullptr, ReluOp<typename traits<T>::acc>{}, size));
    return check_launch("relu_kernel") ? 0 : -1;
}

int backwards_relu_device(const void* grad_c, const void* x, void* grad_x, size_t size, int dtype) {
    RP_REQUIRE(grad_c && x && grad_x && size, "backwards_relu_device");
    RP_DISPATCH_DTYPE(dtype, launch_map<T, true>((T*)grad_x, (const T*)grad_c, (const T*)x, BackReluOp<typename traits<T>::acc>{}, size));
    return check_launch("backwards_relu_kernel") ? 0 : -1;
}

static int softmax_any(void* out, const void* x, size_t outer, size_t dim, size_t inner, int dtype, bool take_log) {
    RP_REQUIRE(out && x && outer && dim && inner, "softmax_kernel_device");
    if (inner == 1) {
        unsigned blocks = grid_for(outer * 64, kThreads, 1u << 16);
        RP_DISPATCH_DTYPE(dtype, {
            if (launch_softmax_reg<T>((T*)out, (const T*)x, outer, dim, blocks, take_log)) {}
            else if (take_log) hipLaunchKernelGGL((softmax_rows_kernel<T, true>), dim3(blocks), dim3(kThreads), 0, current_stream(), (T*)out, (const T*)x, outer, dim);
            else          hipLaunchKernelGGL((softmax_rows_kernel<T, false>), dim3(blocks), dim3(kThreads), 0, current_stream(), (T*)out, (const T*)x, outer, dim);
        });
    } else {
        unsigned blocks = grid_for(outer * inner);
        RP_DISPATCH_DTYPE(dtype, {
            if (take_log) hipLaunchKernelGGL((softmax_strided_kernel<T, true>), dim3(blocks), dim3(kThreads), 0, current_stream(), (T*)out, (const T*)x, outer, dim, inner);
            else          hipLaunchKernelGGL((softmax_strided_kernel<T, false>), dim3(blocks), dim3(kThreads), 0, current_stream(), (T*)out, (const T*)x, outer, dim, inner);
        });
    }
    return check_launch("softmax kernel") ? 0 : -1;
}

int softmax_kernel_device(void* out, const void* x, size_t outer_size, size_t dim_size, size_t inner_size, int dtype) {
    return softmax_any(out, x, outer_size, dim_size, inner_size, dtype, false);
}

int log_softmax_kernel_device(void* out, const void* x, size_t outer_size, size_t dim_size, size_t inner_size, int dtype) {
    return softmax_any(out, x, outer_size, dim_size, inner_size, dtype, true);
}

int backwards_softmax_device(const void* grad_c, const void* softmax_out, void* grad_x,
                             size_t outer_size, size_t dim_size, size_t inner_size, int dtype) {
    RP_REQUIRE(grad_c && softmax_out && grad_x && outer_size && dim_size && inner_size, "backwards_softmax_device");
    if (inner_size == 1) {
        unsigned blocks = grid_for(outer_size * 64, kThreads, 1u << 16);
        RP_DISPATCH_DTYPE(dtype, {
            if (launch_bsoftmax_reg<T>((const T*)grad_c, (const T*)softmax_out, (T*)grad_x, outer_size, dim_size, blocks)) {}
            else hipLaunchKernelGGL(backwards_softmax_rows_kernel<T>, dim3(blocks), dim3(kThreads), 0, current_stream(),
                                    (const T*)grad_c, (const T*)softmax_out, (T*)grad_x, outer_size, dim_size);
        });
    } else {
        RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(backwards_softmax_strided_kernel<T>, dim3(grid_for(outer_size * inner_size)), dim3(kThreads), 0,
                                                   current_stream(), (const T*)grad_c, (const T*)softmax_out, (T*)grad_x,
                                                   outer_size, dim_size, inner_size));
    }
    return check_launch("backwards_softmax kernel") ? 0 : -1;
}

int rp_hip_mul_scalar_deferred(void* out, const void* x, const void* scalar, size_t size, int dtype) {
    RP_REQUIRE(out && x && scalar && size, "rp_hip_mul_scalar_deferred");
    if (!dtype_size(dtype)) { set_error("rp_hip_mul_scalar_deferred: unsupported dtype %d", dtype); return -1; }
    flush_deferred();
    g_deferred.out = out; g_deferred.x = x; g_deferred.size = size; g_deferred.dtype = dtype;
    if (dtype == RP_DTYPE_FLOAT64) { g_deferred.sd = *(const double*)scalar; g_deferred.sf = (float)g_deferred.sd; }
    else { g_deferred.sf = *(const float*)scalar; g_deferred.sd = (double)g_deferred.sf; }
    g_deferred.active = true;
    return 0;
}

int rp_hip_take_deferred(const void* out, const void** x, double* scalar) {
    if (!g_deferred.active || g_deferred.out != out) return 0;
    if (x) *x = g_deferred.x;
    if (scalar) *scalar = g_deferred.sd;
    g_deferred.active = false;
    return 1;
}

int rp_hip_scaled_softmax(void* out, const void* x, const void* scalar, size_t outer_size, size_t dim_size, size_t inner_size, int dtype) {
    RP_REQUIRE(out && x && scalar && outer_size && dim_size && inner_size, "rp_hip_scaled_softmax");
    if (inner_size == 1) {
        bool done = false;
        unsigned blocks = grid_for(outer_size * 64, kThreads, 1u << 16);
        RP_DISPATCH_DTYPE(dtype, {
            using A = typename traits<T>::acc;
            done = launch_softmax_reg<T>((T*)out, (const T*)x, outer_size, dim_size, blocks, false, true, *(const A*)scalar);
        });
        if (done) return check_launch("softmax kernel") ? 0 : -1;
    }
    // rows the one-pass kernel does not take: the two passes, the product going through `out`
    if (mul_scalar_kernel_device(out, x, scalar, outer_size * dim_size * inner_size, dtype) != 0) return -1;
    return softmax_kernel_device(out, out, outer_size, dim_size, inner_size, dtype);
}

int rp_hip_backwards_scaled_softmax(const void* grad_c, const void* softmax_out, void* grad_x, const void* scalar,
                                    size_t outer_size, size_t dim_size, size_t inner_size, int dtype) {
    RP_REQUIRE(grad_c && softmax_out && grad_x && scalar && outer_size && dim_size && inner_size, "rp_hip_backwards_scaled_softmax");
    if (inner_size == 1) {
        bool done = false;
        unsigned blocks = grid_for(outer_size * 64, kThreads, 1u << 16);
        RP_DISPATCH_DTYPE(dtype, {
            using A = typename traits<T>::acc;
            done = launch_bsoftmax_reg<T>((const T*)grad_c, (const T*)softmax_out, (T*)grad_x, outer_size, dim_size, blocks, true, *(const A*)scalar);
        });
        if (done) return check_launch("backwards_softmax kernel") ? 0 : -1;
    }
    if (backwards_softmax_device(grad_c, softmax_out, grad_x, outer_size, dim_size, inner_size, dtype) != 0) return -1;
    return mul_scalar_kernel_device(grad_x, grad_x, scalar, outer_size * dim_size * inner_size, dtype);
}

int backwards_log_softmax_device(const void* grad_c, const void* log_softmax_out, void* grad_x,
                                 size_t outer_size, size_t dim_size, size_t inner_size, int dtype) {
    RP_REQUIRE(grad_c && log_softmax_out && grad_x && outer_size && dim_size && inner_size, "backwards_log_softmax_device");
    if (inner_size == 1) {
        unsigned blocks = grid_for(outer_size * 64, kThreads, 1u << 16);       // a wave per row
        RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(backwards_log_softmax_rows_kernel<T>, dim3(blocks), dim3(kThreads), 0, current_stream(),
                                                    (const T*)grad_c, (const T*)log_softmax_out, (T*)grad_x, outer_size, dim_size));
    } else {
        RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(backwards_log_softmax_strided_kernel<T>, dim3(grid_for(outer_size * inner_size)), dim3(kThreads), 0,
                                                    current_stream(), (const T*)grad_c, (const T*)log_softmax_out, (T*)grad_x, outer_size, dim_size, inner_size));
    }
    return check_launch("backwards_log_softmax kernel") ? 0 : -1;
}

int contiguous_copy_kernel_device(void* out, const void* in, int ndim, int* shape, int* strides, size_t size, int dtype) {
    RP_REQUIRE(out && in && shape && strides && size && ndim > 0, "contiguous_copy_kernel_device");
    if (ndim > kMaxDims) { set_error("contiguous_copy_kernel_device: more than %d dimensions", kMaxDims); return -1; }
    GatherArgs a;
    a.ndim = ndim;
    for (int d = 0; d < ndim; d++) { a.shape[d] = shape[d]; a.strides[d] = strides[d]; }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(gather_kernel<T>, dim3(grid_for(size)), dim3(kThreads), 0, current_stream(),
                                               (T*)out, (const T*)in, a, size));
    return check_launch("gather_kernel") ? 0 : -1;
}

static int sum_all_any(void* out, const void* x, size_t size, int dtype, double scale) {
    RP_REQUIRE(out && x && size, "sum_all_kernel_device");
    unsigned blocks = grid_for(size, kThreads * 16, kMaxPartials);
    RP_DISPATCH_DTYPE(dtype, {
        hipLaunchKernelGGL(sum_partials_kernel<T>, dim3(blocks), dim3(kThreads), 0, current_stream(), (const T*)x, size);
        hipLaunchKernelGGL(sum_finish_kernel<T>, dim3(1), dim3(1), 0, current_stream(), (T*)out, (int)blocks, scale);
    });
    return check_launch("sum_all kernels") ? 0 : -1;
}

int sum_all_kernel_device(void* out, const void* x, size_t size, int dtype) { return sum_all_any(out, x, size, dtype, 1.0); }

int mean_all_kernel_device(void* out, const void* x, size_t size, int dtype) { return sum_all_any(out, x, size, dtype, (double)size); }

int sum_dim_kernel_device(void* out, const void* x, size_t outer_size, size_t dim_size, size_t inner_size, int dtype) {
    RP_REQUIRE(out && x && outer_size && dim_size && inner_size, "sum_dim_kernel_device");
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(sum_dim_kernel<T>, dim3(grid_for(outer_size * inner_size)), dim3(kThreads), 0, current_stream(),
                                               (T*)out, (const T*)x, outer_size, dim_size, inner_size));
    return check_launch("sum_dim_kernel") ? 0 : -1;
}

int rp_hip_fill(void* ptr, double value, size_t size, int dtype) {
    RP_REQUIRE(ptr && size, "rp_hip_fill");
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(fill_kernel<T>, dim3(grid_for(size * sizeof(T) / 16 + 16)), dim3(kThreads), 0, current_stream(),
                                               (T*)ptr, host_narrow<T>(value), size));
    return check_launch("fill_kernel") ? 0 : -1;
}

int rp_hip_convert(void* dst, int dst_dtype, const void* src, int src_dtype, size_t size) {
    RP_REQUIRE(dst && src && size, "rp_hip_convert");
    RP_DISPATCH_DTYPE(dst_dtype, return convert_from<T>(dst, src, src_dtype, size));
    return -1;
}

int rp_hip_reduce_rows(void* out, const void* grad, int rows, int cols, int accumulate, int dtype) {
    RP_REQUIRE(out && grad && rows > 0 && cols > 0, "rp_hip_reduce_rows");
    unsigned blocks = (unsigned)((cols + 63) / 64);
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(reduce_rows_kernel<T>, dim3(blocks), dim3(64), 0, current_stream(),
                                               (T*)out, (const T*)grad, rows, cols, accumulate));
    return check_launch("reduce_rows_kernel") ? 0 : -1;
}

int rp_hip_cross_entropy_mean(void* loss_out, void* grad_logits, const void* logits, const int* targets,
                              int batch, int classes, double upstream, int dtype) {
    RP_REQUIRE(logits && targets && batch > 0 && classes > 0 && (loss_out || grad_logits), "rp_hip_cross_entropy_mean");
    if (dtype != RP_DTYPE_FLOAT32 && dtype != RP_DTYPE_FLOAT64) {
        set_error("rp_hip_cross_entropy_mean: float32 and float64 only");
        return -1;
    }
    if (dtype == RP_DTYPE_FLOAT32)
        hipLaunchKernelGGL(cross_entropy_kernel<float>, dim3(1), dim3(kThreads), 0, current_stream(), (float*)loss_out, (float*)grad_logits,
                           (const float*)logits, targets, batch, classes, (float)upstream, (const float*)nullptr);
    else
        hipLaunchKernelGGL(cross_entropy_kernel<double>, dim3(1), dim3(kThreads), 0, current_stream(), (double*)loss_out, (double*)grad_logits,
                           (const double*)logits, targets, batch, classes, upstream, (const double*)nullptr);
    return check_launch("cross_entropy_kernel") ? 0 : -1;
}

int rp_hip_cross_entropy_backward(void* grad_logits, const void* logits, const int* targets, int batch, int classes,
                                  const void* upstream_dev, int dtype) {
    RP_REQUIRE(grad_logits && logits && targets && upstream_dev && batch > 0 && classes > 0, "rp_hip_cross_entropy_backward");
    if (dtype != RP_DTYPE_FLOAT32 && dtype != RP_DTYPE_FLOAT64) {
        set_error("rp_hip_cross_entropy_backward: float32 and float64 only");
        return -1;
    }
    if (dtype == RP_DTYPE_FLOAT32)
        hipLaunchKernelGGL(cross_entropy_kernel<float>, dim3(1), dim3(kThreads), 0, current_stream(), (float*)nullptr, (float*)grad_logits,
                           (const float*)logits, targets, batch, classes, 1.0f, (const float*)upstream_dev);
    else
        hipLaunchKernelGGL(cross_entropy_kernel<double>, dim3(1), dim3(kThreads), 0, current_stream(), (double*)nullptr, (double*)grad_logits,
                           (const double*)logits, targets, batch, classes, 1.0, (const double*)upstream_dev);
    return check_launch("cross_entropy_kernel") ? 0 : -1;
}

int rp_hip_cross_entropy_forward(void* loss_out, const void* x, const int* targets, int batch, int classes,
                                 int reduction, int from_logits, int dtype) {
    RP_REQUIRE(loss_out && x && targets && batch > 0 && classes > 0 && reduction >= 0 && reduction <= 2, "rp_hip_cross_entropy_forward");
    if (dtype != RP_DTYPE_FLOAT32 && dtype != RP_DTYPE_FLOAT64) { set_error("rp_hip_cross_entropy_forward: float32 and float64 only"); return -1; }
    if (dtype == RP_DTYPE_FLOAT32)
        hipLaunchKernelGGL(cross_entropy_any_kernel<float>, dim3(1), dim3(kThreads), 0, current_stream(), (float*)loss_out, (float*)nullptr,
                           (const float*)x, targets, batch, classes, reduction, from_logits ? 1 : 0, (const float*)nullptr);
    else
        hipLaunchKernelGGL(cross_entropy_any_kernel<double>, dim3(1), dim3(kThreads), 0, current_stream(), (double*)loss_out, (double*)nullptr,
                           (const double*)x, targets, batch, classes, reduction, from_logits ? 1 : 0, (const double*)nullptr);
    return check_launch("cross_entropy_any_kernel") ? 0 : -1;
}

int rp_hip_cross_entropy_grad(void* grad_x, const void* x, const int* targets, int batch, int classes,
                              int reduction, int from_logits, const void* upstream_dev, int dtype) {
    RP_REQUIRE(grad_x && x && targets && upstream_dev && batch > 0 && classes > 0 && reduction >= 0 && reduction <= 2, "rp_hip_cross_entropy_grad");
    if (dtype != RP_DTYPE_FLOAT32 && dtype != RP_DTYPE_FLOAT64) { set_error("rp_hip_cross_entropy_grad: float32 and float64 only"); return -1; }
    if (dtype == RP_DTYPE_FLOAT32)
        hipLaunchKernelGGL(cross_entropy_any_kernel<float>, dim3(1), dim3(kThreads), 0, current_stream(), (float*)nullptr, (float*)grad_x,
                           (const float*)x, targets, batch, classes, reduction, from_logits ? 1 : 0, (const float*)upstream_dev);
    else
        hipLaunchKernelGGL(cross_entropy_any_kernel<double>, dim3(1), dim3(kThreads), 0, current_stream(), (double*)nullptr, (double*)grad_x,
                           (const double*)x, targets, batch, classes, reduction, from_logits ? 1 : 0, (const double*)upstream_dev);
    return check_launch("cross_entropy_any_kernel") ? 0 : -1;
}

int rp_hip_fill_scaled(void* ptr, const void* scalar_dev, double scale, size_t size, int dtype) {
    RP_REQUIRE(ptr && scalar_dev && size, "rp_hip_fill_scaled");
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(fill_scaled_kernel<T>, dim3(grid_for(size * sizeof(T) / 16 + 16)), dim3(kThreads), 0, current_stream(),
                                               (T*)ptr, (const T*)scalar_dev, scale, size));
    return check_launch("fill_scaled_kernel") ? 0 : -1;
}

}  // extern "C"
