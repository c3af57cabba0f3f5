// conv2d as a caller of the strided-batched GEMM: the lowering kernels either side of it.
//
//   forward   col[n] = im2col(x[n])                 [C_in*kH*kW, oH*oW]   one launch for the whole batch
//             y[n]   = W[C_out, C_in*kH*kW] . col[n]                      one batched GEMM, W shared (batch stride 0)
//             y[n, c] += bias[c]                                          channel_bias_add
//   backward  dcol[n] = W^T . dy[n]                                       one batched GEMM, W^T a stride view
//             dx[n]   = col2im(dcol[n])                                   gather: one thread per input pixel, no atomics
//             dW      = sum_n dy[n] . col[n]^T                            one batched GEMM + a sum over the batch
//             db[c]   = sum_{n, hw} dy[n, c, hw]                          channel_sums
//
// The reference lowers one sample at a time (ops/ops.c:4759-4770 forward, 4533-4551 and 4575-4617 backward) with the
// kernels of functional/functional_device.cu:1664-1721; its col2im scatters with atomicAdd, so for 16-bit types the
// sum is rounded after every add in an order that changes from run to run.  Here col2im gathers: each input pixel adds
// its (kh, kw) contributions in ascending order in the accumulate type and rounds once, which is what the reference's
// host path computes (functional/functional.c:885-912, functional_host.c:1291-1313) and is repeatable.
#include "rp_common.h"

namespace rp {

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

struct ConvGeom {
    int N, C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW;
};

// VEC neighbouring elements row[start .. start + VEC) of a row of `len` >= VEC elements, zeros where the span sticks
// out of the row: one vector load from the nearest start that keeps the load inside the row, shifted into place as
// a 128-bit value.  No lane takes a different path, so a wave that holds interior and border spans runs this once.
template <typename T, int VEC>
__device__ __forceinline__ void load_span(T (&v)[VEC], const T* row, int start, int len) {
    static_assert(VEC * sizeof(T) == 16, "one 16-byte vector");
    constexpr int EB = 8 * (int)sizeof(T);
    const int s = start < 0 ? 0 : (start > len - VEC ? len - VEC : start);
    int shift = start - s;                                  // elements; beyond +-(VEC - 1) nothing of the span is inside
    shift = shift > VEC - 1 ? VEC - 1 : (shift < -(VEC - 1) ? -(VEC - 1) : shift);
    unsigned __int128 bits;
    memcpy(&bits, row + s, 16);
    bits = shift >= 0 ? bits >> (shift * EB) : bits << (-shift * EB);
    memcpy(v, &bits, 16);
#pragma unroll
    for (int e = 0; e < VEC; e++)
        if (start + e < 0 || start + e >= len) memset(&v[e], 0, sizeof(T));
}

// One thread owns VEC consecutive columns (output positions) of one (n, c) plane and writes them into every tap's
// col row (VEC = 1 when rows are not whole vectors).  With unit stride along w the VEC inputs of one tap are
// neighbours in memory and come in with a single (unaligned) vector load, borders included (load_span); spans that
// wrap to the next output row, and other strides, go one by one.  The taps' loads overlap almost entirely and hit
// in the vector cache; the stores of a wave are whole kilobytes of one col row.
// TAPS3: the kernel is 3 x 3 (the tap loops unroll, so that all nine loads of a thread are in flight together).
template <typename T, int VEC, bool TAPS3>
__global__ void __launch_bounds__(256) im2col_kernel(T* col, const T* im, ConvGeom g, unsigned total_vec) {
    const int cols = g.oH * g.oW;
    const unsigned vec_per_row = cols / VEC;
    const unsigned gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= total_vec) return;
    const unsigned plane_id = gid / vec_per_row, pv = gid % vec_per_row;
    const T* plane = im + (size_t)plane_id * g.H * g.W;
    T* dst = col + ((size_t)plane_id * (g.kH * g.kW)) * cols + (size_t)pv * VEC;
    const int p = pv * VEC;
    const int oh0 = p / g.oW, ow0 = p % g.oW;
    const bool span = VEC > 1 && g.sw == 1 && ow0 + VEC <= g.oW && g.W >= VEC;
    auto tap = [&](int kh, int kw, T* dst) {
            T v[VEC];
            if constexpr (VEC > 1) {
                if (span) {
                    const int h0 = oh0 * g.sh + kh * g.dh - g.ph, w0 = ow0 + kw * g.dw - g.pw;
                    const bool row_inside = h0 >= 0 && h0 < g.H;
                    load_span<T, VEC>(v, plane + (size_t)(row_inside ? h0 : 0) * g.W, row_inside ? w0 : -VEC, g.W);
                }
            }
            if (!span) {
                int oh = oh0, ow = ow0;
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    const int h_in = oh * g.sh + kh * g.dh - g.ph, w_in = ow * g.sw + kw * g.dw - g.pw;
                    T x;
                    if (h_in >= 0 && h_in < g.H && w_in >= 0 && w_in < g.W) x = plane[(size_t)h_in * g.W + w_in];
                    else memset(&x, 0, sizeof(T));
                    v[e] = x;
                    if (++ow == g.oW) { ow = 0; oh++; }
                }
            }
            if (VEC * sizeof(T) == 16) {
                u32x4_t w;
                memcpy(&w, v, 16);
                __builtin_nontemporal_store(w, (u32x4_t*)dst);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; e++) dst[e] = v[e];
            }
    };
    if constexpr (TAPS3) {
#pragma unroll
        for (int t = 0; t < 9; t++) tap(t / 3, t % 3, dst + (size_t)t * cols);
    } else {
        for (int kh = 0; kh < g.kH; kh++)
            for (int kw = 0; kw < g.kW; kw++, dst += cols) tap(kh, kw, dst);
    }
}

// One thread per VEC neighbouring input pixels of a row (VEC = 1 when W is not a whole number of vectors).
// START_FROM_IM: the sums start from the pixels' current values (the reference's "im += ..." contract); otherwise from
// zero and the pixels are overwritten.  Every pixel adds its taps in ascending (kh, kw) order; with unit stride
// along w the VEC values of one tap are neighbours in the col row and come in with one vector load.
template <typename T, int VEC, bool START_FROM_IM>
__global__ void __launch_bounds__(256) col2im_gather_kernel(T* im, const T* col, ConvGeom g, unsigned total_vec) {
    using A = typename traits<T>::acc;
    const int cols = g.oH * g.oW;
    const unsigned vec_per_plane = g.H * g.W / VEC;
    const unsigned gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= total_vec) return;
    const unsigned t = gid / vec_per_plane;                 // n * C + c
    const int pix = (int)(gid % vec_per_plane) * VEC;
    const int h = pix / g.W, w0 = pix % g.W;
    {
        const size_t idx = gid;
        const T* rows = col + t * (size_t)g.kH * g.kW * cols;
        T* dst = im + idx * VEC;
        A acc[VEC];
        if (START_FROM_IM) {
            T cur[VEC];
            memcpy(cur, dst, VEC * sizeof(T));
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] = widen(cur[e]);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; e++) acc[e] = (A)0;
        }
        for (int kh = 0; kh < g.kH; kh++) {
            const int hh = h + g.ph - kh * g.dh;
            if (hh < 0 || hh % g.sh) continue;
            const int oh = hh / g.sh;
            if (oh >= g.oH) continue;
            for (int kw = 0; kw < g.kW; kw++) {
                const T* row = rows + (size_t)(kh * g.kW + kw) * cols + (size_t)oh * g.oW;
                const int ww0 = w0 + g.pw - kw * g.dw;
                bool done = false;
                if constexpr (VEC > 1) {
                    if (g.sw == 1 && g.oW >= VEC) {
                        T x[VEC];
                        load_span<T, VEC>(x, row, ww0, g.oW);
#pragma unroll
                        for (int e = 0; e < VEC; e++) acc[e] += widen(x[e]);
                        done = true;
                    }
                }
                if (!done) {
#pragma unroll
                    for (int e = 0; e < VEC; e++) {
                        const int ww = ww0 + e;
                        if (ww < 0 || ww % g.sw) continue;
                        const int ow = ww / g.sw;
                        if (ow < g.oW) acc[e] += widen(row[ow]);
                    }
                }
            }
        }
        T out[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) out[e] = narrow<T>(acc[e]);
        memcpy(dst, out, VEC * sizeof(T));
    }
}

// y[n, c, :] += bias[c]: one rounding add per element, as the reference's loop does (ops/ops.c:4776-4783).
// VEC elements per thread when a channel's plane is a whole number of vectors (they then share one bias value).
template <typename T, int VEC>
__global__ void __launch_bounds__(256) channel_bias_add_kernel(T* y, const T* bias, int channels, int hw, size_t total_vec) {
    const int vec_per_plane = hw / VEC;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total_vec; idx += (size_t)gridDim.x * 256) {
        const int c = (int)((idx / vec_per_plane) % channels);
        const auto b = widen(bias[c]);
        T v[VEC];
        memcpy(v, y + idx * VEC, VEC * sizeof(T));
#pragma unroll
        for (int e = 0; e < VEC; e++) v[e] = narrow<T>(widen(v[e]) + b);
        memcpy(y + idx * VEC, v, VEC * sizeof(T));
    }
}

// db[c] = sum over n and hw of g[n, c, hw], in the accumulate type (fp32 for 16-bit and fp32 tensors, as the
// reference's host loop, ops/ops.c:4634-4650; fp64 for fp64).  Two steps, so that the whole chip reads: one block per
// (n, c) plane leaves the plane's sum in partial[n, c]; then one thread per channel adds its partials in batch order.
template <typename T>
__global__ void __launch_bounds__(256) plane_sums_kernel(typename traits<T>::acc* partial, const T* g, int hw) {
    using A = typename traits<T>::acc;
    constexpr int VEC = 16 / (int)sizeof(T);
    __shared__ A part[256];
    const T* p = g + (size_t)blockIdx.x * hw;
    A s = 0;
    const int lead = (int)(((16 - ((uintptr_t)p & 15)) & 15) / sizeof(T));      // elements before the first 16-byte boundary
    const int head = lead < hw ? lead : hw;
    const int nvec = (hw - head) / VEC;
    if ((int)threadIdx.x < head) s += widen(p[threadIdx.x]);
    for (int i = threadIdx.x; i < nvec; i += 256) {
        T v[VEC];
        const u32x4_t raw = __builtin_nontemporal_load((const u32x4_t*)(p + head) + i);
        memcpy(v, &raw, 16);
#pragma unroll
        for (int e = 0; e < VEC; e++) s += widen(v[e]);
    }
    for (int i = head + nvec * VEC + threadIdx.x; i < hw; i += 256) s += widen(p[i]);
    part[threadIdx.x] = s;
    __syncthreads();
    for (int half = 128; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) part[threadIdx.x] += part[threadIdx.x + half];
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[blockIdx.x] = part[0];
}

template <typename T>
__global__ void channel_sums_finish_kernel(T* out, const typename traits<T>::acc* partial, int batch, int channels, int accumulate) {
    using A = typename traits<T>::acc;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    A s = 0;
    int n = 0;
    constexpr int U = 16;                       // independent loads in flight; the adds stay in batch order
    for (; n + U <= batch; n += U) {
        A v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = partial[(size_t)(n + u) * channels + c];
#pragma unroll
        for (int u = 0; u < U; u++) s += v[u];
    }
    for (; n < batch; n++) s += partial[(size_t)n * channels + c];
    T r = narrow<T>(s);
    if (accumulate) r = narrow<T>(widen(out[c]) + widen(r));
    out[c] = r;
}

static bool geom_ok(const ConvGeom& g) {
    if (g.N <= 0 || g.C <= 0 || g.H <= 0 || g.W <= 0 || g.kH <= 0 || g.kW <= 0 || g.sh <= 0 || g.sw <= 0 || g.ph < 0 || g.pw < 0 ||
        g.dh <= 0 || g.dw <= 0 || g.oH <= 0 || g.oW <= 0) return false;
    // the output extent must be the one the geometry implies, or the gathers would leave the image
    const long long eh = ((long long)g.H + 2 * g.ph - (long long)g.dh * (g.kH - 1) - 1) / g.sh + 1;
    const long long ew = ((long long)g.W + 2 * g.pw - (long long)g.dw * (g.kW - 1) - 1) / g.sw + 1;
    if (g.oH != eh || g.oW != ew) return false;
    return (long long)g.C * g.kH * g.kW * (long long)g.oH * g.oW < (1ll << 31) && (long long)g.H * g.W < (1ll << 31) &&
           (long long)g.N * g.C < (1ll << 31) && (long long)g.H * g.W < (1ll << 30) && (long long)g.oH * g.oW < (1ll << 30);
}

static unsigned conv_grid(size_t work) {
    size_t b = (work + 255) / 256;
    return (unsigned)(b < 1 ? 1 : (b > (1u << 20) ? (1u << 20) : b));
}

// the lowering kernels index their threads with 32 bits: a launch covers at most this many vectors, larger
// batches go plane range by plane range
constexpr unsigned kMaxVecPerLaunch = 1u << 30;

template <typename T>
static void launch_im2col(void* col, const void* im, const ConvGeom& g) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int cols = g.oH * g.oW, planes = g.N * g.C;
    const bool vec = cols % VEC == 0 && ((uintptr_t)col & 15) == 0;
    const unsigned per_plane = vec ? cols / VEC : cols;
    const int planes_per_launch = (int)(kMaxVecPerLaunch / per_plane) > 0 ? (int)(kMaxVecPerLaunch / per_plane) : 1;
    const size_t esz = sizeof(T);
    for (int p0 = 0; p0 < planes; p0 += planes_per_launch) {
        const int np = planes - p0 < planes_per_launch ? planes - p0 : planes_per_launch;
        const unsigned total = (unsigned)np * per_plane;
        T* c0 = (T*)((char*)col + (size_t)p0 * g.kH * g.kW * cols * esz);
        const T* i0 = (const T*)((const char*)im + (size_t)p0 * g.H * g.W * esz);
        const dim3 grid((total + 255) / 256);
        if (vec && g.kH == 3 && g.kW == 3) hipLaunchKernelGGL((im2col_kernel<T, VEC, true>), grid, dim3(256), 0, current_stream(), c0, i0, g, total);
        else if (vec) hipLaunchKernelGGL((im2col_kernel<T, VEC, false>), grid, dim3(256), 0, current_stream(), c0, i0, g, total);
        else hipLaunchKernelGGL((im2col_kernel<T, 1, false>), grid, dim3(256), 0, current_stream(), c0, i0, g, total);
    }
}

template <typename T>
static void launch_col2im(void* im, const void* col, const ConvGeom& g, bool start_from_im) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int cols = g.oH * g.oW, planes = g.N * g.C;
    const bool vec = g.W % VEC == 0 && ((uintptr_t)im & 15) == 0;
    const unsigned per_plane = vec ? g.H * g.W / VEC : g.H * g.W;
    const int planes_per_launch = (int)(kMaxVecPerLaunch / per_plane) > 0 ? (int)(kMaxVecPerLaunch / per_plane) : 1;
    const size_t esz = sizeof(T);
    for (int p0 = 0; p0 < planes; p0 += planes_per_launch) {
        const int np = planes - p0 < planes_per_launch ? planes - p0 : planes_per_launch;
        const unsigned total = (unsigned)np * per_plane;
        const dim3 grid((total + 255) / 256);
        const T* c0 = (const T*)((const char*)col + (size_t)p0 * g.kH * g.kW * cols * esz);
        T* i0 = (T*)((char*)im + (size_t)p0 * g.H * g.W * esz);
        if (vec) {
            if (start_from_im) hipLaunchKernelGGL((col2im_gather_kernel<T, VEC, true>), grid, dim3(256), 0, current_stream(), i0, c0, g, total);
            else hipLaunchKernelGGL((col2im_gather_kernel<T, VEC, false>), grid, dim3(256), 0, current_stream(), i0, c0, g, total);
        } else {
            if (start_from_im) hipLaunchKernelGGL((col2im_gather_kernel<T, 1, true>), grid, dim3(256), 0, current_stream(), i0, c0, g, total);
            else hipLaunchKernelGGL((col2im_gather_kernel<T, 1, false>), grid, dim3(256), 0, current_stream(), i0, c0, g, total);
        }
    }
}

template <typename T>
static void launch_bias_add(void* y, const void* bias, int batch, int channels, int hw) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const size_t total = (size_t)batch * channels * hw;
    if (hw % VEC == 0 && ((uintptr_t)y & 15) == 0)
        hipLaunchKernelGGL((channel_bias_add_kernel<T, VEC>), dim3(conv_grid(total / VEC)), dim3(256), 0, current_stream(), (T*)y, (const T*)bias, channels, hw, total / VEC);
    else
        hipLaunchKernelGGL((channel_bias_add_kernel<T, 1>), dim3(conv_grid(total)), dim3(256), 0, current_stream(), (T*)y, (const T*)bias, channels, hw, total);
}

template <typename T>
static void launch_channel_sums(void* out, const void* grad, void* partial, int batch, int channels, int hw, int accumulate) {
    using A = typename traits<T>::acc;
    hipLaunchKernelGGL(plane_sums_kernel<T>, dim3((unsigned)(batch * channels)), dim3(256), 0, current_stream(), (A*)partial, (const T*)grad, hw);
    hipLaunchKernelGGL(channel_sums_finish_kernel<T>, dim3((channels + 63) / 64), dim3(64), 0, current_stream(), (T*)out, (const A*)partial, batch, channels, accumulate);
}

}  // namespace rp

using namespace rp;

extern "C" {

int rp_hip_im2col_batched(void* col, const void* im, int batch, int C_in, int H, int W, int kH, int kW,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w,
                          int out_H, int out_W, int dtype) {
    ConvGeom g{batch, C_in, H, W, kH, kW, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, out_H, out_W};
    if (!col || !im || !geom_ok(g)) { set_error("rp_hip_im2col_batched: null operand or inconsistent geometry"); return -1; }
    RP_DISPATCH_DTYPE(dtype, launch_im2col<T>(col, im, g));
    return check_launch("im2col_kernel") ? 0 : -1;
}

int rp_hip_col2im_batched(void* im, const void* col, int batch, int C_in, int H, int W, int kH, int kW,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w,
                          int out_H, int out_W, int accumulate, int dtype) {
    ConvGeom g{batch, C_in, H, W, kH, kW, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, out_H, out_W};
    if (!col || !im || !geom_ok(g)) { set_error("rp_hip_col2im_batched: null operand or inconsistent geometry"); return -1; }
    RP_DISPATCH_DTYPE(dtype, launch_col2im<T>(im, col, g, accumulate != 0));
    return check_launch("col2im_gather_kernel") ? 0 : -1;
}

int im2col_kernel_device(void* col, const void* im, int C_in, int H, int W, int kH, int kW, int stride_h, int stride_w,
                         int pad_h, int pad_w, int dilation_h, int dilation_w, int out_H, int out_W, int dtype) {
    return rp_hip_im2col_batched(col, im, 1, C_in, H, W, kH, kW, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, out_H, out_W, dtype);
}

int col2im_kernel_device(void* im, const void* col, int C_in, int H, int W, int kH, int kW, int stride_h, int stride_w,
                         int pad_h, int pad_w, int dilation_h, int dilation_w, int out_H, int out_W, int dtype) {
    return rp_hip_col2im_batched(im, col, 1, C_in, H, W, kH, kW, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, out_H, out_W, 1, dtype);
}

int rp_hip_channel_bias_add(void* y, const void* bias, int batch, int channels, int hw, int dtype) {
    if (!y || !bias || batch <= 0 || channels <= 0 || hw <= 0) { set_error("rp_hip_channel_bias_add: null operand or non-positive extent"); return -1; }
    RP_DISPATCH_DTYPE(dtype, launch_bias_add<T>(y, bias, batch, channels, hw));
    return check_launch("channel_bias_add_kernel") ? 0 : -1;
}

int rp_hip_channel_sums(void* out, const void* grad, int batch, int channels, int hw, int accumulate, int dtype) {
    if (!out || !grad || batch <= 0 || channels <= 0 || hw <= 0 || (long long)batch * channels >= (1ll << 31)) {
        set_error("rp_hip_channel_sums: null operand or extent out of range");
        return -1;
    }
    if (!dtype_size(dtype)) { set_error("rp_hip_channel_sums: unsupported dtype %d", dtype); return -1; }
    void* partial = nullptr;                 // one accumulate-type value per (n, c) plane, from the stream-ordered pool
    if (rp_hip_malloc(&partial, (size_t)batch * channels * 8) != 0) return -1;
    RP_DISPATCH_DTYPE(dtype, launch_channel_sums<T>(out, grad, partial, batch, channels, hw, accumulate));
    const bool ok = check_launch("channel_sums kernels");
    rp_hip_free(partial);
    return ok ? 0 : -1;
}

}  // extern "C"
