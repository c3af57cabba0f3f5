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

// One thread writes VEC consecutive columns of one col row (VEC = 1 when rows are not whole vectors).
template <typename T, int VEC>
__global__ void __launch_bounds__(256) im2col_kernel(T* col, const T* im, ConvGeom g, size_t total_vec) {
    const int cols = g.oH * g.oW;
    const int vec_per_row = cols / VEC;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total_vec; idx += (size_t)gridDim.x * 256) {
        const int pv = (int)(idx % vec_per_row);
        size_t t = idx / vec_per_row;
        const int kw = (int)(t % g.kW); t /= g.kW;
        const int kh = (int)(t % g.kH); t /= g.kH;
        const int c = (int)(t % g.C);
        const size_t n = t / g.C;
        const T* plane = im + (n * g.C + c) * (size_t)g.H * g.W;
        int p = pv * VEC;
        int oh = p / g.oW, ow = p % g.oW;
        T v[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const int h_in = oh * g.sh + kh * g.dh - g.ph, w_in = ow * g.sw + kw * g.dw - g.pw;
            T x;
            if (h_in >= 0 && h_in < g.H && w_in >= 0 && w_in < g.W) x = plane[(size_t)h_in * g.W + w_in];
            else memset(&x, 0, sizeof(T));
            v[e] = x;
            if (++ow == g.oW) { ow = 0; oh++; }
        }
        // idx enumerates (n, c, kh, kw, pv) in the order the rows lie in memory
        T* dst = col + idx * VEC;
        if (VEC * sizeof(T) == 16) {
            u32x4_t w;
            memcpy(&w, v, 16);
            __builtin_nontemporal_store(w, (u32x4_t*)dst);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; e++) dst[e] = v[e];
        }
    }
}

// One thread per input pixel.  START_FROM_IM: the sum starts from the pixel's current value (the reference's
// "im += ..." contract); otherwise from zero and the pixel is overwritten.
template <typename T, bool START_FROM_IM>
__global__ void __launch_bounds__(256) col2im_gather_kernel(T* im, const T* col, ConvGeom g, size_t total) {
    using A = typename traits<T>::acc;
    const int cols = g.oH * g.oW;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
        const int w = (int)(idx % g.W);
        size_t t = idx / g.W;
        const int h = (int)(t % g.H); t /= g.H;          // t = n * C + c
        const T* rows = col + t * (size_t)g.kH * g.kW * cols;
        A acc = START_FROM_IM ? widen(im[idx]) : (A)0;
        for (int kh = 0; kh < g.kH; kh++) {
            const int hh = h + g.ph - kh * g.dh;
            if (hh < 0 || hh % g.sh) continue;
            const int oh = hh / g.sh;
            if (oh >= g.oH) continue;
            for (int kw = 0; kw < g.kW; kw++) {
                const int ww = w + g.pw - kw * g.dw;
                if (ww < 0 || ww % g.sw) continue;
                const int ow = ww / g.sw;
                if (ow >= g.oW) continue;
                acc += widen(rows[(size_t)(kh * g.kW + kw) * cols + oh * g.oW + ow]);
            }
        }
        im[idx] = narrow<T>(acc);
    }
}

// y[n, c, :] += bias[c]: one rounding add per element, as the reference's loop does (ops/ops.c:4776-4783).
template <typename T>
__global__ void __launch_bounds__(256) channel_bias_add_kernel(T* y, const T* bias, int channels, int hw, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
        const int c = (int)((idx / hw) % channels);
        y[idx] = narrow<T>(widen(y[idx]) + widen(bias[c]));
    }
}

// db[c] = sum over n and hw of g[n, c, hw].  One block per channel; every thread adds a strided share in the
// accumulate type (fp32 for 16-bit and fp32 tensors, as the reference's host loop does, ops/ops.c:4634-4650;
// fp64 for fp64), the block combines the shares through LDS.
template <typename T>
__global__ void __launch_bounds__(256) channel_sums_kernel(T* out, const T* g, int batch, int channels, int hw, int accumulate) {
    using A = typename traits<T>::acc;
    __shared__ A part[256];
    const int c = blockIdx.x;
    A s = 0;
    for (int n = 0; n < batch; n++) {
        const T* p = g + ((size_t)n * channels + c) * hw;
        for (int i = threadIdx.x; i < hw; i += 256) s += widen(p[i]);
    }
    part[threadIdx.x] = s;
    __syncthreads();
    for (int half = 128; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) part[threadIdx.x] += part[threadIdx.x + half];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        T r = narrow<T>(part[0]);
        if (accumulate) r = narrow<T>(widen(out[c]) + widen(r));
        out[c] = r;
    }
}

static bool geom_ok(const ConvGeom& g) {
    if (g.N <= 0 || g.C <= 0 || g.H <= 0 || g.W <= 0 || g.kH <= 0 || g.kW <= 0 || g.sh <= 0 || g.sw <= 0 || g.ph < 0 || g.pw < 0 ||
        g.dh <= 0 || g.dw <= 0 || g.oH <= 0 || g.oW <= 0) return false;
    // the output extent must be the one the geometry implies, or the gathers would leave the image
    const long long eh = ((long long)g.H + 2 * g.ph - (long long)g.dh * (g.kH - 1) - 1) / g.sh + 1;
    const long long ew = ((long long)g.W + 2 * g.pw - (long long)g.dw * (g.kW - 1) - 1) / g.sw + 1;
    if (g.oH != eh || g.oW != ew) return false;
    return (long long)g.C * g.kH * g.kW * (long long)g.oH * g.oW < (1ll << 31) && (long long)g.oH * g.oW < (1ll << 31);
}

static unsigned conv_grid(size_t work) {
    size_t b = (work + 255) / 256;
    return (unsigned)(b < 1 ? 1 : (b > (1u << 20) ? (1u << 20) : b));
}

template <typename T>
static void launch_im2col(void* col, const void* im, const ConvGeom& g) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const size_t total = (size_t)g.N * g.C * g.kH * g.kW * g.oH * g.oW;
    if ((g.oH * g.oW) % VEC == 0 && ((uintptr_t)col & 15) == 0)
        hipLaunchKernelGGL((im2col_kernel<T, VEC>), dim3(conv_grid(total / VEC)), dim3(256), 0, current_stream(), (T*)col, (const T*)im, g, total / VEC);
    else
        hipLaunchKernelGGL((im2col_kernel<T, 1>), dim3(conv_grid(total)), dim3(256), 0, current_stream(), (T*)col, (const T*)im, g, total);
}

template <typename T>
static void launch_col2im(void* im, const void* col, const ConvGeom& g, bool start_from_im) {
    const size_t total = (size_t)g.N * g.C * g.H * g.W;
    if (start_from_im)
        hipLaunchKernelGGL((col2im_gather_kernel<T, true>), dim3(conv_grid(total)), dim3(256), 0, current_stream(), (T*)im, (const T*)col, g, total);
    else
        hipLaunchKernelGGL((col2im_gather_kernel<T, false>), dim3(conv_grid(total)), dim3(256), 0, current_stream(), (T*)im, (const T*)col, g, total);
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
    const size_t total = (size_t)batch * channels * hw;
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(channel_bias_add_kernel<T>, dim3(conv_grid(total)), dim3(256), 0, current_stream(),
                                               (T*)y, (const T*)bias, channels, hw, total));
    return check_launch("channel_bias_add_kernel") ? 0 : -1;
}

int rp_hip_channel_sums(void* out, const void* grad, int batch, int channels, int hw, int accumulate, int dtype) {
    if (!out || !grad || batch <= 0 || channels <= 0 || hw <= 0) { set_error("rp_hip_channel_sums: null operand or non-positive extent"); return -1; }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(channel_sums_kernel<T>, dim3(channels), dim3(256), 0, current_stream(),
                                               (T*)out, (const T*)grad, batch, channels, hw, accumulate));
    return check_launch("channel_sums_kernel") ? 0 : -1;
}

}  // extern "C"
