// LSTM and GRU cells as callers of the GEMM: the element-wise half of a step, fused.
//
// A cell step is two GEMMs into the gate pre-activations (x . W_ih and h . W_hh; for the LSTM the second one
// accumulates into the first's output, beta = 1) followed by a chain of sigmoid / tanh / mul / add ops, each its own
// launch and its own tensor in the reference (recpulse/module.py:281-300 LSTM, 334-351 GRU).  Here the chain is one
// kernel forward and one backward.  Every intermediate the reference materialises is rounded to the tensor dtype at
// the same point (sigmoid and tanh outputs, the two products of c_next, tanh(c_next), ...), so 16-bit results follow
// the reference's chain of roundings; arithmetic is float32 (float64 for float64).
//
// Layouts (row-major, H = hidden size):
//   LSTM  gates [B, 4H] = i | f | g | o      (reference gate order, recpulse/module.py:289-293)
//         hc    [B, 2H] = h_next | c_next    (one tensor so that the step is one autograd node; the halves are views)
//   GRU   gi, gh [B, 3H] = r | z | n         (recpulse/module.py:339-344)
#include "rp_common.h"

namespace rp {

template <typename A> __device__ __forceinline__ A sigmoid_acc(A x);
template <> __device__ __forceinline__ float sigmoid_acc<float>(float x) { return 1.0f / (1.0f + expf(-x)); }      // reference functional_host.c:533
template <> __device__ __forceinline__ double sigmoid_acc<double>(double x) { return 1.0 / (1.0 + exp(-x)); }
template <typename A> __device__ __forceinline__ A tanh_acc(A x);
template <> __device__ __forceinline__ float tanh_acc<float>(float x) { return tanhf(x); }
template <> __device__ __forceinline__ double tanh_acc<double>(double x) { return tanh(x); }

// round to the tensor dtype and come back: the value a materialised intermediate of the reference would hold
template <typename T> __device__ __forceinline__ typename traits<T>::acc rt(typename traits<T>::acc v) { return widen(narrow<T>(v)); }

// act [B, 4H] receives the activated gates (saved for the backward); hc [B, 2H] the new state.
template <typename T>
__global__ void __launch_bounds__(256) lstm_cell_forward_kernel(T* hc, T* act, const T* gates, const T* b_ih, const T* b_hh, const T* c_prev, long long c_rs,
                                                                 int batch, int hidden) {
    using A = typename traits<T>::acc;
    const size_t total = (size_t)batch * hidden;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
        const size_t b = idx / hidden, j = idx % hidden;
        const T* g = gates + b * 4 * hidden + j;
        // (gates + b_ih) + b_hh, a rounding after each add (recpulse/module.py:285-287)
        auto pre = [&](int q) {
            A v = widen(g[q * (size_t)hidden]);
            if (b_ih) v = rt<T>(v + widen(b_ih[q * (size_t)hidden + j]));
            if (b_hh) v = rt<T>(v + widen(b_hh[q * (size_t)hidden + j]));
            return v;
        };
        const A i_g = rt<T>(sigmoid_acc<A>(pre(0)));
        const A f_g = rt<T>(sigmoid_acc<A>(pre(1)));
        const A g_g = rt<T>(tanh_acc<A>(pre(2)));
        const A o_g = rt<T>(sigmoid_acc<A>(pre(3)));
        const A c = widen(c_prev[b * c_rs + j]);
        const A c_next = rt<T>(rt<T>(f_g * c) + rt<T>(i_g * g_g));
        const A h_next = o_g * rt<T>(tanh_acc<A>(c_next));
        T* a = act + b * 4 * hidden + j;
        a[0] = narrow<T>(i_g); a[hidden] = narrow<T>(f_g); a[2 * (size_t)hidden] = narrow<T>(g_g); a[3 * (size_t)hidden] = narrow<T>(o_g);
        hc[b * 2 * hidden + j] = narrow<T>(h_next);
        hc[b * 2 * hidden + hidden + j] = narrow<T>(c_next);
    }
}

// dgates [B, 4H] (gradient of the pre-activations) and dc_prev [B, H] from dhc [B, 2H] (gradient of h_next | c_next).
template <typename T>
__global__ void __launch_bounds__(256) lstm_cell_backward_kernel(T* dgates, T* dc_prev, const T* dhc, const T* act, const T* hc, const T* c_prev,
                                                                  long long c_rs, int batch, int hidden) {
    using A = typename traits<T>::acc;
    const size_t total = (size_t)batch * hidden;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
        const size_t b = idx / hidden, j = idx % hidden;
        const T* a = act + b * 4 * hidden + j;
        const A i_g = widen(a[0]), f_g = widen(a[hidden]), g_g = widen(a[2 * (size_t)hidden]), o_g = widen(a[3 * (size_t)hidden]);
        const A dh = widen(dhc[b * 2 * hidden + j]), dc_in = widen(dhc[b * 2 * hidden + hidden + j]);
        const A tc = rt<T>(tanh_acc<A>(widen(hc[b * 2 * hidden + hidden + j])));
        const A c = widen(c_prev[b * c_rs + j]);
        // h = o * tanh(c_next); c_next = f * c + i * g       (mul, tanh, add backward: reference ops/grad_host.c:365-400, 622-660)
        const A d_o = rt<T>(dh * tc);
        const A d_tc = rt<T>(dh * o_g);
        const A dc = rt<T>(dc_in + rt<T>(d_tc * ((A)1 - tc * tc)));
        const A d_f = rt<T>(dc * c), d_c = rt<T>(dc * f_g), d_i = rt<T>(dc * g_g), d_g = rt<T>(dc * i_g);
        T* dg = dgates + b * 4 * hidden + j;
        dg[0] = narrow<T>(d_i * i_g * ((A)1 - i_g));
        dg[hidden] = narrow<T>(d_f * f_g * ((A)1 - f_g));
        dg[2 * (size_t)hidden] = narrow<T>(d_g * ((A)1 - g_g * g_g));
        dg[3 * (size_t)hidden] = narrow<T>(d_o * o_g * ((A)1 - o_g));
        dc_prev[idx] = narrow<T>(d_c);
    }
}

// h_next [B, H]; act [B, 3H] = r | z | n (saved for the backward).
template <typename T>
__global__ void __launch_bounds__(256) gru_cell_forward_kernel(T* h_next, T* act, const T* gi, const T* gh, const T* h_prev, long long h_rs, int batch, int hidden) {
    using A = typename traits<T>::acc;
    const size_t total = (size_t)batch * hidden;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
        const size_t b = idx / hidden, j = idx % hidden;
        const T* pi = gi + b * 3 * hidden + j;
        const T* ph = gh + b * 3 * hidden + j;
        const A r = rt<T>(sigmoid_acc<A>(rt<T>(widen(pi[0]) + widen(ph[0]))));
        const A z = rt<T>(sigmoid_acc<A>(rt<T>(widen(pi[hidden]) + widen(ph[hidden]))));
        const A n = rt<T>(tanh_acc<A>(rt<T>(widen(pi[2 * (size_t)hidden]) + rt<T>(r * widen(ph[2 * (size_t)hidden])))));
        const A h = widen(h_prev[b * h_rs + j]);
        // (1 - z) * n + z * h          (rsub_scalar, mul, mul, add: recpulse/module.py:350)
        const A out = rt<T>(rt<T>((A)1 - z) * n) + rt<T>(z * h);
        T* a = act + b * 3 * hidden + j;
        a[0] = narrow<T>(r); a[hidden] = narrow<T>(z); a[2 * (size_t)hidden] = narrow<T>(n);
        h_next[idx] = narrow<T>(out);
    }
}

// dgi, dgh [B, 3H] and the direct part of dh_prev [B, H] (dh_next * z; the part through gh comes from the GEMM).
template <typename T>
__global__ void __launch_bounds__(256) gru_cell_backward_kernel(T* dgi, T* dgh, T* dh_prev, const T* dh_next, const T* act, const T* gh, const T* h_prev,
                                                                 long long h_rs, int batch, int hidden) {
    using A = typename traits<T>::acc;
    const size_t total = (size_t)batch * hidden;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
        const size_t b = idx / hidden, j = idx % hidden;
        const T* a = act + b * 3 * hidden + j;
        const A r = widen(a[0]), z = widen(a[hidden]), n = widen(a[2 * (size_t)hidden]);
        const A h_n = widen(gh[b * 3 * hidden + 2 * (size_t)hidden + j]);
        const A h = widen(h_prev[b * h_rs + j]);
        const A dh = widen(dh_next[idx]);
        const A one_minus_z = rt<T>((A)1 - z);
        const A d_n = rt<T>(dh * one_minus_z);
        const A d_z = rt<T>(rt<T>(dh * h) - rt<T>(dh * n));          // through z * h and through (1 - z) * n
        const A d_pre_n = rt<T>(d_n * ((A)1 - n * n));
        const A d_r = rt<T>(d_pre_n * h_n);
        const A d_pre_r = rt<T>(d_r * r * ((A)1 - r));
        const A d_pre_z = rt<T>(d_z * z * ((A)1 - z));
        T* pi = dgi + b * 3 * hidden + j;
        T* ph = dgh + b * 3 * hidden + j;
        pi[0] = narrow<T>(d_pre_r); pi[hidden] = narrow<T>(d_pre_z); pi[2 * (size_t)hidden] = narrow<T>(d_pre_n);
        ph[0] = narrow<T>(d_pre_r); ph[hidden] = narrow<T>(d_pre_z); ph[2 * (size_t)hidden] = narrow<T>(d_pre_n * r);
        dh_prev[idx] = narrow<T>(dh * z);
    }
}

// dst[strided index] = src[dense index] over a shape of up to 8 dimensions: the scatter that puts the gradient of a
// slice back into (a zeroed copy of) the sliced tensor's shape.
struct ScatterArgs {
    int ndim;
    int shape[8];
    long long strides[8];
};

template <typename T>
__global__ void scatter_strided_kernel(T* dst, const T* src, ScatterArgs a, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        size_t rem = i;
        long long off = 0;
        for (int d = a.ndim - 1; d >= 0; d--) {
            off += (long long)(rem % a.shape[d]) * a.strides[d];
            rem /= a.shape[d];
        }
        dst[off] = src[i];
    }
}

static unsigned rnn_grid(size_t work) {
    size_t b = (work + 255) / 256;
    return (unsigned)(b < 1 ? 1 : (b > (1u << 20) ? (1u << 20) : b));
}

}  // namespace rp

using namespace rp;

extern "C" {

int rp_hip_lstm_cell_forward(void* hc, void* act, const void* gates, const void* b_ih, const void* b_hh, const void* c_prev, long long c_prev_row_stride,
                             int batch, int hidden, int dtype) {
    if (!hc || !act || !gates || !c_prev || batch <= 0 || hidden <= 0 || c_prev_row_stride < 0) { set_error("rp_hip_lstm_cell_forward: null operand or non-positive extent"); return -1; }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(lstm_cell_forward_kernel<T>, dim3(rnn_grid((size_t)batch * hidden)), dim3(256), 0, current_stream(),
                                               (T*)hc, (T*)act, (const T*)gates, (const T*)b_ih, (const T*)b_hh, (const T*)c_prev, c_prev_row_stride, batch, hidden));
    return check_launch("lstm_cell_forward_kernel") ? 0 : -1;
}

int rp_hip_lstm_cell_backward(void* dgates, void* dc_prev, const void* dhc, const void* act, const void* hc, const void* c_prev,
                              long long c_prev_row_stride, int batch, int hidden, int dtype) {
    if (!dgates || !dc_prev || !dhc || !act || !hc || !c_prev || batch <= 0 || hidden <= 0 || c_prev_row_stride < 0) {
        set_error("rp_hip_lstm_cell_backward: null operand or non-positive extent");
        return -1;
    }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(lstm_cell_backward_kernel<T>, dim3(rnn_grid((size_t)batch * hidden)), dim3(256), 0, current_stream(),
                                               (T*)dgates, (T*)dc_prev, (const T*)dhc, (const T*)act, (const T*)hc, (const T*)c_prev, c_prev_row_stride, batch, hidden));
    return check_launch("lstm_cell_backward_kernel") ? 0 : -1;
}

int rp_hip_gru_cell_forward(void* h_next, void* act, const void* gi, const void* gh, const void* h_prev, long long h_prev_row_stride, int batch, int hidden, int dtype) {
    if (!h_next || !act || !gi || !gh || !h_prev || batch <= 0 || hidden <= 0 || h_prev_row_stride < 0) { set_error("rp_hip_gru_cell_forward: null operand or non-positive extent"); return -1; }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(gru_cell_forward_kernel<T>, dim3(rnn_grid((size_t)batch * hidden)), dim3(256), 0, current_stream(),
                                               (T*)h_next, (T*)act, (const T*)gi, (const T*)gh, (const T*)h_prev, h_prev_row_stride, batch, hidden));
    return check_launch("gru_cell_forward_kernel") ? 0 : -1;
}

int rp_hip_gru_cell_backward(void* dgi, void* dgh, void* dh_prev, const void* dh_next, const void* act, const void* gh, const void* h_prev,
                             long long h_prev_row_stride, int batch, int hidden, int dtype) {
    if (!dgi || !dgh || !dh_prev || !dh_next || !act || !gh || !h_prev || batch <= 0 || hidden <= 0 || h_prev_row_stride < 0) {
        set_error("rp_hip_gru_cell_backward: null operand or non-positive extent");
        return -1;
    }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(gru_cell_backward_kernel<T>, dim3(rnn_grid((size_t)batch * hidden)), dim3(256), 0, current_stream(),
                                               (T*)dgi, (T*)dgh, (T*)dh_prev, (const T*)dh_next, (const T*)act, (const T*)gh, (const T*)h_prev, h_prev_row_stride, batch, hidden));
    return check_launch("gru_cell_backward_kernel") ? 0 : -1;
}

int rp_hip_scatter_strided(void* dst, const void* src, int ndim, const int* shape, const long long* dst_strides, size_t size, int dtype) {
    if (!dst || !src || !shape || !dst_strides || ndim <= 0 || ndim > 8 || size == 0) { set_error("rp_hip_scatter_strided: null operand, empty tensor or more than 8 dimensions"); return -1; }
    ScatterArgs a;
    a.ndim = ndim;
    size_t n = 1;
    for (int d = 0; d < ndim; d++) {
        if (shape[d] <= 0 || dst_strides[d] < 0) { set_error("rp_hip_scatter_strided: non-positive extent or negative stride"); return -1; }
        a.shape[d] = shape[d]; a.strides[d] = dst_strides[d];
        n *= (size_t)shape[d];
    }
    if (n != size) { set_error("rp_hip_scatter_strided: size does not match the shape"); return -1; }
    RP_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(scatter_strided_kernel<T>, dim3(rnn_grid(size)), dim3(256), 0, current_stream(), (T*)dst, (const T*)src, a, size));
    return check_launch("scatter_strided_kernel") ? 0 : -1;
}

}  // extern "C"
