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
#include "rp_gemm.h"

namespace rp {

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

// The common case on its own: 3 x 3 taps, stride 1, padding 1, no dilation, rows a whole number of vectors (so
// oH = H, oW = W and every vector of a row is 16-byte aligned in the image and in every col row).  The three taps of
// one image row are the aligned vector at the thread's columns shifted by -1, 0 and +1 elements: one vector load and
// its two neighbouring elements per image row, no per-element masks and no variable shifts (the general kernel is
// bound by that arithmetic, not by memory).
template <typename T, int VEC>
__global__ void __launch_bounds__(256) im2col_3x3_kernel(T* col, const T* im, int H, int W, unsigned total_vec) {
    const unsigned vec_per_row = W / VEC, vec_per_plane = H * vec_per_row;
    const unsigned gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= total_vec) return;
    const unsigned plane_id = gid / vec_per_plane, pv = gid % vec_per_plane;
    const int h = pv / vec_per_row, w0 = (pv % vec_per_row) * VEC;
    const size_t cols = (size_t)H * W;
    const T* plane = im + plane_id * cols;
    T* dst = col + (size_t)plane_id * 9 * cols + (size_t)pv * VEC;
    T zero;
    memset(&zero, 0, sizeof(T));
#pragma unroll
    for (int kh = 0; kh < 3; kh++) {
        const int h_in = h + kh - 1;
        const bool inside = h_in >= 0 && h_in < H;
        const T* row = plane + (size_t)(inside ? h_in : h) * W;
        T v[VEC + 2];                                          // columns w0 - 1 .. w0 + VEC of the image row
        const u32x4_t raw = *(const u32x4_t*)(row + w0);
        memcpy(&v[1], &raw, 16);
        v[0] = row[w0 > 0 ? w0 - 1 : 0];
        v[VEC + 1] = row[w0 + VEC < W ? w0 + VEC : W - 1];
        if (!inside || w0 == 0) v[0] = zero;
        if (!inside || w0 + VEC >= W) v[VEC + 1] = zero;
        if (!inside) {
#pragma unroll
            for (int e = 1; e <= VEC; e++) v[e] = zero;
        }
#pragma unroll
        for (int kw = 0; kw < 3; kw++) {
            u32x4_t out;
            memcpy(&out, &v[kw], 16);
            *(u32x4_t*)(dst + (size_t)(kh * 3 + kw) * cols) = out;
        }
    }
}

// The adjoint of im2col_3x3_kernel, as a gather: pixel (h, w) adds col row (kh, kw) at (h + 1 - kh, w + 1 - kw), taps in
// ascending (kh, kw) order.  Per tap one aligned vector load and one neighbouring element.
template <typename T, int VEC, bool START_FROM_IM>
__global__ void __launch_bounds__(256) col2im_3x3_kernel(T* im, const T* col, int H, int W, unsigned total_vec) {
    using A = typename traits<T>::acc;
    const unsigned vec_per_row = W / VEC, vec_per_plane = H * vec_per_row;
    const unsigned gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= total_vec) return;
    const unsigned plane_id = gid / vec_per_plane, pv = gid % vec_per_plane;
    const int h = pv / vec_per_row, w0 = (pv % vec_per_row) * VEC;
    const size_t cols = (size_t)H * W;
    const T* rows = col + (size_t)plane_id * 9 * cols;
    T* dst = im + (size_t)gid * VEC;
    A acc[VEC];
    if (START_FROM_IM) {
        T cur[VEC];
        memcpy(cur, dst, 16);
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = widen(cur[e]);
    } else {
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = (A)0;
    }
    const bool has_left = w0 > 0, has_right = w0 + VEC < W;
#pragma unroll
    for (int kh = 0; kh < 3; kh++) {
        const int oh = h + 1 - kh;
        const bool inside = oh >= 0 && oh < H;
        const T* base = rows + (size_t)(kh * 3) * cols + (size_t)(inside ? oh : h) * W;
#pragma unroll
        for (int kw = 0; kw < 3; kw++) {
            const T* row = base + (size_t)kw * cols;
            T v[VEC + 2];                                      // columns w0 - 1 .. w0 + VEC of the col row; only the ones this tap uses are loaded
            const u32x4_t raw = *(const u32x4_t*)(row + w0);
            memcpy(&v[1], &raw, 16);
            if (kw == 0) v[VEC + 1] = row[has_right ? w0 + VEC : W - 1];
            if (kw == 2) v[0] = row[has_left ? w0 - 1 : 0];
            // pixel w0 + e takes column w0 + e + 1 - kw, i.e. v[e + 2 - kw]
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                const bool there = inside && (kw != 0 || e < VEC - 1 || has_right) && (kw != 2 || e > 0 || has_left);
                const A sum = acc[e] + widen(v[e + 2 - kw]);
                acc[e] = there ? sum : acc[e];
            }
        }
    }
    T out[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) out[e] = narrow<T>(acc[e]);
    u32x4_t packed;
    memcpy(&packed, out, 16);
    *(u32x4_t*)dst = packed;
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

// ---- convolution without a lowered matrix (stride 1, "same" padding) ----
// With the image copied once into planes of pitch Wp >= W + 2 * pad with a zero border, output position f = oh * Wp + ow
// of tap (kh, kw) reads padded element f + kh * Wp + kw: every tap is the same matrix [C, H * Wp] at a different
// offset, which the GEMM reads in place as a segment of its k axis (GemmArgs::seg_*).  The product comes out in the
// same pitch (columns ow >= W hold sums that nobody uses): the GEMM's epilogue stores only the valid columns, folded
// into dense planes, and adds the bias per output channel (GemmArgs::c_fold_*, bias_by_row) when image rows are whole
// 16-byte vectors; otherwise the product stays in the planes' pitch and unpad_planes_kernel copies the valid part.
struct PadGeom {
    int H, W, ph, pw, Hp, Wp;
    long long P;                  // elements per padded plane (Hp * Wp plus the slack the last tap may read)
};

// Weights [C_out, C_in, taps] reordered for the segmented GEMM.  Forward: [C_out][tap][C_in].  Backward to the input:
// [C_in][tap][C_out] with the taps reversed (the gradient is a correlation with the kernel turned by 180 degrees).
// The job rides on the launch that pads the planes (its last `blocks` workgroups): the GEMM that needs both comes next
// anyway, and a launch of its own costs more than the 70 KB it moves.
struct WeightJob {
    void* out;
    const void* w;
    int C_out, C_in, taps, for_input_grad, blocks;       // blocks == 0: no job
};

template <typename T>
__device__ __forceinline__ void weights_by_tap(const WeightJob& j, int block, int nblocks) {
    T* out = (T*)j.out;
    const T* w = (const T*)j.w;
    const int total = j.C_out * j.C_in * j.taps;
    for (int i = block * 256 + threadIdx.x; i < total; i += nblocks * 256) {
        if (!j.for_input_grad) {
            const int ci = i % j.C_in, tap = (i / j.C_in) % j.taps, co = i / (j.C_in * j.taps);
            out[i] = w[((size_t)co * j.C_in + ci) * j.taps + tap];
        } else {
            const int co = i % j.C_out, tap = (i / j.C_out) % j.taps, ci = i / (j.C_out * j.taps);
            out[i] = w[((size_t)co * j.C_in + ci) * j.taps + (j.taps - 1 - tap)];
        }
    }
}

template <typename T, int VEC, bool ALIGNED_ROWS>
__global__ void __launch_bounds__(256) pad_planes_kernel(T* out, const T* in, PadGeom g, unsigned total_vec, WeightJob job) {
    const unsigned pad_blocks = gridDim.x - job.blocks;
    if (blockIdx.x >= pad_blocks) { weights_by_tap<T>(job, blockIdx.x - pad_blocks, job.blocks); return; }
    const unsigned vec_per_plane = (unsigned)(g.P / VEC);
    const unsigned gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= total_vec) return;
    const unsigned plane = gid / vec_per_plane, pv = gid % vec_per_plane;
    const int e0 = (int)pv * VEC, r = e0 / g.Wp, c0 = e0 % g.Wp;           // Wp is a whole number of vectors: one row per vector
    const int h = r - g.ph;
    T v[VEC];
    if (ALIGNED_ROWS && g.pw == 1) {
        // W a whole number of vectors and one column of border: the aligned vector at c0 moved up one element, with
        // the element before it in front
        const bool row_inside = h >= 0 && h < g.H;
        const T* row = in + ((size_t)plane * g.H + (row_inside ? h : 0)) * g.W;
        T w[VEC + 1];
        const bool have_vec = row_inside && c0 < g.W, have_left = row_inside && c0 >= 1 && c0 <= g.W;
        const u32x4_t raw = *(const u32x4_t*)(row + (have_vec ? c0 : 0));
        memcpy(&w[1], &raw, 16);
        w[0] = row[have_left ? c0 - 1 : 0];
        if (!have_left) memset(&w[0], 0, sizeof(T));
        if (!have_vec) memset(&w[1], 0, VEC * sizeof(T));
        memcpy(v, w, VEC * sizeof(T));
    } else if (h >= 0 && h < g.H && g.W >= VEC) {
        load_span<T, VEC>(v, in + ((size_t)plane * g.H + h) * g.W, c0 - g.pw, g.W);
    } else {
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const int w = c0 + e - g.pw;
            if (h >= 0 && h < g.H && w >= 0 && w < g.W) v[e] = in[((size_t)plane * g.H + h) * g.W + w];
            else memset(&v[e], 0, sizeof(T));
        }
    }
    u32x4_t raw;
    memcpy(&raw, v, 16);
    *(u32x4_t*)(out + (size_t)plane * g.P + e0) = raw;
}

template <typename T>
static void launch_pad(T* out, const T* in, const PadGeom& pg, unsigned vecs, WeightJob job = WeightJob{nullptr, nullptr, 0, 0, 0, 0, 0}) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const dim3 grid((vecs + 255) / 256 + job.blocks);
    if (pg.W % VEC == 0 && ((uintptr_t)in & 15) == 0) hipLaunchKernelGGL((pad_planes_kernel<T, VEC, true>), grid, dim3(256), 0, current_stream(), out, in, pg, vecs, job);
    else hipLaunchKernelGGL((pad_planes_kernel<T, VEC, false>), grid, dim3(256), 0, current_stream(), out, in, pg, vecs, job);
}

static WeightJob weight_job(void* out, const void* w, int C_out, int C_in, int taps, bool for_input_grad) {
    const int total = C_out * C_in * taps;
    return WeightJob{out, w, C_out, C_in, taps, for_input_grad ? 1 : 0, (total + 255) / 256 > 64 ? 64 : (total + 255) / 256};
}

// y[plane][h][w] = yp[plane][h * Wp + w] (+ bias[channel], one rounding add as channel_bias_add_kernel does)
template <typename T, int VEC>
__global__ void __launch_bounds__(256) unpad_planes_kernel(T* y, const T* yp, const T* bias, int channels, int H, int W, int Wp, unsigned total_vec) {
    const unsigned vec_per_plane = (unsigned)(H * W / VEC);
    const unsigned gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= total_vec) return;
    const unsigned plane = gid / vec_per_plane;
    const int e0 = (int)(gid % vec_per_plane) * VEC;
    const T* src = yp + (size_t)plane * H * Wp;
    T v[VEC];
    if constexpr (VEC > 1) {                               // W is a whole number of vectors: the vector stays inside one row
        const u32x4_t raw = *(const u32x4_t*)(src + (size_t)(e0 / W) * Wp + e0 % W);
        memcpy(v, &raw, 16);
    } else {
        v[0] = src[(size_t)(e0 / W) * Wp + e0 % W];
    }
    if (bias) {
        const auto b = widen(bias[plane % channels]);
#pragma unroll
        for (int e = 0; e < VEC; e++) v[e] = narrow<T>(widen(v[e]) + b);
    }
    memcpy(y + (size_t)gid * VEC, v, VEC * sizeof(T));
}

static PadGeom pad_geom(int H, int W, int kH, int kW, int vec);

// Bytes of padded planes and products held at a time (the batch goes in chunks).  RP_CONV_WORKSPACE_BYTES overrides the
// 1 GiB default; it is read at every call so that tests can force several chunks.
static long long same_conv_workspace() {
    const char* e = getenv("RP_CONV_WORKSPACE_BYTES");
    const long long v = e ? atoll(e) : 0;
    return v > 0 ? v : (1ll << 30);
}

static bool same_conv_ok(int reduced_channels, int H, int W, int kH, int kW, int dtype) {
    // the channels summed over come in whole k slabs of the GEMM kernel that runs: 64 (16-bit), 32 (float32), 16 (float64)
    const int slab = (dtype == RP_DTYPE_BFLOAT16 || dtype == RP_DTYPE_FLOAT16) ? M16_BK : (dtype == RP_DTYPE_FLOAT32 ? 32 : 16);
    return dtype_size(dtype) != 0 && reduced_channels >= 0 && reduced_channels % slab == 0 &&
           H > 0 && W > 0 && kH > 0 && kW > 0 && kH % 2 == 1 && kW % 2 == 1 && kH * kW > 1 && kW <= 15 && kH <= 15 &&
           (long long)(H + kH) * (W + kW + 8) < (1ll << 21);
}

// out[nb, C_to, H, W] (dense) = sum over taps and C_from of wt[C_to][tap][C_from] . padded[nb, C_from, planes of pg], (+ bias per
// channel): the GEMM whose k axis walks the taps as segments.  When image rows are whole 16-byte vectors its epilogue
// stores only the valid columns, folded into dense planes, and adds the bias; otherwise the product goes to `product`
// ([nb, C_to, H * Wp]) and a copy kernel drops the unused columns.
template <typename T>
static int taps_gemm(T* out, void* product, const void* wt, const void* padded, const void* bias, int nb, int C_from, int C_to,
                     const PadGeom& pg, int kH, int kW, int dtype) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int H = pg.H, W = pg.W;
    const long long cols = (long long)H * pg.Wp;
    const bool fold = W % VEC == 0 && ((uintptr_t)out & 15) == 0;
    GemmArgs g{};
    g.A = wt; g.B = padded;
    g.batch = nb; g.m = C_to; g.k = kH * kW * C_from; g.n = (int)cols;
    g.a_bs = 0; g.a_rs = (long long)kH * kW * C_from; g.a_cs = 1;
    g.b_bs = (long long)C_from * pg.P; g.b_rs = pg.P; g.b_cs = 1;
    g.seg_k = C_from; g.seg_w = kW; g.seg_sh = pg.Wp; g.seg_sw = 1; g.b_extent = (long long)C_from * pg.P;
    g.c_cs = 1;
    if (fold) {
        g.C = out; g.c_bs = (long long)C_to * H * W; g.c_rs = (long long)H * W;
        g.c_fold_from = pg.Wp; g.c_fold_to = W; g.bias = bias; g.bias_by_row = 1;
    } else {
        g.C = product; g.c_bs = (long long)C_to * cols; g.c_rs = cols;
    }
    if (launch_gemm_segmented_b(g, dtype) != 0) return -1;
    if (!fold) {
        const unsigned elems = (unsigned)((long long)nb * C_to * H * W);
        hipLaunchKernelGGL((unpad_planes_kernel<T, 1>), dim3((elems + 255) / 256), dim3(256), 0, current_stream(), out, (const T*)product, (const T*)bias, C_to, H, W, pg.Wp, elems);
    }
    return 0;
}

// out[batch, C_to, H, W] = sum over taps and C_from of wt . padded(in[batch, C_from, H, W]); wt as weights_by_tap
// leaves it ([C_to][tap][C_from]).  bias may be null.  The batch goes in chunks that keep the workspace under same_conv_workspace().
template <typename T>
static int same_conv_run(void* out, const void* in, const void* wt, const void* bias, int batch, int C_from, int C_to,
                         int H, int W, int kH, int kW, int dtype, WeightJob job) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const PadGeom pg = pad_geom(H, W, kH, kW, VEC);
    const long long cols = (long long)H * pg.Wp;
    const long long per_sample = ((long long)C_from * pg.P + (long long)C_to * cols) * (long long)sizeof(T);
    long long chunk = same_conv_workspace() / per_sample;
    chunk = chunk < 1 ? 1 : (chunk > 32768 ? 32768 : chunk);
    if (chunk > batch) chunk = batch;
    if (chunk * (long long)C_from * (pg.P / VEC) >= (1ll << 31) || chunk * (long long)C_to * H * W >= (1ll << 31)) {
        set_error("conv2d: one sample is too large for the padded-plane path");
        return -1;
    }
    void* padded = nullptr;
    void* product = nullptr;
    if (rp_hip_malloc(&padded, (size_t)(chunk * C_from * pg.P) * sizeof(T)) != 0) return -1;
    if (rp_hip_malloc(&product, (size_t)(chunk * C_to * cols) * sizeof(T)) != 0) { rp_hip_free(padded); return -1; }
    int rc = 0;
    for (int b0 = 0; b0 < batch && rc == 0; b0 += (int)chunk) {
        const int nb = batch - b0 < chunk ? batch - b0 : (int)chunk;
        const T* in0 = (const T*)in + (size_t)b0 * C_from * H * W;
        T* out0 = (T*)out + (size_t)b0 * C_to * H * W;
        const unsigned pad_vecs = (unsigned)((long long)nb * C_from * (pg.P / VEC));
        launch_pad<T>((T*)padded, in0, pg, pad_vecs, job);          // the first chunk's launch reorders the weights too
        job.blocks = 0;
        rc = taps_gemm<T>(out0, product, wt, padded, bias, nb, C_from, C_to, pg, kH, kW, dtype);
    }
    if (rc == 0 && !check_launch("padded-plane convolution kernels")) rc = -1;
    rp_hip_free(product);
    rp_hip_free(padded);
    return rc;
}

template <typename T>
static int same_conv(void* out, const void* in, const void* w, const void* bias, int batch, int C_from, int C_to,
                     int H, int W, int kH, int kW, bool for_input_grad, int dtype) {
    const int taps = kH * kW, total = C_from * C_to * taps;
    void* wt = nullptr;
    if (rp_hip_malloc(&wt, (size_t)total * sizeof(T)) != 0) return -1;
    // w is [C_out, C_in, taps]: forward reduces over C_in (C_from = C_in, C_to = C_out), the input gradient over C_out
    const int C_out = for_input_grad ? C_from : C_to, C_in = for_input_grad ? C_to : C_from;
    const int rc = same_conv_run<T>(out, in, wt, bias, batch, C_from, C_to, H, W, kH, kW, dtype, weight_job(wt, w, C_out, C_in, taps, for_input_grad));
    rp_hip_free(wt);
    return rc;
}

// dw[co][ci][tap] (+)= sum over the nb samples of per_sample[n][co][tap][ci]: the per-sample products added top to bottom in
// the accumulate type and rounded once (what rp_hip_reduce_rows does), written back in the weights' own order.
// accumulate: a later chunk of the batch adds to what the earlier ones left, with a rounding of its own.
template <typename T>
__global__ void conv_dw_from_samples_kernel(T* dw, const T* per_sample, int nb, int C_out, int C_in, int taps, int accumulate) {
    using A = typename traits<T>::acc;
    const int total = C_out * C_in * taps;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;             // index in [co][tap][ci] order: neighbouring threads read neighbouring elements
    if (i >= total) return;
    const int ci = i % C_in, tap = (i / C_in) % taps, co = i / (C_in * taps);
    A s = 0;
    int n = 0;
    constexpr int U = 16;                                            // independent loads in flight; the adds stay in sample order
    for (; n + U <= nb; n += U) {
        A v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = widen(per_sample[(size_t)(n + u) * total + i]);
#pragma unroll
        for (int u = 0; u < U; u++) s += v[u];
    }
    for (; n < nb; n++) s += widen(per_sample[(size_t)n * total + i]);
    T r = narrow<T>(s);
    T* dst = dw + ((size_t)co * C_in + ci) * taps + tap;
    if (accumulate) r = narrow<T>(widen(*dst) + widen(r));
    *dst = r;
}

static PadGeom pad_geom(int H, int W, int kH, int kW, int vec) {
    PadGeom pg;
    pg.H = H; pg.W = W; pg.ph = kH / 2; pg.pw = kW / 2; pg.Hp = H + kH - 1;
    pg.Wp = (W + kW - 1 + vec - 1) / vec * vec;
    pg.P = (long long)pg.Hp * pg.Wp + 16;                    // the last tap of the last position reads up to kW - 2 <= 13 elements past Hp * Wp
    return pg;
}

// Both gradients of a same-padding convolution from one zero-bordered copy of dy (either output may be null).
//   dx[n, ci]       = sum over taps and co of w[co, ci, reversed tap] . padded(dy)[n, co] shifted by the tap      (segments along k)
//   dw[co, ci, tap] = sum over n and positions of padded(dy)[n, co] . padded(x)[n, ci] shifted by the tap          (segments along n),
// the per-sample products rounded to T and then added over the batch in the accumulate type, as the lowered path does.
template <typename T>
static int same_conv_backward(void* dx, void* dw, const void* dy, const void* x, const void* w, int batch, int C_in, int H, int W,
                              int C_out, int kH, int kW, int dtype) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const PadGeom pg = pad_geom(H, W, kH, kW, VEC);
    const int taps = kH * kW;
    const long long cols = (long long)H * pg.Wp, w_n = (long long)C_out * C_in * taps;
    const long long product_n = (dx && (long long)C_in * cols > (dw ? w_n : 0)) ? (long long)C_in * cols : (dw ? w_n : (long long)C_in * cols);
    const long long per_sample = ((long long)C_out * pg.P + (dw ? (long long)C_in * pg.P : 0) + product_n) * (long long)sizeof(T);
    long long chunk = same_conv_workspace() / per_sample;
    chunk = chunk < 1 ? 1 : (chunk > 32768 ? 32768 : chunk);
    if (chunk > batch) chunk = batch;
    const long long most_channels = C_in > C_out ? C_in : C_out;
    if (chunk * most_channels * (pg.P / VEC) >= (1ll << 31) || chunk * (long long)C_in * H * W >= (1ll << 31) || w_n >= (1ll << 31) ||
        most_channels * pg.P >= (1ll << 30)) {
        set_error("conv2d backward: one sample is too large for the padded-plane path");
        return -1;
    }
    void *dy_pad = nullptr, *x_pad = nullptr, *product = nullptr, *wt = nullptr;
    bool ok = rp_hip_malloc(&dy_pad, (size_t)(chunk * C_out * pg.P) * sizeof(T)) == 0 &&
              rp_hip_malloc(&product, (size_t)(chunk * product_n) * sizeof(T)) == 0 &&
              (!dx || rp_hip_malloc(&wt, (size_t)w_n * sizeof(T)) == 0) &&
              (!dw || rp_hip_malloc(&x_pad, (size_t)(chunk * C_in * pg.P) * sizeof(T)) == 0);
    WeightJob job = dx ? weight_job(wt, w, C_out, C_in, taps, true) : WeightJob{nullptr, nullptr, 0, 0, 0, 0, 0};
    for (int b0 = 0; ok && b0 < batch; b0 += (int)chunk) {
        const int nb = batch - b0 < chunk ? batch - b0 : (int)chunk;
        const T* dy0 = (const T*)dy + (size_t)b0 * C_out * H * W;
        const unsigned dy_vecs = (unsigned)((long long)nb * C_out * (pg.P / VEC));
        launch_pad<T>((T*)dy_pad, dy0, pg, dy_vecs, job);          // the first chunk's launch reorders the weights for dx too
        job.blocks = 0;
        if (dx) {
            T* dx0 = (T*)dx + (size_t)b0 * C_in * H * W;
            ok = taps_gemm<T>(dx0, product, wt, dy_pad, nullptr, nb, C_out, C_in, pg, kH, kW, dtype) == 0;
            if (!ok) break;
        }
        if (dw) {
            const T* x0 = (const T*)x + (size_t)b0 * C_in * H * W;
            const unsigned x_vecs = (unsigned)((long long)nb * C_in * (pg.P / VEC));
            launch_pad<T>((T*)x_pad, x0, pg, x_vecs);
            GemmArgs g{};
            g.C = product;
            g.A = (const T*)dy_pad + (size_t)pg.ph * pg.Wp + pg.pw;          // dy in the pitch of the padded planes, zeros in the columns past W
            g.B = x_pad;
            g.batch = nb; g.m = C_out; g.k = (int)cols; g.n = taps * C_in;
            g.a_bs = (long long)C_out * pg.P; g.a_rs = pg.P; g.a_cs = 1;
            g.b_bs = (long long)C_in * pg.P; g.b_rs = 1; g.b_cs = pg.P;
            g.c_bs = w_n; g.c_rs = (long long)taps * C_in; g.c_cs = 1;
            g.seg_n = C_in; g.seg_w = kW; g.seg_sh = pg.Wp; g.seg_sw = 1; g.b_extent = (long long)C_in * pg.P;
            ok = launch_gemm_segmented_b(g, dtype) == 0;
            if (ok) hipLaunchKernelGGL(conv_dw_from_samples_kernel<T>, dim3((unsigned)((w_n + 255) / 256)), dim3(256), 0, current_stream(),
                                       (T*)dw, (const T*)product, nb, C_out, C_in, taps, b0 > 0 ? 1 : 0);
        }
    }
    if (ok && !check_launch("padded-plane convolution kernels")) ok = false;
    for (void* p : {dy_pad, x_pad, product, wt})
        if (p) rp_hip_free(p);
    return ok ? 0 : -1;
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

// 3 x 3 taps, stride 1, padding 1, no dilation, rows a whole number of vectors: the shape the *_3x3 kernels take
static bool same_3x3(const ConvGeom& g, int vec) {
    return g.kH == 3 && g.kW == 3 && g.sh == 1 && g.sw == 1 && g.ph == 1 && g.pw == 1 && g.dh == 1 && g.dw == 1 && g.W % vec == 0 && g.W >= vec;
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
        if (vec && same_3x3(g, VEC) && ((uintptr_t)im & 15) == 0) hipLaunchKernelGGL((im2col_3x3_kernel<T, VEC>), grid, dim3(256), 0, current_stream(), c0, i0, g.H, g.W, total);
        else if (vec && g.kH == 3 && g.kW == 3) hipLaunchKernelGGL((im2col_kernel<T, VEC, true>), grid, dim3(256), 0, current_stream(), c0, i0, g, total);
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
        if (vec && same_3x3(g, VEC) && ((uintptr_t)col & 15) == 0) {
            if (start_from_im) hipLaunchKernelGGL((col2im_3x3_kernel<T, VEC, true>), grid, dim3(256), 0, current_stream(), i0, c0, g.H, g.W, total);
            else hipLaunchKernelGGL((col2im_3x3_kernel<T, VEC, false>), grid, dim3(256), 0, current_stream(), i0, c0, g.H, g.W, total);
        } else if (vec) {
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

int rp_hip_conv2d_same_supported(int reduced_channels, int H, int W, int kH, int kW, int dtype) {
    return same_conv_ok(reduced_channels, H, W, kH, kW, dtype) ? 1 : 0;
}

int rp_hip_conv2d_same_forward(void* y, const void* x, const void* w, const void* bias, int batch, int C_in, int H, int W,
                               int C_out, int kH, int kW, int dtype) {
    if (!y || !x || !w || batch <= 0 || C_out <= 0 || !same_conv_ok(C_in, H, W, kH, kW, dtype) || ((uintptr_t)x & 1) || ((uintptr_t)y & 1)) {
        set_error("rp_hip_conv2d_same_forward: null operand or a shape outside rp_hip_conv2d_same_supported");
        return -1;
    }
    const size_t esz = dtype_size(dtype);
    if (((uintptr_t)x | (uintptr_t)y) & (esz - 1)) { set_error("rp_hip_conv2d_same_forward: misaligned operand"); return -1; }
    RP_DISPATCH_DTYPE(dtype, return same_conv<T>(y, x, w, bias, batch, C_in, C_out, H, W, kH, kW, false, dtype));
    return -1;
}

int rp_hip_conv2d_same_backward_input(void* dx, const void* dy, const void* w, int batch, int C_in, int H, int W,
                                      int C_out, int kH, int kW, int dtype) {
    if (!dx || !dy || !w || batch <= 0 || C_in <= 0 || !same_conv_ok(C_out, H, W, kH, kW, dtype) || ((uintptr_t)dx & 1) || ((uintptr_t)dy & 1)) {
        set_error("rp_hip_conv2d_same_backward_input: null operand or a shape outside rp_hip_conv2d_same_supported");
        return -1;
    }
    RP_DISPATCH_DTYPE(dtype, return same_conv_backward<T>(dx, nullptr, dy, nullptr, w, batch, C_in, H, W, C_out, kH, kW, dtype));
    return -1;
}

int rp_hip_conv2d_same_backward(void* dx, void* dw, const void* dy, const void* x, const void* w, int batch, int C_in, int H, int W,
                                int C_out, int kH, int kW, int dtype) {
    const bool shapes = batch > 0 && C_in > 0 && C_out > 0 && same_conv_ok(dx ? C_out : 0, H, W, kH, kW, dtype);
    if ((!dx && !dw) || !dy || (dx && !w) || (dw && !x) || !shapes) {
        set_error("rp_hip_conv2d_same_backward: null operand or a shape outside rp_hip_conv2d_same_supported");
        return -1;
    }
    RP_DISPATCH_DTYPE(dtype, return same_conv_backward<T>(dx, dw, dy, x, w, batch, C_in, H, W, C_out, kH, kW, dtype));
    return -1;
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
