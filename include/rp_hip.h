/*
 * rp_hip.h — C ABI of librp_hip.so, the MI355X (gfx950) device layer for the
 * RecPulse matmul path.
 *
 * Plain C: pointers, sizes, ints.  Every function returns 0 on success and -1
 * on failure (the reference's convention for its *_kernel_device functions);
 * rp_hip_last_error() gives the text.  Device pointers are raw HIP device
 * addresses.  All work is enqueued on the calling thread's current stream
 * (the null stream unless rp_hip_set_stream() changed it) and is NOT waited
 * for: completion is stream-ordered, as with the reference's CUDA entry points.
 *
 * Entry points that keep the reference's own symbol name replace the function
 * of that name in the reference's CUDA files one for one, so the reference's
 * host C links against this library unchanged.  Entry points named rp_hip_*
 * are new; each comment names the reference code it stands in for.
 */
#ifndef RP_HIP_H
#define RP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes: identical to the reference's DType (core/tensor.h:7-13). */
enum {
    RP_DTYPE_FLOAT32 = 0,
    RP_DTYPE_FLOAT64 = 1,
    RP_DTYPE_FLOAT16 = 2,
    RP_DTYPE_BFLOAT16 = 3
};

/* ------------------------------------------------------------------------
 * Device runtime shim.  Replaces the direct CUDA runtime calls the
 * reference's host C makes (cudaGetDeviceCount core/tensor.c:14; cudaSetDevice
 * e.g. functional/functional.c:1004; cudaMalloc + cudaMemset
 * core/tensor_device.cu:44-46; cudaFree core/tensor_device.cu:273-281;
 * cudaMemcpy H2D/D2H/D2D core/tensor_device.cu:295-531; the error text and
 * device synchronisation of core/cuda_helpers.cu:6-26).
 * ---------------------------------------------------------------------- */
int rp_hip_device_count(int* count);
int rp_hip_set_device(int device_id);
int rp_hip_get_device(int* device_id);
/* Allocations come from a per-device caching pool (freed blocks are kept and
 * handed out again, so a steady-state training step performs no hipMalloc).
 * Blocks are reused in stream order on one stream; a caller that uses several
 * streams must synchronise before freeing.  RP_HIP_NO_CACHE=1 in the
 * environment turns the pool off. */
int rp_hip_malloc(void** ptr, size_t bytes);
int rp_hip_free(void* ptr);
int rp_hip_empty_cache(void);
/* Allocator counters of the process (no counterpart in the reference, which calls cudaMalloc / cudaFree directly):
 * calls to rp_hip_malloc so far, how many of them reached hipMalloc, blocks handed out and not yet freed, blocks
 * cached for reuse.  Any pointer may be NULL.  A caller that must not allocate (a serving loop, a graph recording)
 * checks that the first two stand still across the calls it makes. */
int rp_hip_memory_stats(long long* malloc_requests, long long* device_mallocs, long long* live_blocks, long long* cached_blocks);
int rp_hip_memset(void* ptr, int value, size_t bytes);
int rp_hip_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes);
int rp_hip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes);
int rp_hip_memcpy_d2d(void* dst_device, const void* src_device, size_t bytes);
int rp_hip_synchronize(void);
const char* rp_hip_last_error(void);
/* Stream the calling thread's launches go to; stream is a hipStream_t (NULL = null stream). */
int rp_hip_set_stream(void* stream);
void* rp_hip_get_stream(void);
/* Streams (default priority, non-blocking) and the current stream's completion. */
int rp_hip_stream_create(void** stream);
int rp_hip_stream_destroy(void* stream);
int rp_hip_stream_synchronize(void);
/* HIP graphs: record what the calling thread enqueues on its current (created) stream between
 * begin and end, then replay it with one launch.  The library's entry points only launch kernels
 * (clears are fill kernels, never memset nodes), so recorded sequences replay exactly; run the
 * sequence once before capturing so that the allocation pool already holds every block it needs,
 * and keep host-blocking copies outside.  No counterpart in the reference, whose ops synchronise
 * the device after every launch (core/cuda_helpers.cu:14-26). */
int rp_hip_graph_capture_begin(void);
int rp_hip_graph_capture_end(void** graph_exec);
int rp_hip_graph_launch(void* graph_exec);
int rp_hip_graph_destroy(void* graph_exec);
/* HIP events on the current stream, for timing from hosts that have no HIP binding. */
int rp_hip_event_create(void** event);
int rp_hip_event_record(void* event);
int rp_hip_event_synchronize(void* event);
int rp_hip_event_elapsed_ms(float* ms, void* start, void* stop);
int rp_hip_event_destroy(void* event);

/* ------------------------------------------------------------------------
 * GEMM.
 * ---------------------------------------------------------------------- */

/* Dense row-major C[m,n] = A[m,k] · B[k,n], C fully overwritten.
 * Same name, arguments and meaning as the reference's cuBLAS-backed seam
 * (functional/functional.h:426, functional/functional_device.cu:991-1071),
 * which rp_matmul calls after selecting the device
 * (functional/functional.c:1004-1005). */
int matmul_kernel_device(void* C, const void* A, const void* B, int m, int k, int n, int dtype);

/* Strided, batched generalisation of the seam with the Linear epilogue:
 *
 *   for z in [0,batch):  C_z = A_z · B_z  (+ bias[j] on every row)  (+ previous C_z)
 *
 * X_z[i,j] lives at X + z*x_bs + i*x_rs + j*x_cs (strides in ELEMENTS, any
 * sign-free combination: transposed and permuted views are passed as they
 * are and are never copied; the batch strides x_bs alone may also be
 * negative, so that one call can cover separately allocated matrices of one
 * shape: pass matrix 0 and the distances to matrix 1).  Output matrices must
 * not overlap.  bias is NULL or a dense vector of n elements.
 * accumulate != 0 adds the product into the existing C (beta = 1).
 * fp16/bf16 accumulate in fp32 and narrow once per reference op in the chain
 * (matmul, then bias add, then accumulation), with the reference's rounding.
 *
 * Stands in for: ensure_contiguous + rp_matmul in op_matmul
 * (ops/ops.c:6830-6838); rp_transpose + rp_contiguous + rp_matmul + rp_add in
 * backward_matmul_fn (ops/ops.c:6770-6811); the broadcasting op_add that
 * Linear.forward issues after the matmul (recpulse/module.py:110-114,
 * ops/ops.c:129-210).  The reference has no batched matmul (op_matmul is 2-D
 * only, ops/ops.c:6818); batch > 1 equals a loop of 2-D calls. */
int rp_hip_gemm_strided_batched(void* C, const void* A, const void* B, const void* bias,
                                int batch, int m, int k, int n,
                                long long a_bs, long long a_rs, long long a_cs,
                                long long b_bs, long long b_rs, long long b_cs,
                                long long c_bs, long long c_rs, long long c_cs,
                                int accumulate, int dtype);

/* The same product from a caller that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Arguments, results and errors are those
 * of rp_hip_gemm_strided_batched, bit for bit; the difference is that the split-k kernels take their partial sums and
 * arrival counters from a fixed device array of RP_HIP_NOALLOC_WORKSPACE_BYTES (+ 4 KiB) that every GPU the library
 * runs on holds until the process ends, and that no hipMalloc, hipFree or pool call is made.  A shape whose split-k
 * workspace would exceed the array returns -1 with a message that names both sizes.  All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (different streams or threads) race on it and must be serialised
 * by the caller.  The first call on a device resolves the array's address and should be made outside a recording. */
#define RP_HIP_NOALLOC_WORKSPACE_BYTES 16777216 /* 16 MiB */
int rp_hip_gemm_strided_batched_noalloc(void* C, const void* A, const void* B, const void* bias,
                                        int batch, int m, int k, int n,
                                        long long a_bs, long long a_rs, long long a_cs,
                                        long long b_bs, long long b_rs, long long b_cs,
                                        long long c_bs, long long c_rs, long long c_cs,
                                        int accumulate, int dtype);

/* Name of the kernel family the dispatcher picks for a problem, for logs and
 * tests ("mfma16_256x256", "skinny", "generic", ...).  No device work. */
const char* rp_hip_gemm_kernel_name(int batch, int m, int k, int n,
                                    long long a_rs, long long a_cs,
                                    long long b_rs, long long b_cs,
                                    long long c_rs, long long c_cs, int dtype);
/* Name of the kernel family and tile that the calling thread's most recent GEMM entry-point call dispatched ("none"
 * before the first): unlike rp_hip_gemm_kernel_name it reflects the bias, the accumulate flag and the pointers of that
 * call.  No counterpart in the reference (whose device GEMM is one cuBLAS call). */
const char* rp_hip_last_gemm_kernel(void);

/* ------------------------------------------------------------------------
 * The other device entry points the benchmark configurations touch.  Names and
 * arguments are the reference's (functional/functional.h:363-428,
 * ops/ops.h backwards_*_device declarations).
 * ---------------------------------------------------------------------- */
/* functional/functional_device.cu:94-246 */
int add_kernel_device(void* out, const void* x1, const void* x2, size_t size, int dtype);
/* functional/functional_device.cu:248-330: out is dense row-major of out_shape;
 * operands are indexed with per-dimension element strides (0 = broadcast). */
int add_strided_kernel_device(void* out, const void* x1, const void* x2, int ndim, const int* out_shape,
                              const int* x1_strides, const int* x2_strides, size_t out_size, int dtype);
/* functional/functional_device.cu:333-389: scalar points to HOST memory holding
 * a double for float64 and a float for every other dtype. */
int mul_scalar_kernel_device(void* out, const void* x, const void* scalar, size_t size, int dtype);
/* functional/functional_device.cu:495-523 */
int relu_kernel_device(void* out, const void* x, size_t size, int dtype);
/* ops/grad_device.cu:523-555 */
int backwards_relu_device(const void* grad_c, const void* x, void* grad_x, size_t size, int dtype);
/* functional/functional_device.cu:1486-1565: tensor viewed as [outer, dim, inner] */
int softmax_kernel_device(void* out, const void* x, size_t outer_size, size_t dim_size, size_t inner_size, int dtype);
int log_softmax_kernel_device(void* out, const void* x, size_t outer_size, size_t dim_size, size_t inner_size, int dtype);
/* ops/grad_device.cu:1236-1291 */
int backwards_softmax_device(const void* grad_c, const void* softmax_out, void* grad_x,
                             size_t outer_size, size_t dim_size, size_t inner_size, int dtype);
/* softmax(x * scalar) and its gradient in one pass each, with the roundings of the two reference ops they stand for
 * (mul_scalar_kernel_device then softmax_kernel_device, functional/functional.h:380,404; their gradients in reverse
 * order): bit for bit what the two launches leave, without writing or re-reading the scaled tensor.  scalar: float*
 * for every dtype but float64 (double*), as for mul_scalar_kernel_device.  out may not alias x. */
int rp_hip_scaled_softmax(void* out, const void* x, const void* scalar, size_t outer_size, size_t dim_size, size_t inner_size, int dtype);
int rp_hip_backwards_scaled_softmax(const void* grad_c, const void* softmax_out, void* grad_x, const void* scalar,
                                    size_t outer_size, size_t dim_size, size_t inner_size, int dtype);
/* mul_scalar_kernel_device whose launch may be postponed until the calling thread's next call into this library (any
 * call: launches, copies, synchronisation, freeing one of the two buffers), which then runs it first, so later work
 * sees the product as if it had been launched at once.  A host layer that learns, at that next call, that the product
 * will never be read (an eager API cannot know it earlier) takes the record back with rp_hip_take_deferred(out, &x,
 * &scalar) (1 and the source and scalar when a multiply into `out` was still pending, 0 otherwise) and passes them
 * to rp_hip_scaled_softmax instead.  One record per thread.  No counterpart in the reference, whose ops launch at once. */
int rp_hip_mul_scalar_deferred(void* out, const void* x, const void* scalar, size_t size, int dtype);
int rp_hip_take_deferred(const void* out, const void** x, double* scalar);
/* ops/ops.h:260, ops/grad_device.cu:1256-1310 (values of ops/grad_host.c:1428-1500): grad_x = grad_c - exp(y) * sum over
 * the axis of grad_c, with y the output of log_softmax; the gradient of op_log_softmax (ops/ops.c:5693-5719). */
int backwards_log_softmax_device(const void* grad_c, const void* log_softmax_out, void* grad_x,
                                 size_t outer_size, size_t dim_size, size_t inner_size, int dtype);
/* functional/functional_device.cu:1197-1266: gather a strided view (element strides) into dense memory */
int contiguous_copy_kernel_device(void* out, const void* in, int ndim, int* shape, int* strides, size_t size, int dtype);
/* functional/functional_device.cu:756-989: out is a one-element device buffer */
int sum_all_kernel_device(void* out, const void* x, size_t size, int dtype);
int mean_all_kernel_device(void* out, const void* x, size_t size, int dtype);
/* functional/functional_device.cu:1348-1484: reduce the middle axis of [outer, dim, inner] */
int sum_dim_kernel_device(void* out, const void* x, size_t outer_size, size_t dim_size, size_t inner_size, int dtype);

/* core/tensor_device.cu:66-114 (fill_value_kernel, copy_value_kernel<Src,Dst>) */
int rp_hip_fill(void* ptr, double value, size_t size, int dtype);
/* ptr[i] = scalar_dev[0] * scale (product in double, narrowed once): the gradient of sum_all / mean_all
 * (backward_sum_all_fn / backward_mean_all_fn, ops/ops.c:2059-2110: a fill with grad_output or grad_output / size) with grad_output read where it
 * lives instead of on the host */
int rp_hip_fill_scaled(void* ptr, const void* scalar_dev, double scale, size_t size, int dtype);
int rp_hip_convert(void* dst, int dst_dtype, const void* src, int src_dtype, size_t size);

/* The backward of y = x . w + b for 2-D operands in one call: dx [m, k] = dy . w^T, dw [k, n] = x^T . dy,
 * db [n] = column sums of dy (rows added top to bottom, as rp_hip_reduce_rows).  dy [m, n] is dense; x [m, k], w [k, n],
 * dx and dw carry (row, column) strides in elements; any of dx, dw, db may be NULL; accumulate_* = 1 adds to what the
 * output holds.  Same values, bit for bit, as two rp_hip_gemm_strided_batched calls with the transposes as swapped
 * strides (backward_matmul_fn, ops/ops.c:6759-6814) and rp_hip_reduce_rows; for small float32 layers (the
 * one-launch 16 x 16-tile kernel's range) the three run as ONE launch, which is most of such a layer's time. */
int rp_hip_linear_backward(void* dx, void* dw, void* db, const void* dy, const void* x, const void* w, int m, int k, int n,
                           long long x_rs, long long x_cs, long long w_rs, long long w_cs,
                           long long dx_rs, long long dx_cs, long long dw_rs, long long dw_cs,
                           int accumulate_dx, int accumulate_dw, int accumulate_db, int dtype);

/* Bias gradient of Linear on the device: grad [rows, cols] dense -> out [cols],
 * each column summed top to bottom in fp32 (fp64 for float64).  Stands in for
 * the device->host->device round trip of reduce_grad_to_shape
 * (ops/ops.c:6970-7101) in the [rows, cols] -> [cols] case. */
int rp_hip_reduce_rows(void* out, const void* grad, int rows, int cols, int accumulate, int dtype);

/* Mean cross-entropy on logits [batch, classes] (float32 / float64) on the
 * device.  targets: device int32[batch], range-checked by the caller (the
 * reference checks them on the host, ops/ops.c:5547-5549; an out-of-range
 * index here yields a NaN loss, never an out-of-bounds read).  loss_out: one
 * element of dtype.
 * grad_logits (may be NULL): (softmax - onehot) * (1/batch) * upstream.
 * Stands in for op_cross_entropy_loss / backward_cross_entropy_loss_fn, which
 * run the NLL sum and the whole backward on the host (ops/ops.c:5318-5352,
 * 5412-5543, 5545-5643). */
int rp_hip_cross_entropy_mean(void* loss_out, void* grad_logits, const void* logits, const int* targets,
                              int batch, int classes, double upstream, int dtype);

/* The grad_logits half of rp_hip_cross_entropy_mean with the upstream factor read from one device element of
 * dtype (the gradient of the loss as autograd holds it), so that the backward pass never waits on a
 * device-to-host copy (the reference reads it on the host, ops/ops.c:5412-5543). */
int rp_hip_cross_entropy_backward(void* grad_logits, const void* logits, const int* targets, int batch, int classes,
                                  const void* upstream_dev, int dtype);

/* Cross-entropy with every reduction (0 none, 1 mean, 2 sum: ops/ops.h:109-111) on logits (from_logits != 0:
 * log_softmax + softmax inside) or on probabilities (from_logits == 0: log(x), as op_cross_entropy_loss does when its
 * input came out of op_softmax, ops/ops.c:5553-5585).  x [batch, classes], float32 / float64; targets: device
 * int32[batch].  loss_out: batch elements for 'none', one otherwise (the NLL terms summed in batch order in double,
 * ops/ops.c:5342-5352). */
int rp_hip_cross_entropy_forward(void* loss_out, const void* x, const int* targets, int batch, int classes,
                                 int reduction, int from_logits, int dtype);
/* Its gradient (backward_cross_entropy_loss_fn, ops/ops.c:5412-5543, which the reference builds on the host):
 * softmax - onehot, or -1 / p at the target for probabilities; times 1 / batch for 'mean'; times the upstream
 * gradient read on the device (batch elements for 'none', one otherwise). */
int rp_hip_cross_entropy_grad(void* grad_x, const void* x, const int* targets, int batch, int classes,
                              int reduction, int from_logits, const void* upstream_dev, int dtype);

/* ---- conv2d lowering (the callers of the GEMM in op_conv2d, ops/ops.c:4723-4870 and 4473-4720) ---- */

/* Same contract as the reference's single-sample entry points (functional/functional.h:183-190,
 * functional/functional_device.cu:1723-1761): col [C_in*kH*kW, out_H*out_W] row-major from im [C_in, H, W], and
 * the adjoint, which ADDS col's entries into im (the reference zeroes im first, ops/ops.c:4541).  col2im here is a
 * gather in (kh, kw) order with one rounding, i.e. the value of the reference's host path
 * (functional/functional.c:885-912), where the reference's device kernel scatters with atomicAdd. */
int im2col_kernel_device(void* col, const void* im, int C_in, int H, int W, int kH, int kW, int stride_h, int stride_w,
                         int pad_h, int pad_w, int dilation_h, int dilation_w, int out_H, int out_W, int dtype);
int col2im_kernel_device(void* im, const void* col, int C_in, int H, int W, int kH, int kW, int stride_h, int stride_w,
                         int pad_h, int pad_w, int dilation_h, int dilation_w, int out_H, int out_W, int dtype);

/* The same for a whole batch in one launch: im [batch, C_in, H, W], col [batch, C_in*kH*kW, out_H*out_W].  This is what
 * lets op_conv2d replace the reference's per-sample loop of im2col + rp_matmul (ops/ops.c:4759-4770) with one
 * lowering and one rp_hip_gemm_strided_batched call.  accumulate = 0 overwrites im, 1 adds to it. */
int rp_hip_im2col_batched(void* col, const void* im, int batch, int C_in, int H, int W, int kH, int kW,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w,
                          int out_H, int out_W, int dtype);
int rp_hip_col2im_batched(void* im, const void* col, int batch, int C_in, int H, int W, int kH, int kW,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w,
                          int out_H, int out_W, int accumulate, int dtype);

/* Convolution without the lowered matrix, for stride 1, no dilation, odd kernels with padding (k - 1) / 2 ("same"
 * output size) when the channel count that is summed over is a multiple of 64 (bfloat16 / float16), 32 (float32)
 * or 16 (float64); rp_hip_conv2d_same_supported says whether a shape qualifies, reduced_channels 0 asks about
 * geometry and dtype alone.  x [batch, C_in, H, W], w [C_out, C_in, kH, kW], y / dy [batch, C_out, H, W], all dense.
 * The input is copied once into zero-bordered planes and the GEMM reads every tap from that copy in place; the sum
 * over taps and channels is kept in the accumulate type (fp32; fp64 for float64) and rounded once, then the bias
 * is added with its own rounding as in rp_hip_channel_bias_add.  They stand in for the per-sample
 * im2col + matmul (+ col2im) loops of op_conv2d and backward_conv2d_fn (ops/ops.c:4759-4783, 4533-4551). */
int rp_hip_conv2d_same_supported(int reduced_channels, int H, int W, int kH, int kW, int dtype);
int rp_hip_conv2d_same_forward(void* y, const void* x, const void* w, const void* bias, int batch, int C_in, int H, int W,
                               int C_out, int kH, int kW, int dtype);
int rp_hip_conv2d_same_backward_input(void* dx, const void* dy, const void* w, int batch, int C_in, int H, int W,
                                      int C_out, int kH, int kW, int dtype);
/* Both gradients from one zero-bordered copy of dy; dx or dw may be NULL (x is read only for dw, w only for dx).
 * dx needs rp_hip_conv2d_same_supported(C_out, ...); dw [C_out, C_in, kH, kW] needs
 * rp_hip_conv2d_same_supported(0, ...), i.e. only the geometry and the dtype: its reduction runs over the positions
 * of a sample (every (tap, channel) column of the GEMM is a shifted plane of the padded input), the per-sample
 * products are rounded and then summed over the batch in fp32 as in the lowered path (ops/ops.c:4575-4617). */
int rp_hip_conv2d_same_backward(void* dx, void* dw, const void* dy, const void* x, const void* w, int batch, int C_in, int H, int W,
                                int C_out, int kH, int kW, int dtype);

/* y[n, c, :] += bias[c] for y [batch, channels, hw]: the reference pulls y to the host for this loop
 * (ops/ops.c:4772-4836). */
int rp_hip_channel_bias_add(void* y, const void* bias, int batch, int channels, int hw, int dtype);

/* out[c] (+)= sum over n and hw of grad[n, c, hw], accumulated in float32 (float64 for float64): the bias gradient
 * that the reference sums on the host (ops/ops.c:4620-4716). */
int rp_hip_channel_sums(void* out, const void* grad, int batch, int channels, int hw, int accumulate, int dtype);

/* ---- LSTM / GRU cells (recpulse/module.py:255-351): the element-wise half of a step, fused ---- */

/* LSTM: gates [batch, 4*hidden] = i | f | g | o pre-activations x.W_ih + h.W_hh (two calls of
 * rp_hip_gemm_strided_batched, the second with accumulate = 1); b_ih, b_hh [4*hidden] or NULL are added here, in the
 * reference's order (recpulse/module.py:285-287); c_prev [batch, hidden] with the given row stride.
 * Writes act [batch, 4*hidden] (sigmoid / tanh of the gates, kept for the backward) and hc [batch, 2*hidden] =
 * h_next | c_next.  Replaces the reference's chunk, 3 sigmoid, 2 tanh, 3 mul and 1 add launches
 * (recpulse/module.py:289-299; ops/ops.c op_sigmoid, op_tanh, op_mul, op_add), with a rounding to the tensor dtype
 * wherever the reference materialises a tensor. */
int rp_hip_lstm_cell_forward(void* hc, void* act, const void* gates, const void* b_ih, const void* b_hh,
                             const void* c_prev, long long c_prev_row_stride, int batch, int hidden, int dtype);
/* dgates [batch, 4*hidden] and dc_prev [batch, hidden] from dhc [batch, 2*hidden] (gradient of h_next | c_next):
 * the backward functions of the same ops (ops/grad_host.c:365-400 tanh, 622-660 sigmoid; mul and add in ops/ops.c). */
int rp_hip_lstm_cell_backward(void* dgates, void* dc_prev, const void* dhc, const void* act, const void* hc,
                              const void* c_prev, long long c_prev_row_stride, int batch, int hidden, int dtype);

/* GRU: gi = x.W_ih + b_ih and gh = h.W_hh + b_hh, [batch, 3*hidden] = r | z | n; h_prev [batch, hidden] with the given
 * row stride.  Writes h_next [batch, hidden] and act [batch, 3*hidden] = r | z | n after their nonlinearities.
 * Replaces recpulse/module.py:343-351 (2 chunk, 5 add, 2 sigmoid, 1 tanh, 3 mul, 1 rsub_scalar launches). */
int rp_hip_gru_cell_forward(void* h_next, void* act, const void* gi, const void* gh, const void* h_prev,
                            long long h_prev_row_stride, int batch, int hidden, int dtype);
/* dgi, dgh [batch, 3*hidden] and the direct part dh_next * z of dh_prev [batch, hidden] (the part through gh is the
 * GEMM dgh . W_hh^T, to be accumulated onto it). */
int rp_hip_gru_cell_backward(void* dgi, void* dgh, void* dh_prev, const void* dh_next, const void* act, const void* gh,
                             const void* h_prev, long long h_prev_row_stride, int batch, int hidden, int dtype);

/* dst[sum_d idx_d * dst_strides[d]] = src[dense idx]: places the gradient of a slice inside a (zeroed) tensor of the
 * sliced shape, the device half of the reference's backward_slice_fn / backward_chunk_fn (ops/ops.c:7536-7600).
 * shape and dst_strides are host arrays of ndim <= 8 entries. */
int rp_hip_scatter_strided(void* dst, const void* src, int ndim, const int* shape, const long long* dst_strides,
                           size_t size, int dtype);

/* Fused attention forward: O[b] = softmax(scale * Q[b] * K[b]^T) * V[b], the score matrix never leaves the chip.
 * bfloat16 / float16 / float32 with d in {32, 64, 128}.  Q, O: [batch, sq, d]; K, V: [batch, sk, d];
 * d contiguous (unit stride); *_bs / *_rs are the batch and row strides in elements (multiples of 16 bytes; operands
 * 16-byte aligned).  lse (may be NULL): float32 [batch, sq], log of the row sums of exp(scale * scores), for a backward
 * pass.  No counterpart in the reference, which composes the same value from op_matmul, op_mul_scalar, op_softmax and
 * op_matmul (ops/ops.c:6816-6884, 6022-6086, 5721-5788) and rounds the scores to the tensor dtype on the way; here
 * only the probabilities of the 16-bit types are rounded (to 16 bits, nearest even), accumulation is float32. */
int rp_hip_attention_forward(void* O, const void* Q, const void* K, const void* V, float* lse,
                             int batch, int sq, int sk, int d,
                             long long q_bs, long long q_rs, long long k_bs, long long k_rs,
                             long long v_bs, long long v_rs, long long o_bs, long long o_rs,
                             double scale, int dtype);

/* Backward of rp_hip_attention_forward: dQ [batch, sq, d], dK and dV [batch, sk, d] (dense, overwritten) from the
 * forward's operands, its output O, its lse and the upstream gradient dO [batch, sq, d].  The probabilities are
 * recomputed on chip as exp(scale * q.k - lse) in two launches (dQ, then dK and dV); device memory beyond the operands is one float per query row, taken
 * from and returned to the stream-ordered pool.  Same dtype, head-dimension, stride and alignment rules as the forward.
 * No counterpart in the reference, whose autograd runs backward_matmul_fn, backward_softmax_fn, backward_mul_scalar_fn
 * and backward_matmul_fn for the same values (ops/ops.c:6759-6814, 5665-5719, 5966-6020). */
int rp_hip_attention_backward(void* dQ, void* dK, void* dV, const void* Q, const void* K, const void* V,
                              const void* O, const void* dO, const float* lse,
                              int batch, int sq, int sk, int d,
                              long long q_bs, long long q_rs, long long k_bs, long long k_rs,
                              long long v_bs, long long v_rs, long long o_bs, long long o_rs,
                              long long do_bs, long long do_rs, double scale, int dtype);

#ifdef __cplusplus
}
#endif

#endif /* RP_HIP_H */
