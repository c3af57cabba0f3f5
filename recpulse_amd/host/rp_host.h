/*
 * rp_host.h — host-side tensor / functional / autograd layer above the C ABI of
 * librp_hip.so, mirroring the reference's C interface for the matmul path
 * (same names, argument meaning and error behaviour: NULL / -1 on failure).
 *
 *   core        Tensor, Meta, DType, zeros_tensor ... free_tensor   reference core/tensor.h:7-84
 *   functional  rp_* raw-buffer ops and view constructors            reference functional/functional.h:11-239
 *   ops         op_* autograd ops, GradFn                            reference ops/ops.h:14-116
 *
 * This file includes no HIP header: every device action goes through
 * include/rp_hip.h.  Compute runs on the device only — an op on host tensors
 * returns NULL (there is no CPU compute path in this build), except the few
 * element-wise helpers parameter initialisation needs (mul_scalar, fill, dtype
 * conversion, gathers).
 */
#ifndef RP_HOST_H
#define RP_HOST_H

#include <stdbool.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    DTYPE_FLOAT32 = 0,
    DTYPE_FLOAT64 = 1,
    DTYPE_FLOAT16 = 2,
    DTYPE_BFLOAT16 = 3,
    DTYPE_PRESERVE = -1,
} DType;                                            /* reference core/tensor.h:7-13 */

typedef struct Tensor Tensor;
typedef struct GradFn GradFn;

typedef struct {
    bool is_leaf;
    bool requires_grad;
    GradFn* grad_fn;
    Tensor* grad;
} Meta;                                             /* reference core/tensor.h:18-24 */

struct Tensor {                                     /* reference core/tensor.h:27-42 */
    DType dtype;
    void* data;            /* first element of this tensor / view (already offset) */
    int ndim;
    size_t size;
    int* shape;
    int* strides;          /* in elements */
    int device_id;         /* -1 host, >= 0 GPU ordinal */
    bool owns_data;
    int refcount;
    Tensor* base_tensor;   /* root owner of a view's storage */
    Meta* metadata;
};

struct GradFn {                                     /* reference ops/ops.h:14-20 */
    void (*backward)(GradFn* self, Tensor* grad_output);
    Tensor** inputs;
    int num_inputs;
    void* saved_data;
    void (*free_saved)(void* saved_data);
    Tensor* owner;
};

size_t dtype_size(DType dtype);
const char* rp_last_error(void);
#ifdef RP_TEST_HOOKS
void rp_debug_fail_gemm_after(int n);      /* tests of the error paths: the n-th GEMM from now on fails; n <= 0 switches it off.  Only in builds with -DRP_TEST_HOOKS */
#endif

/* ---- core ---- */
bool validate_device_id(int device_id);
Tensor* zeros_tensor(DType dtype, int device_id, int ndim, int* shape, Meta* metadata);
Tensor* ones_tensor(DType dtype, int device_id, int ndim, int* shape, Meta* metadata);
Tensor* empty_tensor(DType dtype, int device_id, int ndim, const int* shape);            /* uninitialised; not in the reference */
Tensor* values_tensor(void* vals, DType vals_dtype, DType target_dtype, int source_device_id, int device_id, int ndim, int* shape, Meta* metadata);
Tensor* fill_value_tensor(double value, Tensor* tensor);
Tensor* tensor_copy(Tensor* tensor);
Tensor* tensor_to(Tensor* src, int target_device_id, DType target_dtype, bool inplace);
int tensor_copy_into(Tensor* dst, Tensor* src);                                          /* Tensor.copy_ */
int tensor_backward(Tensor* tensor);
void tensor_zero_grad(Tensor* tensor);
Tensor* tensor_retain(Tensor* tensor);
void free_tensor(Tensor* tensor);
int tensor_read_scalar(Tensor* t, double* out);                                          /* first element as double */

/* ---- functional ---- */
int rp_matmul(void* C, const void* A, const void* B, int m, int k, int n, DType dtype, int device_id);
int rp_add(void* out, const void* x1, const void* x2, size_t size, DType dtype, int device_id);
int rp_mul_scalar(void* out, const void* x, const void* scalar, size_t size, DType dtype, int device_id);
bool rp_is_contiguous(Tensor* x);
Tensor* rp_contiguous(Tensor* x);
Tensor* rp_transpose(Tensor* x, int dim0, int dim1);
Tensor* rp_permute(Tensor* x, int* dims, int ndim);
Tensor* rp_reshape(Tensor* x, int ndim, int* shape);
Tensor* rp_slice(Tensor* x, int* start, int* stop, int* step);
Tensor* rp_expand(Tensor* x, int ndim, int* shape);

/* ---- autograd ops ---- */
Tensor* op_matmul(Tensor* a, Tensor* b);                 /* 2-D as in the reference; >2-D operands are batched (extension) */
Tensor* op_linear(Tensor* x, Tensor* w, Tensor* bias);   /* x·w + bias in one launch (extension; bias may be NULL) */
Tensor* op_conv2d(Tensor* input, Tensor* weight, Tensor* bias, int stride_h, int stride_w, int pad_h, int pad_w,
                  int dilation_h, int dilation_w);                       /* reference ops/ops.h:89-91 */
Tensor* op_slice(Tensor* x, int* start, int* stop, int* step);          /* reference ops/ops.h:51 */
Tensor* op_lstm_cell(Tensor* x, Tensor* h, Tensor* c, Tensor* w_ih, Tensor* w_hh, Tensor* b_ih, Tensor* b_hh);   /* one step as one node: [B, 2H] = h_next | c_next (extension) */
Tensor* op_gru_cell(Tensor* x, Tensor* h, Tensor* w_ih, Tensor* w_hh, Tensor* b_ih, Tensor* b_hh);                /* one step as one node: h_next (extension) */
Tensor* op_attention(Tensor* q, Tensor* k, Tensor* v, double scale);   /* softmax(scale·q·kᵀ)·v in one launch (extension; 16-bit dtypes and float32) */
Tensor* op_add(Tensor* x1, Tensor* x2);
Tensor* op_relu(Tensor* x);
Tensor* op_softmax(Tensor* x, int dim);
Tensor* op_softmax_consume(Tensor* x, int dim);   /* op_softmax for a caller that states nothing will read x's values after this call (the binding: x is a temporary);
                                                     an x that is a still-unlaunched op_mul_scalar result is then never written: softmax(scale * source) in one pass */
Tensor* op_log_softmax(Tensor* x, int dim);
Tensor* op_mul_scalar(Tensor* x, double scalar);
Tensor* op_sum_all(Tensor* x);
Tensor* op_mean_all(Tensor* x);
Tensor* op_cross_entropy_loss(Tensor* input, const int* targets, int batch_size, int num_classes, int reduction, int from_logits);
Tensor* op_transpose(Tensor* x, int dim0, int dim1);
Tensor* op_permute(Tensor* x, int* dims, int ndim);
Tensor* op_reshape(Tensor* x, int ndim, int* shape);

/* ---- random (any N(0,1) / U(0,1) source satisfies Linear's initialiser) ---- */
void rp_manual_seed(unsigned long long seed);
Tensor* rp_randn(DType dtype, int device_id, int ndim, int* shape);
Tensor* rp_rand(DType dtype, int device_id, int ndim, int* shape);

#ifdef __cplusplus
}
#endif

#endif /* RP_HOST_H */
