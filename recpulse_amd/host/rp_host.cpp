// Host-side tensor, functional and autograd layer for the matmul path, written
// against the C ABI in include/rp_hip.h.  Structure follows the reference's
// three C layers (core / functional / ops) so that its Python-facing behaviour
// can be reproduced; every citation below names the reference code whose
// behaviour the function keeps.
#include "rp_host.h"

#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "../../include/rp_hip.h"

namespace {

thread_local char g_err[512] = "";
// While tensor_backward runs, the first failure of any backward function is kept here: backward functions return
// nothing, so this is how the driver learns that a gradient is missing (reference convention: tensor_backward
// returns -1 and the binding raises, python/tensor_python.c:400-414).
thread_local bool g_in_backward = false;
thread_local char g_backward_err[512] = "";

void fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    if (g_in_backward && !g_backward_err[0]) snprintf(g_backward_err, sizeof(g_backward_err), "%s", g_err[0] ? g_err : "unknown failure");
}

// a device call failed: keep the device layer's own text
int dev_fail(const char* what) {
    fail("%s: %s", what, rp_hip_last_error());
    return -1;
}

bool on_device(int device_id) {
    return device_id >= 0 && rp_hip_set_device(device_id) == 0;
}

// ---- 16-bit conversions on the host, same bit rules as the device layer ----
// (reference core/half_precision.h:20-97: exact widening, narrowing adds the first dropped bit)
float f16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, f = h & 0x3FFu, w;
    float out;
    if (e == 0) {
        if (f == 0) { w = s; memcpy(&out, &w, 4); return out; }
        out = ((float)f / 1024.0f) * (1.0f / 16384.0f);
        return s ? -out : out;
    }
    w = (e == 0x1Fu) ? (s | 0x7F800000u | (f << 13)) : (s | ((e + 112u) << 23) | (f << 13));
    memcpy(&out, &w, 4);
    return out;
}

uint16_t f32_to_f16(float x) {
    uint32_t w;
    memcpy(&w, &x, 4);
    uint32_t s = (w >> 16) & 0x8000u, e32 = (w >> 23) & 0xFFu, f = w & 0x7FFFFFu;
    int e = (int)e32 - 112;
    if (e32 == 0xFFu) return (uint16_t)(f ? (s | 0x7C00u | (f >> 13) | 1u) : (s | 0x7C00u));
    if (e <= 0) {
        if (e < -10) return (uint16_t)s;
        f |= 0x800000u;
        int sh = 14 - e;
        return (uint16_t)((s | (f >> sh)) + ((f >> (sh - 1)) & 1u));
    }
    if (e >= 0x1F) return (uint16_t)(s | 0x7C00u);
    return (uint16_t)((s | ((uint32_t)e << 10) | (f >> 13)) + ((f >> 12) & 1u));
}

float bf16_to_f32(uint16_t h) {
    uint32_t w = (uint32_t)h << 16;
    float out;
    memcpy(&out, &w, 4);
    return out;
}

uint16_t f32_to_bf16(float x) {
    uint32_t w;
    memcpy(&w, &x, 4);
    return (uint16_t)((w >> 16) + ((w >> 15) & 1u));
}

double load_as_double(const void* p, size_t i, DType dt) {
    switch (dt) {
        case DTYPE_FLOAT32: return ((const float*)p)[i];
        case DTYPE_FLOAT64: return ((const double*)p)[i];
        case DTYPE_FLOAT16: return f16_to_f32(((const uint16_t*)p)[i]);
        default: return bf16_to_f32(((const uint16_t*)p)[i]);
    }
}

// the reference converts between dtypes through an fp32 pivot (core/tensor_host.c:130-207)
void store_from_double(void* p, size_t i, DType dt, double v) {
    switch (dt) {
        case DTYPE_FLOAT32: ((float*)p)[i] = (float)v; break;
        case DTYPE_FLOAT64: ((double*)p)[i] = v; break;
        case DTYPE_FLOAT16: ((uint16_t*)p)[i] = f32_to_f16((float)v); break;
        default: ((uint16_t*)p)[i] = f32_to_bf16((float)v); break;
    }
}

void host_convert(void* dst, DType ddt, const void* src, DType sdt, size_t n) {
    if (ddt == sdt) { memcpy(dst, src, n * dtype_size(ddt)); return; }
    for (size_t i = 0; i < n; i++) {
        double v = load_as_double(src, i, sdt);
        if (ddt != DTYPE_FLOAT64 && sdt == DTYPE_FLOAT64) v = (double)(float)v;
        store_from_double(dst, i, ddt, v);
    }
}

size_t shape_size(int ndim, const int* shape) {
    size_t n = 1;
    for (int i = 0; i < ndim; i++) n *= (size_t)shape[i];
    return n;
}

Tensor* alloc_header(DType dtype, int device_id, int ndim, const int* shape) {
    if (ndim <= 0 || !shape || !dtype_size(dtype)) { fail("invalid shape or dtype"); return nullptr; }
    for (int i = 0; i < ndim; i++) if (shape[i] <= 0) { fail("shape entries must be positive"); return nullptr; }
    Tensor* t = (Tensor*)calloc(1, sizeof(Tensor));
    if (!t) return nullptr;
    t->dtype = dtype;
    t->ndim = ndim;
    t->size = shape_size(ndim, shape);
    t->shape = (int*)malloc(sizeof(int) * ndim);
    t->strides = (int*)malloc(sizeof(int) * ndim);
    memcpy(t->shape, shape, sizeof(int) * ndim);
    int s = 1;                                              // row-major strides in elements (reference core/tensor_host.c:31-35)
    for (int d = ndim - 1; d >= 0; d--) { t->strides[d] = s; s *= shape[d]; }
    t->device_id = device_id;
    t->owns_data = true;
    t->refcount = 1;
    return t;
}

void release_storage(Tensor* t) {
    if (!t->owns_data || !t->data) return;
    if (t->device_id == -1) free(t->data);
    else if (on_device(t->device_id)) rp_hip_free(t->data);
    t->data = nullptr;
}

void free_grad_fn(GradFn* gf) {
    if (!gf) return;
    for (int i = 0; i < gf->num_inputs; i++)
        if (gf->inputs[i] && gf->inputs[i] != gf->owner) free_tensor(gf->inputs[i]);        // releases what attach() retained
    free(gf->inputs);
    if (gf->saved_data) { if (gf->free_saved) gf->free_saved(gf->saved_data); else free(gf->saved_data); }
    free(gf);
}

bool needs_grad(const Tensor* t) { return t && t->metadata && t->metadata->requires_grad; }

Meta* ensure_meta(Tensor* t) {
    if (!t->metadata) t->metadata = (Meta*)calloc(1, sizeof(Meta));
    return t->metadata;
}

// Attach a GradFn to an op output; the node retains its inputs (reference ops/ops.c:11-19).
GradFn* attach(Tensor* out, void (*backward)(GradFn*, Tensor*), std::initializer_list<Tensor*> inputs) {
    Meta* m = ensure_meta(out);
    m->requires_grad = true;
    m->is_leaf = false;
    GradFn* gf = (GradFn*)calloc(1, sizeof(GradFn));
    gf->backward = backward;
    gf->num_inputs = (int)inputs.size();
    gf->inputs = (Tensor**)malloc(sizeof(Tensor*) * (gf->num_inputs ? gf->num_inputs : 1));
    int i = 0;
    for (Tensor* t : inputs) { gf->inputs[i++] = t; if (t && t != out) tensor_retain(t); }
    gf->owner = out;
    m->grad_fn = gf;
    return gf;
}

bool same_shape(const Tensor* a, const Tensor* b) {
    if (a->ndim != b->ndim) return false;
    for (int i = 0; i < a->ndim; i++) if (a->shape[i] != b->shape[i]) return false;
    return true;
}

Tensor* make_view(Tensor* x, int ndim, const int* shape, const int* strides, size_t elem_offset) {
    Tensor* v = (Tensor*)calloc(1, sizeof(Tensor));
    v->dtype = x->dtype;
    v->ndim = ndim;
    v->size = shape_size(ndim, shape);
    v->shape = (int*)malloc(sizeof(int) * ndim);
    v->strides = (int*)malloc(sizeof(int) * ndim);
    memcpy(v->shape, shape, sizeof(int) * ndim);
    memcpy(v->strides, strides, sizeof(int) * ndim);
    v->device_id = x->device_id;
    v->owns_data = false;
    v->refcount = 1;
    v->data = (char*)x->data + elem_offset * dtype_size(x->dtype);            // views point at their first element (reference functional/functional.c:1103)
    v->base_tensor = x->base_tensor ? x->base_tensor : x;                    // ... and keep the root owner alive (:1110)
    tensor_retain(v->base_tensor);
    return v;
}

// dense tensor of the same values (new reference either way), like ensure_contiguous (reference ops/ops.c:21-25)
Tensor* dense(Tensor* x) { return rp_is_contiguous(x) ? tensor_retain(x) : rp_contiguous(x); }

// ---- host (CPU) arithmetic for tensors with device_id == -1 ----
// The reference runs these on the host when a tensor lives there (functional/functional.c:978-1003, 58-74).  Results are
// those of its loops: every output element accumulates its products in the order l = 0 .. k-1, multiply then add in the
// accumulation type, no fused multiply-add (the host layer is compiled with -ffp-contract=off); 16-bit operands go
// through float32 and are narrowed once (functional/functional.c:986-1000).  The loops here are blocked over the output
// (4 rows x 64 columns of accumulators, the k loop innermost per block and vectorisable across columns), which changes
// which element is worked on when, not the order of any element's sum.
template <typename A>
void host_matmul_acc(A* C, const A* Am, const A* Bm, int m, int k, int n) {
    constexpr int RB = 4, CB = 64;
    for (int i0 = 0; i0 < m; i0 += RB) {
        const int ib = m - i0 < RB ? m - i0 : RB;
        for (int j0 = 0; j0 < n; j0 += CB) {
            const int jb = n - j0 < CB ? n - j0 : CB;
            A acc[RB][CB];
            for (int ii = 0; ii < ib; ii++) for (int jj = 0; jj < jb; jj++) acc[ii][jj] = (A)0;
            for (int l = 0; l < k; l++) {
                const A* brow = Bm + (size_t)l * n + j0;
                for (int ii = 0; ii < ib; ii++) {
                    const A a = Am[(size_t)(i0 + ii) * k + l];
                    for (int jj = 0; jj < jb; jj++) acc[ii][jj] += a * brow[jj];
                }
            }
            for (int ii = 0; ii < ib; ii++) for (int jj = 0; jj < jb; jj++) C[(size_t)(i0 + ii) * n + j0 + jj] = acc[ii][jj];
        }
    }
}

// element i of a host array as the accumulation type of its dtype (float, or double for float64), and back with one rounding
template <typename A> A host_load(const void* p, size_t i, DType dt) { return (A)load_as_double(p, i, dt); }
template <typename A> void host_store(void* p, size_t i, DType dt, A v) { store_from_double(p, i, dt, (double)v); }

// C[z] = (accumulate ? C[z] : 0) + A[z] . B[z] (+ bias) on strided host operands: each operand is gathered into a dense
// array of the accumulation type (the reference's contiguous copies and its float32 pivot in one step), multiplied, and
// the result goes through the same chain of roundings as the device epilogue: product, + bias, + old value, each rounded
// to the tensor type (ops/ops.c:6838, 162, 6785).
template <typename A>
int host_gemm_t(void* C, const void* Ap, const void* Bp, const void* bias, int batch, int m, int k, int n,
                long long a_bs, long long a_rs, long long a_cs, long long b_bs, long long b_rs, long long b_cs,
                long long c_bs, long long c_rs, long long c_cs, int accumulate, DType dt) {
    std::vector<A> a((size_t)m * k), b((size_t)k * n), c((size_t)m * n);
    for (int z = 0; z < batch; z++) {
        for (int i = 0; i < m; i++) for (int l = 0; l < k; l++) a[(size_t)i * k + l] = host_load<A>(Ap, (size_t)(z * a_bs + i * a_rs + l * a_cs), dt);
        for (int l = 0; l < k; l++) for (int j = 0; j < n; j++) b[(size_t)l * n + j] = host_load<A>(Bp, (size_t)(z * b_bs + l * b_rs + j * b_cs), dt);
        host_matmul_acc<A>(c.data(), a.data(), b.data(), m, k, n);
        for (int i = 0; i < m; i++)
            for (int j = 0; j < n; j++) {
                const size_t at = (size_t)(z * c_bs + i * c_rs + j * c_cs);
                A old = accumulate ? host_load<A>(C, at, dt) : (A)0;
                host_store<A>(C, at, dt, c[(size_t)i * n + j]);
                if (bias) host_store<A>(C, at, dt, host_load<A>(C, at, dt) + host_load<A>(bias, (size_t)j, dt));
                if (accumulate) host_store<A>(C, at, dt, old + host_load<A>(C, at, dt));
            }
    }
    return 0;
}

int host_gemm(void* C, const void* A, const void* B, const void* bias, int batch, int m, int k, int n,
              long long a_bs, long long a_rs, long long a_cs, long long b_bs, long long b_rs, long long b_cs,
              long long c_bs, long long c_rs, long long c_cs, int accumulate, DType dt) {
    if (dt == DTYPE_FLOAT64) return host_gemm_t<double>(C, A, B, bias, batch, m, k, n, a_bs, a_rs, a_cs, b_bs, b_rs, b_cs, c_bs, c_rs, c_cs, accumulate, dt);
    return host_gemm_t<float>(C, A, B, bias, batch, m, k, n, a_bs, a_rs, a_cs, b_bs, b_rs, b_cs, c_bs, c_rs, c_cs, accumulate, dt);
}

// out = x1 + x2 element by element in the accumulation type, rounded once (functional/functional_host.c, 16-bit through float32)
void host_add(void* out, const void* x1, const void* x2, size_t size, DType dt) {
    if (dt == DTYPE_FLOAT64) { for (size_t i = 0; i < size; i++) ((double*)out)[i] = ((const double*)x1)[i] + ((const double*)x2)[i]; return; }
    if (dt == DTYPE_FLOAT32) { for (size_t i = 0; i < size; i++) ((float*)out)[i] = ((const float*)x1)[i] + ((const float*)x2)[i]; return; }
    for (size_t i = 0; i < size; i++) host_store<float>(out, i, dt, host_load<float>(x1, i, dt) + host_load<float>(x2, i, dt));
}

// Accumulate rule of every backward function (reference ops/ops.c:6781-6788): the first gradient is stored,
// later ones are added in place.  `g` is consumed.
void accumulate_grad(Tensor* x, Tensor* g) {
    if (!g) { if (g_in_backward && !g_backward_err[0]) fail("a gradient could not be computed"); return; }
    Meta* m = ensure_meta(x);
    if (!m->grad) { m->grad = g; return; }
    if (m->grad->device_id >= 0) {
        if (on_device(x->device_id)) add_kernel_device(m->grad->data, m->grad->data, g->data, x->size, x->dtype);
    } else {
        Tensor* gd = dense(g);                          // (gradients are made dense before they are added, like on the device)
        if (gd && rp_is_contiguous(m->grad)) host_add(m->grad->data, m->grad->data, gd->data, x->size, x->dtype);
        free_tensor(gd);
    }
    free_tensor(g);
}

std::mt19937_64 g_rng(0x2545F4914F6CDD1Dull);

}  // namespace

extern "C" {

size_t dtype_size(DType dtype) {
    switch (dtype) {
        case DTYPE_FLOAT32: return 4;
        case DTYPE_FLOAT64: return 8;
        case DTYPE_FLOAT16: return 2;
        case DTYPE_BFLOAT16: return 2;
        default: return 0;
    }
}

const char* rp_last_error(void) { return g_err; }

// Fault injection for tests of the error paths: the n-th GEMM issued by the host layer from now on (n = 1 is the next
// one) fails before anything is launched; n <= 0 switches it off.  Nothing else reads this counter.
#ifdef RP_TEST_HOOKS
static thread_local int g_fail_gemm_in = 0;
void rp_debug_fail_gemm_after(int n) { g_fail_gemm_in = n > 0 ? n : 0; }
#endif

// ======================================================================== core
bool validate_device_id(int device_id) {              // reference core/tensor.c:10-16
    if (device_id == -1) return true;
    if (device_id < 0) return false;
    int n = 0;
    if (rp_hip_device_count(&n) != 0) return false;
    return device_id < n;
}

Tensor* empty_tensor(DType dtype, int device_id, int ndim, const int* shape) {
    if (!validate_device_id(device_id)) { fail("invalid device id %d", device_id); return nullptr; }
    Tensor* t = alloc_header(dtype, device_id, ndim, shape);
    if (!t) return nullptr;
    size_t bytes = t->size * dtype_size(dtype);
    if (device_id == -1) t->data = malloc(bytes);
    else if (!on_device(device_id) || rp_hip_malloc(&t->data, bytes) != 0) { dev_fail("device allocation"); t->data = nullptr; }
    if (!t->data) { free(t->shape); free(t->strides); free(t); return nullptr; }
    return t;
}

Tensor* fill_value_tensor(double value, Tensor* t) {
    if (!t) return nullptr;
    if (t->device_id == -1) for (size_t i = 0; i < t->size; i++) store_from_double(t->data, i, t->dtype, t->dtype == DTYPE_FLOAT64 ? value : (double)(float)value);
    else if (!on_device(t->device_id) || rp_hip_fill(t->data, value, t->size, t->dtype) != 0) { dev_fail("fill"); return nullptr; }
    return t;
}

Tensor* zeros_tensor(DType dtype, int device_id, int ndim, int* shape, Meta* metadata) {      // reference core/tensor.h:60
    Tensor* t = empty_tensor(dtype, device_id, ndim, shape);
    if (!t) return nullptr;
    if (device_id == -1) memset(t->data, 0, t->size * dtype_size(dtype));
    else if (rp_hip_memset(t->data, 0, t->size * dtype_size(dtype)) != 0) { dev_fail("memset"); free_tensor(t); return nullptr; }
    t->metadata = metadata;
    return t;
}

Tensor* ones_tensor(DType dtype, int device_id, int ndim, int* shape, Meta* metadata) {
    Tensor* t = empty_tensor(dtype, device_id, ndim, shape);
    if (!t) return nullptr;
    if (!fill_value_tensor(1.0, t)) { free_tensor(t); return nullptr; }
    t->metadata = metadata;
    return t;
}

// vals: host array of vals_dtype with shape_size(shape) elements (source_device_id must be -1 here).
Tensor* values_tensor(void* vals, DType vals_dtype, DType target_dtype, int source_device_id, int device_id, int ndim, int* shape, Meta* metadata) {
    if (!vals || source_device_id != -1) { fail("values_tensor: host source required"); return nullptr; }
    if (target_dtype == DTYPE_PRESERVE) target_dtype = vals_dtype;
    Tensor* host = empty_tensor(target_dtype, -1, ndim, shape);
    if (!host) return nullptr;
    host_convert(host->data, target_dtype, vals, vals_dtype, host->size);
    host->metadata = metadata;
    if (device_id == -1) return host;
    Tensor* dev = tensor_to(host, device_id, target_dtype, false);
    host->metadata = nullptr;
    free_tensor(host);
    if (dev) dev->metadata = metadata;
    return dev;
}

Tensor* tensor_retain(Tensor* t) {                     // reference core/tensor.c:355-360
    if (t) t->refcount++;
    return t;
}

void free_tensor(Tensor* t) {                          // reference core/tensor.c:362-379
    if (!t) return;
    if (t->refcount > 1) { t->refcount--; return; }
    if (t->metadata) {
        if (t->metadata->grad_fn) free_grad_fn(t->metadata->grad_fn);
        if (t->metadata->grad) free_tensor(t->metadata->grad);
        free(t->metadata);
    }
    release_storage(t);
    Tensor* base = t->base_tensor;
    free(t->shape);
    free(t->strides);
    free(t);
    if (base) free_tensor(base);
}

Tensor* tensor_copy(Tensor* t) { return t ? tensor_to(t, t->device_id, t->dtype, false) : nullptr; }

// Move / convert (reference core/tensor.c:82-144): a non-contiguous source is densified first, the gradient
// travels along, and inplace rebinds `src` itself to the new storage.
Tensor* tensor_to(Tensor* src, int target_device_id, DType target_dtype, bool inplace) {
    if (!src) return nullptr;
    if (target_dtype == DTYPE_PRESERVE) target_dtype = src->dtype;
    if (!validate_device_id(target_device_id)) { fail("invalid device id %d", target_device_id); return nullptr; }
    if (inplace && target_device_id == src->device_id && target_dtype == src->dtype && rp_is_contiguous(src) && src->owns_data) return src;
    Tensor* s = dense(src);
    if (!s) return nullptr;
    Tensor* out = empty_tensor(target_dtype, target_device_id, s->ndim, s->shape);
    if (!out) { free_tensor(s); return nullptr; }
    size_t n = s->size;
    int rc = 0;
    if (s->device_id == -1 && target_device_id == -1) {
        host_convert(out->data, target_dtype, s->data, s->dtype, n);
    } else if (s->device_id == -1) {                       // host -> device: convert on the host, then copy up
        void* staged = (target_dtype == s->dtype) ? s->data : malloc(n * dtype_size(target_dtype));
        if (staged != s->data) host_convert(staged, target_dtype, s->data, s->dtype, n);
        rc = on_device(target_device_id) ? rp_hip_memcpy_h2d(out->data, staged, n * dtype_size(target_dtype)) : -1;
        if (staged != s->data) free(staged);
    } else if (target_device_id == -1) {                   // device -> host: copy down, convert on the host
        void* staged = (target_dtype == s->dtype) ? out->data : malloc(n * dtype_size(s->dtype));
        rc = on_device(s->device_id) ? rp_hip_memcpy_d2h(staged, s->data, n * dtype_size(s->dtype)) : -1;
        if (rc == 0 && staged != out->data) host_convert(out->data, target_dtype, staged, s->dtype, n);
        if (staged != out->data) free(staged);
    } else if (s->device_id == target_device_id) {
        rc = on_device(target_device_id) ? (target_dtype == s->dtype ? rp_hip_memcpy_d2d(out->data, s->data, n * dtype_size(s->dtype))
                                                                     : rp_hip_convert(out->data, target_dtype, s->data, s->dtype, n)) : -1;
    } else {
        fail("tensor_to: copies between two GPUs are outside this build");
        rc = -2;
    }
    free_tensor(s);
    if (rc != 0) { if (rc == -1) dev_fail("tensor_to"); free_tensor(out); return nullptr; }
    Tensor* grad = (src->metadata && src->metadata->grad) ? tensor_to(src->metadata->grad, target_device_id, target_dtype, false) : nullptr;
    if (!inplace) {
        if (src->metadata) {
            Meta* m = ensure_meta(out);
            m->requires_grad = src->metadata->requires_grad;
            m->is_leaf = true;
            m->grad = grad;
        }
        return out;
    }
    // inplace: src keeps its identity (and metadata) and takes over the new storage
    release_storage(src);
    if (src->base_tensor) { free_tensor(src->base_tensor); src->base_tensor = nullptr; }
    free(src->shape);
    free(src->strides);
    src->shape = out->shape; src->strides = out->strides; src->data = out->data;
    src->dtype = target_dtype; src->device_id = target_device_id; src->owns_data = true;
    if (src->metadata) { if (src->metadata->grad) free_tensor(src->metadata->grad); src->metadata->grad = grad; }
    else if (grad) free_tensor(grad);
    free(out);
    return src;
}

// Tensor.copy_: overwrite dst's values with src's (same element count), converting dtype / device as needed.
int tensor_copy_into(Tensor* dst, Tensor* src) {
    if (!dst || !src || dst->size != src->size) { fail("copy_: size mismatch"); return -1; }
    if (!rp_is_contiguous(dst)) { fail("copy_: destination must be contiguous"); return -1; }
    Tensor* tmp = tensor_to(src, dst->device_id, dst->dtype, false);
    if (!tmp) return -1;
    size_t bytes = dst->size * dtype_size(dst->dtype);
    int rc = 0;
    if (dst->device_id == -1) memcpy(dst->data, tmp->data, bytes);
    else rc = on_device(dst->device_id) ? rp_hip_memcpy_d2d(dst->data, tmp->data, bytes) : -1;
    free_tensor(tmp);
    return rc == 0 ? 0 : dev_fail("copy_");
}

int tensor_read_scalar(Tensor* t, double* out) {
    if (!t || !out) return -1;
    unsigned char buf[8];
    if (t->device_id == -1) memcpy(buf, t->data, dtype_size(t->dtype));
    else if (!on_device(t->device_id) || rp_hip_memcpy_d2h(buf, t->data, dtype_size(t->dtype)) != 0) return dev_fail("read scalar");
    *out = load_as_double(buf, 0, t->dtype);
    return 0;
}

void tensor_zero_grad(Tensor* t) {                     // frees the gradient rather than zero-filling it (reference core/tensor.c:349-353)
    if (t && t->metadata && t->metadata->grad) { free_tensor(t->metadata->grad); t->metadata->grad = nullptr; }
}

// Reverse-mode driver (reference core/tensor.c:219-347): seed with ones of the root's own shape, run every
// GradFn once all of its consumers have contributed, then free the graph (it is single-use).
int tensor_backward(Tensor* root) {
    if (!root || !needs_grad(root)) { fail("backward: tensor does not require grad"); return -1; }
    if (!root->metadata->grad_fn) return 0;
    if (!root->metadata->grad) {
        root->metadata->grad = ones_tensor(root->dtype, root->device_id, root->ndim, root->shape, nullptr);
        if (!root->metadata->grad) return -1;
    }
    // post-order DFS over grad_fn inputs gives a topological order of the non-leaf tensors
    std::vector<Tensor*> order;
    std::unordered_set<Tensor*> seen;
    std::vector<std::pair<Tensor*, int>> stack{{root, 0}};
    seen.insert(root);
    while (!stack.empty()) {
        auto& [t, next] = stack.back();
        GradFn* gf = t->metadata ? t->metadata->grad_fn : nullptr;
        if (gf && next < gf->num_inputs) {
            Tensor* in = gf->inputs[next++];
            if (in && in->metadata && in->metadata->grad_fn && !seen.count(in)) { seen.insert(in); stack.push_back({in, 0}); }
        } else {
            order.push_back(t);
            stack.pop_back();
        }
    }
    g_in_backward = true;
    g_backward_err[0] = 0;
    for (auto it = order.rbegin(); it != order.rend(); ++it) {
        Tensor* t = *it;
        GradFn* gf = t->metadata->grad_fn;
        if (gf && t->metadata->grad) gf->backward(gf, t->metadata->grad);
    }
    g_in_backward = false;
    for (Tensor* t : order) {
        GradFn* gf = t->metadata->grad_fn;
        t->metadata->grad_fn = nullptr;
        free_grad_fn(gf);                                   // may drop the last reference to intermediates; `order` is not touched again
    }
    // the walk always finishes (the graph is freed either way); the first failure of a backward function decides the result
    if (g_backward_err[0]) { fail("%s", g_backward_err); return -1; }
    return 0;
}

// ================================================================== functional
int rp_matmul(void* C, const void* A, const void* B, int m, int k, int n, DType dtype, int device_id) {    // reference functional/functional.c:978-1006
    if (!C || !A || !B || m <= 0 || k <= 0 || n <= 0) return -1;
    if (device_id == -1) return host_gemm(C, A, B, nullptr, 1, m, k, n, 0, k, 1, 0, n, 1, 0, n, 1, 0, dtype);     // reference :986-1000
    if (!on_device(device_id)) return dev_fail("set device");
    return matmul_kernel_device(C, A, B, m, k, n, dtype) == 0 ? 0 : dev_fail("matmul");
}

int rp_add(void* out, const void* x1, const void* x2, size_t size, DType dtype, int device_id) {           // reference functional/functional.c:58-74
    if (!out || !x1 || !x2 || size == 0) return -1;
    if (device_id == -1) { host_add(out, x1, x2, size, dtype); return 0; }
    if (!on_device(device_id)) return dev_fail("set device");
    return add_kernel_device(out, x1, x2, size, dtype) == 0 ? 0 : dev_fail("add");
}

// scalar: float* for every dtype but float64 (double*), as in the reference (functional/functional.c:241-258).
// The host branch exists because parameter initialisation scales a host randn tensor (recpulse/module.py:97-99).
int rp_mul_scalar(void* out, const void* x, const void* scalar, size_t size, DType dtype, int device_id) {
    if (!out || !x || !scalar || size == 0) return -1;
    if (device_id == -1) {
        if (dtype == DTYPE_FLOAT64) { double s = *(const double*)scalar; for (size_t i = 0; i < size; i++) ((double*)out)[i] = ((const double*)x)[i] * s; return 0; }
        float s = *(const float*)scalar;
        for (size_t i = 0; i < size; i++) {
            float v = (float)load_as_double(x, i, dtype) * s;
            store_from_double(out, i, dtype, v);
        }
        return 0;
    }
    if (!on_device(device_id)) return dev_fail("set device");
    return mul_scalar_kernel_device(out, x, scalar, size, dtype) == 0 ? 0 : dev_fail("mul_scalar");
}

bool rp_is_contiguous(Tensor* x) {                     // reference functional/functional.c:1117-1128
    if (!x) return false;
    int expect = 1;
    for (int d = x->ndim - 1; d >= 0; d--) {
        if (x->shape[d] != 1 && x->strides[d] != expect) return false;
        expect *= x->shape[d];
    }
    return true;
}

Tensor* rp_contiguous(Tensor* x) {                     // reference functional/functional.c:1130-1220
    if (!x) return nullptr;
    Tensor* out = empty_tensor(x->dtype, x->device_id, x->ndim, x->shape);
    if (!out) return nullptr;
    if (x->device_id >= 0) {
        if (!on_device(x->device_id) || contiguous_copy_kernel_device(out->data, x->data, x->ndim, x->shape, x->strides, x->size, x->dtype) != 0) {
            dev_fail("contiguous"); free_tensor(out); return nullptr;
        }
        return out;
    }
    size_t es = dtype_size(x->dtype);
    for (size_t i = 0; i < x->size; i++) {
        size_t rem = i; long long off = 0;
        for (int d = x->ndim - 1; d >= 0; d--) { off += (long long)(rem % x->shape[d]) * x->strides[d]; rem /= x->shape[d]; }
        memcpy((char*)out->data + i * es, (const char*)x->data + off * (long long)es, es);
    }
    return out;
}

Tensor* rp_transpose(Tensor* x, int dim0, int dim1) {  // reference functional/functional.c:1340-1435
    if (!x) return nullptr;
    if (dim0 < 0) dim0 += x->ndim;
    if (dim1 < 0) dim1 += x->ndim;
    if (dim0 < 0 || dim1 < 0 || dim0 >= x->ndim || dim1 >= x->ndim) { fail("transpose: dimension out of range"); return nullptr; }
    std::vector<int> shape(x->shape, x->shape + x->ndim), strides(x->strides, x->strides + x->ndim);
    std::swap(shape[dim0], shape[dim1]);
    std::swap(strides[dim0], strides[dim1]);
    return make_view(x, x->ndim, shape.data(), strides.data(), 0);
}

Tensor* rp_permute(Tensor* x, int* dims, int ndim) {   // reference functional/functional.c:1812-1875
    if (!x || !dims || ndim != x->ndim) { fail("permute: need one entry per dimension"); return nullptr; }
    std::vector<int> shape(ndim), strides(ndim), used(ndim, 0);
    for (int i = 0; i < ndim; i++) {
        int d = dims[i] < 0 ? dims[i] + ndim : dims[i];
        if (d < 0 || d >= ndim || used[d]) { fail("permute: not a permutation"); return nullptr; }
        used[d] = 1;
        shape[i] = x->shape[d];
        strides[i] = x->strides[d];
    }
    return make_view(x, ndim, shape.data(), strides.data(), 0);
}

Tensor* rp_reshape(Tensor* x, int ndim, int* shape) {  // one -1 entry is inferred; a non-contiguous source is copied first
    if (!x || ndim <= 0 || !shape) return nullptr;
    std::vector<int> shp(shape, shape + ndim);
    long long known = 1; int infer = -1;
    for (int i = 0; i < ndim; i++) {
        if (shp[i] == -1) { if (infer >= 0) { fail("reshape: only one -1"); return nullptr; } infer = i; }
        else if (shp[i] <= 0) { fail("reshape: bad extent"); return nullptr; }
        else known *= shp[i];
    }
    if (infer >= 0) { if (known == 0 || x->size % known) { fail("reshape: cannot infer extent"); return nullptr; } shp[infer] = (int)(x->size / known); known *= shp[infer]; }
    if ((size_t)known != x->size) { fail("reshape: element count changes"); return nullptr; }
    Tensor* src = dense(x);
    if (!src) return nullptr;
    std::vector<int> strides(ndim);
    int s = 1;
    for (int d = ndim - 1; d >= 0; d--) { strides[d] = s; s *= shp[d]; }
    Tensor* v = make_view(src, ndim, shp.data(), strides.data(), 0);
    free_tensor(src);
    return v;
}

Tensor* rp_slice(Tensor* x, int* start, int* stop, int* step) {
    if (!x) return nullptr;
    std::vector<int> shape(x->ndim), strides(x->ndim);
    size_t off = 0;
    for (int d = 0; d < x->ndim; d++) {
        int b = start ? start[d] : 0, e = stop ? stop[d] : x->shape[d], st = step ? step[d] : 1;
        if (b < 0) b += x->shape[d];
        if (e < 0) e += x->shape[d];
        if (e > x->shape[d]) e = x->shape[d];
        if (st <= 0 || b < 0 || b >= e) { fail("slice: empty or invalid range in dimension %d", d); return nullptr; }
        shape[d] = (e - b + st - 1) / st;
        strides[d] = x->strides[d] * st;
        off += (size_t)b * x->strides[d];
    }
    return make_view(x, x->ndim, shape.data(), strides.data(), off);
}

Tensor* rp_expand(Tensor* x, int ndim, int* shape) {   // broadcast view: stride 0 along stretched dims (reference functional/functional.c:1931-2003)
    if (!x || ndim < x->ndim) { fail("expand: rank must not shrink"); return nullptr; }
    std::vector<int> strides(ndim);
    int lead = ndim - x->ndim;
    for (int d = 0; d < ndim; d++) {
        if (d < lead) { strides[d] = 0; continue; }
        int xs = x->shape[d - lead];
        if (xs == shape[d]) strides[d] = x->strides[d - lead];
        else if (xs == 1) strides[d] = 0;
        else { fail("expand: extent %d cannot stretch to %d", xs, shape[d]); return nullptr; }
    }
    return make_view(x, ndim, shape, strides.data(), 0);
}

// ========================================================================= ops
namespace {

bool same_place(const Tensor* a, const Tensor* b) { return a->dtype == b->dtype && a->device_id == b->device_id; }

// Describe x's last two dims as a GEMM operand and its leading dims as one batch stride.
// Returns false when the leading dims do not collapse into a single stride.
bool batch_layout(const Tensor* x, int* batch, long long* bs) {
    *batch = 1; *bs = 0;
    int lead = x->ndim - 2;
    if (lead <= 0) return true;
    long long expect = -1;
    for (int d = lead - 1; d >= 0; d--) {
        if (x->shape[d] == 1) continue;
        if (expect >= 0 && x->strides[d] != expect) return false;
        if (*batch == 1) *bs = x->strides[d];
        expect = (long long)x->strides[d] * x->shape[d];
        *batch *= x->shape[d];
    }
    return true;
}

int device_gemm(Tensor* c, Tensor* a, bool a_t, Tensor* b, bool b_t, Tensor* bias, int accumulate) {
    // a, b: tensors whose last two dims are the matrices; *_t reads them transposed (a stride swap, never a copy)
    int an = a->ndim, bn = b->ndim, cn = c->ndim;
    int m = a_t ? a->shape[an - 1] : a->shape[an - 2], k = a_t ? a->shape[an - 2] : a->shape[an - 1];
    int n = b_t ? b->shape[bn - 2] : b->shape[bn - 1];
    long long a_rs = a->strides[an - 2], a_cs = a->strides[an - 1], b_rs = b->strides[bn - 2], b_cs = b->strides[bn - 1];
    if (a_t) std::swap(a_rs, a_cs);
    if (b_t) std::swap(b_rs, b_cs);
    int ba, bb, bc; long long a_bs, b_bs, c_bs;
    if (!batch_layout(a, &ba, &a_bs) || !batch_layout(b, &bb, &b_bs) || !batch_layout(c, &bc, &c_bs)) { fail("matmul: batch dimensions must share one stride"); return -1; }
    int batch = bc;
    if ((ba != batch && ba != 1) || (bb != batch && bb != 1)) { fail("matmul: batch sizes differ"); return -1; }
    if (ba == 1) a_bs = 0;
    if (bb == 1) b_bs = 0;
    if (c->device_id == -1)
        return host_gemm(c->data, a->data, b->data, bias ? bias->data : nullptr, batch, m, k, n, a_bs, a_rs, a_cs, b_bs, b_rs, b_cs,
                         c_bs, c->strides[cn - 2], c->strides[cn - 1], accumulate, c->dtype);
    if (!on_device(c->device_id)) return dev_fail("set device");
#ifdef RP_TEST_HOOKS
    if (g_fail_gemm_in > 0 && --g_fail_gemm_in == 0) { fail("matmul: failure injected by rp_debug_fail_gemm_after"); return -1; }
#endif
    int rc = rp_hip_gemm_strided_batched(c->data, a->data, b->data, bias ? bias->data : nullptr, batch, m, k, n,
                                         a_bs, a_rs, a_cs, b_bs, b_rs, b_cs, c_bs, c->strides[cn - 2], c->strides[cn - 1], accumulate, c->dtype);
    return rc == 0 ? 0 : dev_fail("matmul");
}

// An operand as the strided GEMM entry can read it: itself when its leading dims collapse into one batch stride,
// a dense copy otherwise (the forward's rule in op_matmul).  The result is owned by the caller.
Tensor* gemm_operand(Tensor* x) {
    int bt; long long bs;
    return batch_layout(x, &bt, &bs) ? tensor_retain(x) : rp_contiguous(x);
}

// gradient of a GEMM operand: writes into a fresh tensor, or straight into the existing gradient (beta = 1).
// A failure is recorded (fail / dev_fail) and surfaces from tensor_backward.
void gemm_grad(Tensor* target, Tensor* a, bool a_t, Tensor* b, bool b_t) {
    Meta* m = ensure_meta(target);
    Tensor* aa = gemm_operand(a);
    Tensor* bb = gemm_operand(b);
    if (!aa || !bb) { fail("matmul backward: an operand could not be made dense"); free_tensor(aa); free_tensor(bb); return; }
    if (m->grad && rp_is_contiguous(m->grad)) {
        device_gemm(m->grad, aa, a_t, bb, b_t, nullptr, 1);
    } else {
        Tensor* g = empty_tensor(target->dtype, target->device_id, target->ndim, target->shape);
        if (!g) fail("matmul backward: gradient allocation failed");
        else if (device_gemm(g, aa, a_t, bb, b_t, nullptr, 0) != 0) free_tensor(g);
        else accumulate_grad(target, g);
    }
    free_tensor(aa); free_tensor(bb);
}

// Two operand gradients of equal shapes whose products agree in every stride (the input half and the recurrent half
// of a cell step with input size = hidden size) as ONE launch over a batch of two: matrix 1 of each operand is
// addressed by its distance from matrix 0, which the strided entry accepts with either sign.  Each matrix gets the
// roundings of a gemm_grad call of its own (a k split may add its fp32 partial sums in different groups).  False when
// the pair does not qualify (nothing was launched).
bool same_matrix_layout(const Tensor* p, const Tensor* q) {
    return p->ndim == 2 && q->ndim == 2 && p->dtype == q->dtype && p->device_id == q->device_id && p->shape[0] == q->shape[0] &&
           p->shape[1] == q->shape[1] && p->strides[0] == q->strides[0] && p->strides[1] == q->strides[1];
}

bool element_distance(const Tensor* from, const Tensor* to, long long* out) {
    const long long bytes = (const char*)to->data - (const char*)from->data, esz = (long long)dtype_size(from->dtype);
    if (bytes % esz) return false;
    *out = bytes / esz;
    return true;
}

bool gemm_grad_pair(Tensor* t1, Tensor* a1, Tensor* b1, Tensor* t2, Tensor* a2, Tensor* b2, bool a_t, bool b_t) {
    if (t1 == t2 || t1->device_id < 0 || !same_matrix_layout(a1, a2) || !same_matrix_layout(b1, b2) || a1->dtype != b1->dtype || a1->dtype != t1->dtype ||
        t1->ndim != 2 || t2->ndim != 2 || t1->shape[0] != t2->shape[0] || t1->shape[1] != t2->shape[1] || t1->dtype != t2->dtype ||
        a1->device_id != t1->device_id || b1->device_id != t1->device_id || t2->device_id != t1->device_id)
        return false;
    Meta* m1 = ensure_meta(t1); Meta* m2 = ensure_meta(t2);
    const bool into1 = m1->grad && rp_is_contiguous(m1->grad), into2 = m2->grad && rp_is_contiguous(m2->grad);
    if (into1 != into2 || (!into1 && (m1->grad || m2->grad))) return false;          // both accumulate in place, or both are new
    Tensor* g1 = into1 ? m1->grad : empty_tensor(t1->dtype, t1->device_id, 2, t1->shape);
    Tensor* g2 = into2 ? m2->grad : empty_tensor(t2->dtype, t2->device_id, 2, t2->shape);
    long long a_bs = 0, b_bs = 0, c_bs = 0;
    bool launched = false;
    if (g1 && g2 && g1 != g2 && element_distance(a1, a2, &a_bs) && element_distance(b1, b2, &b_bs) && element_distance(g1, g2, &c_bs) && c_bs != 0 &&
        on_device(t1->device_id)) {
        long long a_rs = a1->strides[0], a_cs = a1->strides[1], b_rs = b1->strides[0], b_cs = b1->strides[1];
        if (a_t) std::swap(a_rs, a_cs);
        if (b_t) std::swap(b_rs, b_cs);
        const int m = a_t ? a1->shape[1] : a1->shape[0], k = a_t ? a1->shape[0] : a1->shape[1], n = b_t ? b1->shape[0] : b1->shape[1];
        launched = true;
        if (rp_hip_gemm_strided_batched(g1->data, a1->data, b1->data, nullptr, 2, m, k, n, a_bs, a_rs, a_cs, b_bs, b_rs, b_cs,
                                        c_bs, g1->strides[0], g1->strides[1], into1 ? 1 : 0, t1->dtype) != 0) {
            dev_fail("matmul backward (pair)");
            if (!into1) { free_tensor(g1); free_tensor(g2); }
        } else if (!into1) {
            accumulate_grad(t1, g1);
            accumulate_grad(t2, g2);
        }
    } else if (!into1) {
        free_tensor(g1); free_tensor(g2);
    }
    return launched;
}

// dA = dC · Bᵀ and dB = Aᵀ · dC (reference ops/ops.c:6759-6814), with the transposes passed as stride views
// and accumulation done by the GEMM itself instead of rp_transpose + rp_contiguous + rp_matmul + rp_add.
void backward_matmul_fn(GradFn* self, Tensor* grad_output) {
    Tensor* a = self->inputs[0];
    Tensor* b = self->inputs[1];
    if (needs_grad(a)) {
        if (a->ndim == b->ndim || b->ndim == 2) gemm_grad(a, grad_output, false, b, true);
    }
    if (needs_grad(b)) {
        if (b->ndim == a->ndim) gemm_grad(b, a, true, grad_output, false);
        else {
            // shared 2-D weight under a batched activation: fold the batch into the rows, dB = A2dᵀ · dC2d
            Tensor* a2 = dense(a); Tensor* g2 = dense(grad_output);
            if (!a2 || !g2) { fail("matmul backward: an operand could not be made dense"); free_tensor(a2); free_tensor(g2); return; }
            int sa[2] = {(int)(a2->size / a2->shape[a2->ndim - 1]), a2->shape[a2->ndim - 1]};
            int sg[2] = {(int)(g2->size / g2->shape[g2->ndim - 1]), g2->shape[g2->ndim - 1]};
            Tensor* av = rp_reshape(a2, 2, sa); Tensor* gv = rp_reshape(g2, 2, sg);
            if (av && gv) gemm_grad(b, av, true, gv, false);
            else fail("matmul backward: operands could not be folded to two dimensions");
            free_tensor(av); free_tensor(gv); free_tensor(a2); free_tensor(g2);
        }
    }
}

// sum a gradient down to a broadcast operand's shape (reference ops/ops.c:6970-7101), on the device
Tensor* reduce_grad_to_shape(Tensor* grad, int target_ndim, const int* target_shape) {
    Tensor* g = dense(grad);
    if (!g) return nullptr;
    size_t target_size = shape_size(target_ndim, target_shape);
    if (g->device_id == -1) {
        // host tensors: the reference's loop (ops/ops.c:7027-7086): every gradient element, in row-major order, is added to
        // the target element its index folds onto, in float32 (float64 for float64), rounded once at the end
        const int lead = g->ndim - target_ndim;
        if (lead < 0) { fail("reduce_grad_to_shape: shapes do not broadcast"); free_tensor(g); return nullptr; }
        std::vector<double> acc64(g->dtype == DTYPE_FLOAT64 ? target_size : 0, 0.0);
        std::vector<float> acc32(g->dtype == DTYPE_FLOAT64 ? 0 : target_size, 0.f);
        std::vector<long long> tstride(target_ndim);
        long long st = 1;
        for (int d = target_ndim - 1; d >= 0; d--) { tstride[d] = st; st *= target_shape[d]; }
        for (size_t i = 0; i < g->size; i++) {
            size_t rem = i; long long to = 0;
            for (int d = g->ndim - 1; d >= 0; d--) {
                const long long c = (long long)(rem % g->shape[d]); rem /= g->shape[d];
                if (d >= lead && target_shape[d - lead] != 1) to += c * tstride[d - lead];
            }
            if (g->dtype == DTYPE_FLOAT64) acc64[to] += ((const double*)g->data)[i];
            else acc32[to] += host_load<float>(g->data, i, g->dtype);
        }
        Tensor* out = empty_tensor(g->dtype, -1, target_ndim, target_shape);
        for (size_t i = 0; out && i < target_size; i++) {
            if (g->dtype == DTYPE_FLOAT64) ((double*)out->data)[i] = acc64[i];
            else host_store<float>(out->data, i, g->dtype, acc32[i]);
        }
        free_tensor(g);
        return out;
    }
    // trailing-dims case (bias of Linear): grad viewed as [outer, inner], columns summed top to bottom
    bool trailing = target_ndim <= g->ndim;
    for (int d = 0; trailing && d < target_ndim; d++) trailing = target_shape[target_ndim - 1 - d] == g->shape[g->ndim - 1 - d];
    if (trailing) {
        Tensor* out = empty_tensor(g->dtype, g->device_id, target_ndim, target_shape);
        size_t rows = g->size / target_size;
        int rc = out ? (rows == 1 ? rp_hip_memcpy_d2d(out->data, g->data, g->size * dtype_size(g->dtype))
                                  : rp_hip_reduce_rows(out->data, g->data, (int)rows, (int)target_size, 0, g->dtype)) : -1;
        free_tensor(g);
        if (rc != 0) { dev_fail("bias gradient"); free_tensor(out); return nullptr; }
        return out;
    }
    // general case: sum one stretched dimension at a time
    int lead = g->ndim - target_ndim;
    Tensor* cur = g;
    for (int d = 0; d < g->ndim; d++) {
        int tgt = d < lead ? 1 : target_shape[d - lead];
        if (cur->shape[d] == tgt) continue;
        if (tgt != 1) { fail("reduce_grad_to_shape: shapes do not broadcast"); free_tensor(cur); return nullptr; }
        std::vector<int> shp(cur->shape, cur->shape + cur->ndim);
        size_t outer = 1, inner = 1;
        for (int i = 0; i < d; i++) outer *= shp[i];
        for (int i = d + 1; i < cur->ndim; i++) inner *= shp[i];
        size_t dim = shp[d];
        shp[d] = 1;
        Tensor* nxt = empty_tensor(cur->dtype, cur->device_id, cur->ndim, shp.data());
        if (!nxt || sum_dim_kernel_device(nxt->data, cur->data, outer, dim, inner, cur->dtype) != 0) { dev_fail("sum_dim"); free_tensor(nxt); free_tensor(cur); return nullptr; }
        free_tensor(cur);
        cur = nxt;
    }
    std::vector<int> tshape(target_shape, target_shape + target_ndim);
    Tensor* out = rp_reshape(cur, target_ndim, tshape.data());
    free_tensor(cur);
    return out;
}

void backward_add_fn(GradFn* self, Tensor* grad_output) {            // reference ops/ops.c:77-127
    for (int i = 0; i < 2; i++) {
        Tensor* x = self->inputs[i];
        if (!needs_grad(x)) continue;
        Tensor* g = same_shape(x, grad_output) ? tensor_copy(grad_output) : reduce_grad_to_shape(grad_output, x->ndim, x->shape);
        accumulate_grad(x, g);
    }
}

// Where a gradient of `target` is to be written: its existing dense gradient (accumulate = 1) or a fresh tensor that
// the caller hands to accumulate_grad afterwards.  Null when the target needs no gradient or the tensor could not be made.
struct GradSlot { Tensor* into; Tensor* fresh; int accumulate; };

GradSlot grad_slot(Tensor* target) {
    GradSlot s{nullptr, nullptr, 0};
    if (!target || !needs_grad(target)) return s;
    Meta* m = ensure_meta(target);
    if (m->grad && rp_is_contiguous(m->grad)) { s.into = m->grad; s.accumulate = 1; return s; }
    s.fresh = empty_tensor(target->dtype, target->device_id, target->ndim, target->shape);
    s.into = s.fresh;
    return s;
}

void backward_linear_fn(GradFn* self, Tensor* grad_output) {
    Tensor* x = self->inputs[0]; Tensor* w = self->inputs[1];
    Tensor* bias = self->num_inputs > 2 ? self->inputs[2] : nullptr;
    if (x->ndim == 2 && w->ndim == 2 && x->device_id >= 0 && on_device(x->device_id)) {
        // one call for the three gradients: a single launch for layers as small as an MLP's
        Tensor* g = dense(grad_output);
        GradSlot sx = grad_slot(x), sw = grad_slot(w), sb = grad_slot(bias);
        const int m = x->shape[0], k = x->shape[1], n = w->shape[1];
        const bool ok = g && rp_hip_linear_backward(sx.into ? sx.into->data : nullptr, sw.into ? sw.into->data : nullptr, sb.into ? sb.into->data : nullptr,
                                                    g->data, x->data, w->data, m, k, n, x->strides[0], x->strides[1], w->strides[0], w->strides[1],
                                                    k, 1, n, 1, sx.accumulate, sw.accumulate, sb.accumulate, x->dtype) == 0;
        Tensor* targets[3] = {x, w, bias};
        GradSlot* slots[3] = {&sx, &sw, &sb};
        for (int i = 0; i < 3; i++) {
            if (!slots[i]->fresh) continue;
            if (ok) accumulate_grad(targets[i], slots[i]->fresh);
            else free_tensor(slots[i]->fresh);
        }
        if (!ok) dev_fail("op_linear backward");
        free_tensor(g);
        return;
    }
    if (bias && needs_grad(bias)) accumulate_grad(bias, reduce_grad_to_shape(grad_output, bias->ndim, bias->shape));
    backward_matmul_fn(self, grad_output);
}

void backward_relu_fn(GradFn* self, Tensor* grad_output) {           // reference ops/ops.c:1590-1617
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    Tensor* xd = dense(x); Tensor* gd = dense(grad_output);
    Tensor* g = empty_tensor(x->dtype, x->device_id, x->ndim, x->shape);
    if (g && xd && gd && on_device(x->device_id) && backwards_relu_device(gd->data, xd->data, g->data, x->size, x->dtype) == 0) accumulate_grad(x, g);
    else { dev_fail("relu backward"); free_tensor(g); }
    free_tensor(xd); free_tensor(gd);
}

struct DimSaved { int dim; };

void split_dims(const Tensor* x, int dim, size_t* outer, size_t* d, size_t* inner) {
    *outer = 1; *inner = 1;
    for (int i = 0; i < dim; i++) *outer *= x->shape[i];
    for (int i = dim + 1; i < x->ndim; i++) *inner *= x->shape[i];
    *d = x->shape[dim];
}

void backward_mul_scalar_fn(GradFn* self, Tensor* grad_output);
double scalar_of(GradFn* mul_scalar_fn);

void backward_softmax_fn(GradFn* self, Tensor* grad_output) {        // reference ops/ops.c:5665-5719; y is the op's own output
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    Tensor* y = self->owner;
    int dim = ((DimSaved*)self->saved_data)->dim;
    size_t outer, d, inner;
    split_dims(y, dim, &outer, &d, &inner);
    Tensor* gd = dense(grad_output);
    // x = source * scalar that nothing but this node refers to (no other consumer, no Python object): its gradient is of
    // no use to anyone, so the source gets its own directly, rounded twice like the two reference ops, in one pass
    GradFn* xf = x->metadata->grad_fn;
    if (xf && xf->backward == backward_mul_scalar_fn && x->refcount == 1 && !x->metadata->grad && !x->metadata->is_leaf && needs_grad(xf->inputs[0])) {
        Tensor* src = xf->inputs[0];
        const double sd = scalar_of(xf);
        const float sf = (float)sd;
        Tensor* g = empty_tensor(src->dtype, src->device_id, src->ndim, src->shape);
        if (g && gd && on_device(x->device_id) &&
            rp_hip_backwards_scaled_softmax(gd->data, y->data, g->data, x->dtype == DTYPE_FLOAT64 ? (const void*)&sd : (const void*)&sf, outer, d, inner, x->dtype) == 0) accumulate_grad(src, g);
        else { dev_fail("softmax backward"); free_tensor(g); }
        free_tensor(gd);
        return;
    }
    Tensor* g = empty_tensor(x->dtype, x->device_id, x->ndim, x->shape);
    if (g && gd && on_device(x->device_id) && backwards_softmax_device(gd->data, y->data, g->data, outer, d, inner, x->dtype) == 0) accumulate_grad(x, g);
    else { dev_fail("softmax backward"); free_tensor(g); }
    free_tensor(gd);
}

void backward_log_softmax_fn(GradFn* self, Tensor* grad_output) {    // reference ops/ops.c:5693-5719; y is the op's own output
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    Tensor* y = self->owner;
    int dim = ((DimSaved*)self->saved_data)->dim;
    size_t outer, d, inner;
    split_dims(y, dim, &outer, &d, &inner);
    Tensor* gd = dense(grad_output);
    Tensor* g = empty_tensor(x->dtype, x->device_id, x->ndim, x->shape);
    if (g && gd && on_device(x->device_id) && backwards_log_softmax_device(gd->data, y->data, g->data, outer, d, inner, x->dtype) == 0) accumulate_grad(x, g);
    else { dev_fail("log_softmax backward"); free_tensor(g); }
    free_tensor(gd);
}

struct ScalarSaved { double s; };
double scalar_of(GradFn* mul_scalar_fn) { return ((ScalarSaved*)mul_scalar_fn->saved_data)->s; }

void backward_mul_scalar_fn(GradFn* self, Tensor* grad_output) {     // reference ops/ops.c:5966-6020
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    double s = ((ScalarSaved*)self->saved_data)->s;
    float sf = (float)s;
    Tensor* gd = dense(grad_output);
    Tensor* g = empty_tensor(x->dtype, x->device_id, x->ndim, x->shape);
    if (g && gd && rp_mul_scalar(g->data, gd->data, x->dtype == DTYPE_FLOAT64 ? (const void*)&s : (const void*)&sf, x->size, x->dtype, x->device_id) == 0) accumulate_grad(x, g);
    else { fail("mul_scalar backward failed: %s", rp_hip_last_error()); free_tensor(g); }
    free_tensor(gd);
}

// Backward of op_attention in two launches (rp_hip_attention_backward): the probabilities are recomputed tile by
// tile from the row-wise log-sum-exp the forward saved, so nothing of size sq x sk is allocated.  The values are those
// of the chain the reference's autograd runs for matmul -> mul_scalar -> softmax -> matmul (ops/ops.c:6759-6814,
// 5966-6020, 5665-5719): dV = P^T dO, dP = dO V^T, dS = softmax'(dP) * scale, dQ = dS K, dK = dS^T Q.
struct AttnSaved { double scale; void* lse; int device_id; };

void free_attn_saved(void* p) {
    AttnSaved* s = (AttnSaved*)p;
    if (s->lse && on_device(s->device_id)) rp_hip_free(s->lse);
    free(s);
}

void backward_attention_fn(GradFn* self, Tensor* grad_output) {
    Tensor* q = self->inputs[0]; Tensor* k = self->inputs[1]; Tensor* v = self->inputs[2];
    if (!needs_grad(q) && !needs_grad(k) && !needs_grad(v)) return;
    AttnSaved* sv = (AttnSaved*)self->saved_data;
    Tensor* o = self->owner;
    const int nd = q->ndim, sq = q->shape[nd - 2], sk = k->shape[nd - 2], d = q->shape[nd - 1];
    const int batch = (int)(q->size / ((size_t)sq * d));
    Tensor* g = dense(grad_output);
    Tensor* od = o ? dense(o) : nullptr;
    Tensor* qd = dense(q); Tensor* kd = dense(k); Tensor* vd = dense(v);        // the operands as the forward read them
    Tensor* dq = empty_tensor(q->dtype, q->device_id, nd, q->shape);
    Tensor* dk = empty_tensor(k->dtype, k->device_id, nd, k->shape);
    Tensor* dv = empty_tensor(v->dtype, v->device_id, nd, v->shape);
    const long long qs = (long long)sq * d, ks = (long long)sk * d;
    bool ok = g && od && qd && kd && vd && dq && dk && dv && on_device(q->device_id) &&
              rp_hip_attention_backward(dq->data, dk->data, dv->data, qd->data, kd->data, vd->data, od->data, g->data, (const float*)sv->lse,
                                        batch, sq, sk, d, qs, d, ks, d, ks, d, qs, d, qs, d, sv->scale, q->dtype) == 0;
    if (!ok) dev_fail("op_attention backward");
    if (ok && needs_grad(q)) accumulate_grad(q, dq); else free_tensor(dq);
    if (ok && needs_grad(k)) accumulate_grad(k, dk); else free_tensor(dk);
    if (ok && needs_grad(v)) accumulate_grad(v, dv); else free_tensor(dv);
    free_tensor(g); free_tensor(od); free_tensor(qd); free_tensor(kd); free_tensor(vd);
}

// ---- conv2d ----------------------------------------------------------------------------
// The reference lowers one sample at a time: im2col, rp_matmul, and for the gradients col2im or a densified transpose
// per sample (ops/ops.c:4759-4770, 4533-4551, 4575-4617), with the bias and its gradient done on the host.  Here a
// chunk of the batch is lowered at once and multiplied by one strided-batched GEMM whose weight operand has batch
// stride 0 and whose transposes are stride views; the chunk keeps the lowered matrix under a fixed budget.
struct ConvSaved { int sh, sw, ph, pw, dh, dw, N, C, H, W, Co, kH, kW, oH, oW; };

long long conv_col_budget() {                            // bytes of lowered activations held at a time
    const char* e = getenv("RP_CONV_COL_BYTES");         // read at every call: tests shrink it to force several chunks
    const long long v = e ? atoll(e) : 0;
    return v > 0 ? v : (2ll << 30);
}

int conv_chunk(const ConvSaved& c, size_t esz) {
    const long long per_sample = (long long)c.C * c.kH * c.kW * c.oH * c.oW * (long long)esz;
    long long n = conv_col_budget() / (per_sample > 0 ? per_sample : 1);
    return (int)(n < 1 ? 1 : (n > c.N ? c.N : n));
}

bool conv_is_pointwise(const ConvSaved& c) {              // 1x1, unit stride, no padding: the activations are the lowered matrix
    return c.kH == 1 && c.kW == 1 && c.sh == 1 && c.sw == 1 && c.ph == 0 && c.pw == 0;
}

// Stride 1, no dilation, odd kernel with padding (k - 1) / 2 and `reduced` channels in whole k slabs of
// the GEMM: the convolution (reduced = C_in) or its input gradient (reduced = C_out) reads its taps from zero-bordered
// planes and never builds the lowered matrix.  RP_CONV_NO_DIRECT=1 keeps the lowered path (read at every call).
bool conv_direct(const ConvSaved& c, DType dt, int reduced) {
    const char* e = getenv("RP_CONV_NO_DIRECT");
    if (e && e[0] == '1') return false;
    return c.sh == 1 && c.sw == 1 && c.dh == 1 && c.dw == 1 && c.kH % 2 == 1 && c.kW % 2 == 1 && c.ph == c.kH / 2 && c.pw == c.kW / 2 &&
           rp_hip_conv2d_same_supported(reduced, c.H, c.W, c.kH, c.kW, dt) == 1;
}

int conv_lower(void* col, const void* x, int nb, const ConvSaved& c, DType dt) {
    return rp_hip_im2col_batched(col, x, nb, c.C, c.H, c.W, c.kH, c.kW, c.sh, c.sw, c.ph, c.pw, c.dh, c.dw, c.oH, c.oW, dt);
}

void backward_conv2d_fn(GradFn* self, Tensor* grad_output) {         // reference ops/ops.c:4473-4720
    Tensor* x = self->inputs[0]; Tensor* w = self->inputs[1];
    Tensor* bias = self->num_inputs > 2 ? self->inputs[2] : nullptr;
    const ConvSaved& c = *(ConvSaved*)self->saved_data;
    if (!needs_grad(x) && !needs_grad(w) && !needs_grad(bias)) return;
    if (!on_device(x->device_id)) { dev_fail("op_conv2d backward"); return; }
    const DType dt = x->dtype;
    const size_t esz = dtype_size(dt);
    const int rows = c.C * c.kH * c.kW, cols = c.oH * c.oW;
    const long long x_n = (long long)c.C * c.H * c.W, y_n = (long long)c.Co * cols, col_n = (long long)rows * cols;
    const bool pointwise = conv_is_pointwise(c);
    const int chunk = conv_chunk(c, esz);
    Tensor* g = dense(grad_output);
    Tensor* xd = dense(x); Tensor* wd = dense(w);
    void* col = nullptr;
    bool ok = g && xd && wd;
    const bool direct_dx = !pointwise && conv_direct(c, dt, c.Co), direct_dw = !pointwise && conv_direct(c, dt, 0);
    if (ok && !pointwise && ((needs_grad(x) && !direct_dx) || (needs_grad(w) && !direct_dw))) ok = rp_hip_malloc(&col, (size_t)chunk * col_n * esz) == 0;
    if (ok && ((needs_grad(x) && direct_dx) || (needs_grad(w) && direct_dw))) {
        // both gradients from one zero-bordered copy of dy, no lowered matrix
        Tensor* dx = (needs_grad(x) && direct_dx) ? empty_tensor(dt, x->device_id, x->ndim, x->shape) : nullptr;
        Tensor* dw = (needs_grad(w) && direct_dw) ? empty_tensor(dt, w->device_id, w->ndim, w->shape) : nullptr;
        const bool good = (dx || dw) && rp_hip_conv2d_same_backward(dx ? dx->data : nullptr, dw ? dw->data : nullptr, g->data, xd->data, wd->data,
                                                                    c.N, c.C, c.H, c.W, c.Co, c.kH, c.kW, dt) == 0;
        if (good) { if (dx) accumulate_grad(x, dx); if (dw) accumulate_grad(w, dw); }
        else { dev_fail("op_conv2d backward (padded planes)"); free_tensor(dx); free_tensor(dw); ok = false; }
    }
    if (ok && needs_grad(x) && !direct_dx) {
        // dcol[n] = W^T . dy[n], then each input pixel gathers its taps
        Tensor* dx = empty_tensor(dt, x->device_id, x->ndim, x->shape);
        bool good = dx != nullptr;
        for (int n0 = 0; good && n0 < c.N; n0 += chunk) {
            const int nb = c.N - n0 < chunk ? c.N - n0 : chunk;
            char* dx_n = (char*)dx->data + n0 * x_n * esz;
            const char* g_n = (const char*)g->data + n0 * y_n * esz;
            good = rp_hip_gemm_strided_batched(pointwise ? (void*)dx_n : col, wd->data, g_n, nullptr, nb, rows, c.Co, cols,
                                               0, 1, rows, y_n, cols, 1, col_n, cols, 1, 0, dt) == 0 &&
                   (pointwise || rp_hip_col2im_batched(dx_n, col, nb, c.C, c.H, c.W, c.kH, c.kW, c.sh, c.sw, c.ph, c.pw, c.dh, c.dw, c.oH, c.oW, 0, dt) == 0);
        }
        if (good) accumulate_grad(x, dx); else { dev_fail("op_conv2d backward (input)"); free_tensor(dx); }
    }
    if (ok && needs_grad(w) && !direct_dw) {
        // per-sample dy[n] . col[n]^T as one batched GEMM, then the sum over the batch in the accumulate type
        Tensor* dw = empty_tensor(dt, w->device_id, w->ndim, w->shape);
        void* per_sample = nullptr;
        bool good = dw && rp_hip_malloc(&per_sample, (size_t)chunk * c.Co * rows * esz) == 0;
        for (int n0 = 0; good && n0 < c.N; n0 += chunk) {
            const int nb = c.N - n0 < chunk ? c.N - n0 : chunk;
            const char* x_nptr = (const char*)xd->data + n0 * x_n * esz;
            const char* g_n = (const char*)g->data + n0 * y_n * esz;
            good = (pointwise || conv_lower(col, x_nptr, nb, c, dt) == 0) &&
                   rp_hip_gemm_strided_batched(per_sample, g_n, pointwise ? (const void*)x_nptr : col, nullptr, nb, c.Co, cols, rows,
                                               y_n, cols, 1, col_n, 1, cols, (long long)c.Co * rows, rows, 1, 0, dt) == 0 &&
                   rp_hip_reduce_rows(dw->data, per_sample, nb, c.Co * rows, n0 > 0, dt) == 0;
        }
        if (per_sample) rp_hip_free(per_sample);
        if (good) accumulate_grad(w, dw); else { dev_fail("op_conv2d backward (weight)"); free_tensor(dw); }
    }
    if (ok && needs_grad(bias)) {
        Tensor* db = empty_tensor(dt, bias->device_id, bias->ndim, bias->shape);
        if (db && rp_hip_channel_sums(db->data, g->data, c.N, c.Co, cols, 0, dt) == 0) accumulate_grad(bias, db);
        else { dev_fail("op_conv2d backward (bias)"); free_tensor(db); }
    }
    if (col) rp_hip_free(col);
    free_tensor(g); free_tensor(xd); free_tensor(wd);
}

// ---- slice with a gradient (reference ops/ops.c op_slice, backward_slice_fn :7536-7600) ----
struct SliceSaved { int ndim; int start[8]; int step[8]; };

void backward_slice_fn(GradFn* self, Tensor* grad_output) {
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    const SliceSaved& sv = *(SliceSaved*)self->saved_data;
    // the slice's gradient, placed inside a zeroed tensor of x's shape
    Tensor* g = dense(grad_output);
    Tensor* full = zeros_tensor(x->dtype, x->device_id, x->ndim, x->shape, nullptr);
    bool ok = g && full && on_device(x->device_id);
    if (ok) {
        long long strides[8], off = 0;
        for (int d = 0; d < sv.ndim; d++) { strides[d] = (long long)full->strides[d] * sv.step[d]; off += (long long)sv.start[d] * full->strides[d]; }
        ok = rp_hip_scatter_strided((char*)full->data + off * (long long)dtype_size(x->dtype), g->data, sv.ndim, grad_output->shape, strides, g->size, x->dtype) == 0;
    }
    if (ok) accumulate_grad(x, full); else { dev_fail("slice backward"); free_tensor(full); }
    free_tensor(g);
}

// ---- LSTM / GRU cells ----------------------------------------------------------------
// One autograd node per cell step: two GEMMs into the gate pre-activations, one fused element-wise kernel, and in
// the backward one element-wise kernel followed by the four GEMMs and the bias reductions.  The reference composes a
// step from about twenty ops (recpulse/module.py:281-300, 334-351).
struct CellSaved { Tensor* act; Tensor* pre; Tensor* state; };       // activated gates; gh (GRU only); the previous c (LSTM) or h (GRU), unit column stride

void free_cell_saved(void* p) {
    CellSaved* s = (CellSaved*)p;
    free_tensor(s->act); free_tensor(s->pre); free_tensor(s->state);
    free(s);
}

Tensor* unit_columns(Tensor* x) { return x->strides[x->ndim - 1] == 1 ? tensor_retain(x) : rp_contiguous(x); }

void bias_grad(Tensor* bias, Tensor* dgates) {
    if (bias && needs_grad(bias)) accumulate_grad(bias, reduce_grad_to_shape(dgates, bias->ndim, bias->shape));
}

// The four products of a cell's backward: dx = dgi · W_ihᵀ, dh = dgh · W_hhᵀ, dW_ih = xᵀ · dgi, dW_hh = hᵀ · dgh
// (h_grad_to: the tensor that receives dh; null when the caller has already issued that product; h_operand: the
// recurrent input when it differs from h_grad_to).  The two input gradients, and the two weight gradients, go out as
// one launch each where their shapes agree.
void cell_gemm_grads(Tensor* x, Tensor* h_grad_to, Tensor* w_ih, Tensor* w_hh, Tensor* dgi, Tensor* dgh, Tensor* h_operand = nullptr) {
    Tensor* h = h_operand ? h_operand : h_grad_to;
    const bool dx = needs_grad(x), dh = h_grad_to && needs_grad(h_grad_to);
    if (!(dx && dh && gemm_grad_pair(x, dgi, w_ih, h_grad_to, dgh, w_hh, false, true))) {
        if (dx) gemm_grad(x, dgi, false, w_ih, true);
        if (dh) gemm_grad(h_grad_to, dgh, false, w_hh, true);
    }
    const bool dwi = needs_grad(w_ih), dwh = needs_grad(w_hh);
    if (!(dwi && dwh && gemm_grad_pair(w_ih, x, dgi, w_hh, h, dgh, true, false))) {
        if (dwi) gemm_grad(w_ih, x, true, dgi, false);
        if (dwh) gemm_grad(w_hh, h, true, dgh, false);
    }
}

void backward_lstm_cell_fn(GradFn* self, Tensor* grad_output) {
    Tensor* x = self->inputs[0]; Tensor* h = self->inputs[1]; Tensor* c = self->inputs[2];
    Tensor* w_ih = self->inputs[3]; Tensor* w_hh = self->inputs[4]; Tensor* b_ih = self->inputs[5]; Tensor* b_hh = self->inputs[6];
    CellSaved* sv = (CellSaved*)self->saved_data;
    Tensor* hc = self->owner;
    const int batch = x->shape[0], hidden = hc->shape[1] / 2;
    int gshape[2] = {batch, 4 * hidden}, cshape[2] = {batch, hidden};
    Tensor* dhc = dense(grad_output);
    Tensor* hcd = dense(hc);
    Tensor* dgates = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* dc = empty_tensor(x->dtype, x->device_id, 2, cshape);
    bool ok = dhc && hcd && dgates && dc && on_device(x->device_id) &&
              rp_hip_lstm_cell_backward(dgates->data, dc->data, dhc->data, sv->act->data, hcd->data, sv->state->data, sv->state->strides[0], batch, hidden, x->dtype) == 0;
    if (!ok) dev_fail("op_lstm_cell backward");
    if (ok && needs_grad(c)) { accumulate_grad(c, dc); dc = nullptr; }
    if (ok) cell_gemm_grads(x, h, w_ih, w_hh, dgates, dgates);
    if (ok) { bias_grad(b_ih, dgates); bias_grad(b_hh, dgates); }
    free_tensor(dhc); free_tensor(hcd); free_tensor(dgates); free_tensor(dc);
}

void backward_gru_cell_fn(GradFn* self, Tensor* grad_output) {
    Tensor* x = self->inputs[0]; Tensor* h = self->inputs[1];
    Tensor* w_ih = self->inputs[2]; Tensor* w_hh = self->inputs[3]; Tensor* b_ih = self->inputs[4]; Tensor* b_hh = self->inputs[5];
    CellSaved* sv = (CellSaved*)self->saved_data;
    const int batch = x->shape[0], hidden = self->owner->shape[1];
    int gshape[2] = {batch, 3 * hidden}, hshape[2] = {batch, hidden};
    Tensor* dh = dense(grad_output);
    Tensor* dgi = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* dgh = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* dh_direct = empty_tensor(x->dtype, x->device_id, 2, hshape);
    bool ok = dh && dgi && dgh && dh_direct && on_device(x->device_id) &&
              rp_hip_gru_cell_backward(dgi->data, dgh->data, dh_direct->data, dh->data, sv->act->data, sv->pre->data, sv->state->data, sv->state->strides[0],
                                       batch, hidden, x->dtype) == 0;
    if (!ok) dev_fail("op_gru_cell backward");
    if (ok && needs_grad(h)) {
        accumulate_grad(h, dh_direct); dh_direct = nullptr;           // dh * z, then the part through gh on top of it
        gemm_grad(h, dgh, false, w_hh, true);
    }
    if (ok) cell_gemm_grads(x, nullptr, w_ih, w_hh, dgi, dgh, h);
    if (ok) { bias_grad(b_ih, dgi); bias_grad(b_hh, dgh); }
    free_tensor(dh); free_tensor(dgi); free_tensor(dgh); free_tensor(dh_direct);
}

// A one-element gradient that already sits on x's device in x's dtype can be read by the kernel that uses it;
// fetching it to the host first would make every backward pass wait for the GPU to drain.
bool scalar_beside(const Tensor* s, const Tensor* x) {
    return s && s->size == 1 && s->device_id == x->device_id && s->dtype == x->dtype && on_device(x->device_id);
}

void backward_reduce_all_fn(GradFn* self, Tensor* grad_output) {     // sum_all / mean_all: every element receives g (or g / size)
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    double g0 = 0, scale = ((ScalarSaved*)self->saved_data)->s;
    Tensor* g = empty_tensor(x->dtype, x->device_id, x->ndim, x->shape);
    bool ok = g != nullptr;
    if (ok && scalar_beside(grad_output, x)) {                       // the upstream scalar never visits the host
        ok = rp_hip_fill_scaled(g->data, grad_output->data, scale, g->size, g->dtype) == 0;
        if (!ok) dev_fail("fill scaled");
    } else if (ok) ok = tensor_read_scalar(grad_output, &g0) == 0 && fill_value_tensor(g0 * scale, g);
    if (ok) accumulate_grad(x, g);
    else { if (!g_backward_err[0]) fail("sum_all / mean_all backward failed"); free_tensor(g); }
}

struct CESaved { int batch, classes; void* targets_dev; int device_id; int reduction, from_logits; };

void free_ce_saved(void* p) {
    CESaved* s = (CESaved*)p;
    if (s->targets_dev && on_device(s->device_id)) rp_hip_free(s->targets_dev);
    free(s);
}

// (softmax - onehot) / batch * upstream on the device (reference ops/ops.c:5412-5543 builds it on the host)
void backward_cross_entropy_fn(GradFn* self, Tensor* grad_output) {
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    CESaved* s = (CESaved*)self->saved_data;
    // the upstream gradient is read where it lives: one element for 'mean' / 'sum', one per row for 'none'
    Tensor* up = nullptr;
    const size_t want = s->reduction == 0 ? (size_t)s->batch : 1;
    if (grad_output->size == want && grad_output->device_id == x->device_id && grad_output->dtype == x->dtype) up = dense(grad_output);
    else if (grad_output->size == want) up = tensor_to(grad_output, x->device_id, x->dtype, false);
    Tensor* xd = dense(x);
    Tensor* g = empty_tensor(x->dtype, x->device_id, x->ndim, x->shape);
    int rc = -1;
    if (g && xd && up && on_device(x->device_id))
        rc = rp_hip_cross_entropy_grad(g->data, xd->data, (const int*)s->targets_dev, s->batch, s->classes, s->reduction, s->from_logits, up->data, x->dtype);
    if (rc == 0) accumulate_grad(x, g);
    else { if (up) dev_fail("cross-entropy backward"); else fail("cross-entropy backward: upstream gradient has the wrong size"); free_tensor(g); }
    free_tensor(xd); free_tensor(up);
}

struct PermSaved { int ndim; int dims[8]; };

void backward_permute_fn(GradFn* self, Tensor* grad_output) {        // inverse permutation of the gradient (reference ops/ops.c:7977-8014)
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    PermSaved* p = (PermSaved*)self->saved_data;
    int inv[8];
    for (int i = 0; i < p->ndim; i++) inv[p->dims[i]] = i;
    Tensor* v = rp_permute(grad_output, inv, p->ndim);
    Tensor* g = v ? rp_contiguous(v) : nullptr;
    free_tensor(v);
    accumulate_grad(x, g);
}

void backward_reshape_fn(GradFn* self, Tensor* grad_output) {
    Tensor* x = self->inputs[0];
    if (!needs_grad(x)) return;
    Tensor* gd = rp_contiguous(grad_output);
    Tensor* v = gd ? rp_reshape(gd, x->ndim, x->shape) : nullptr;
    Tensor* g = v ? rp_contiguous(v) : nullptr;
    free_tensor(v); free_tensor(gd);
    accumulate_grad(x, g);
}

Tensor* unary_device_op(Tensor* x, int (*kernel)(void*, const void*, size_t, int)) {
    if (!x) return nullptr;
    if (x->device_id == -1) { fail("this op runs on the device only; move the tensor to a GPU"); return nullptr; }
    Tensor* xd = dense(x);
    Tensor* out = xd ? empty_tensor(x->dtype, x->device_id, x->ndim, x->shape) : nullptr;
    if (!out || !on_device(x->device_id) || kernel(out->data, xd->data, x->size, x->dtype) != 0) { dev_fail("device op"); free_tensor(out); out = nullptr; }
    free_tensor(xd);
    return out;
}

}  // namespace

Tensor* op_matmul(Tensor* a, Tensor* b) {              // reference ops/ops.c:6816-6884; ndim > 2 is the batched extension
    if (!a || !b) return nullptr;
    if (a->ndim < 2 || b->ndim < 2) { fail("op_matmul: operands need at least two dimensions"); return nullptr; }
    if (!same_place(a, b)) { fail("op_matmul: dtype or device mismatch"); return nullptr; }
    if (a->shape[a->ndim - 1] != b->shape[b->ndim - 2]) { fail("op_matmul: inner dimensions differ"); return nullptr; }
    if (b->ndim > 2 && b->ndim != a->ndim) { fail("op_matmul: batched operands need equal rank"); return nullptr; }
    for (int d = 0; b->ndim > 2 && d < a->ndim - 2; d++)
        if (a->shape[d] != b->shape[d]) { fail("op_matmul: batch dimensions differ"); return nullptr; }
    std::vector<int> shape(a->shape, a->shape + a->ndim);
    shape[a->ndim - 1] = b->shape[b->ndim - 1];
    Tensor* out = empty_tensor(a->dtype, a->device_id, a->ndim, shape.data());
    if (!out) return nullptr;
    // strided operands go to the GEMM as they are; only batch dims that do not share one stride are densified
    int bt; long long bs;
    Tensor* aa = batch_layout(a, &bt, &bs) ? tensor_retain(a) : rp_contiguous(a);
    Tensor* bb = batch_layout(b, &bt, &bs) ? tensor_retain(b) : rp_contiguous(b);
    int rc = (aa && bb) ? device_gemm(out, aa, false, bb, false, nullptr, 0) : -1;
    free_tensor(aa); free_tensor(bb);
    if (rc != 0) { free_tensor(out); return nullptr; }
    if (needs_grad(a) || needs_grad(b)) attach(out, backward_matmul_fn, {a, b});
    return out;
}

Tensor* op_linear(Tensor* x, Tensor* w, Tensor* bias) {
    if (!x || !w) return nullptr;
    if (x->ndim < 2 || w->ndim != 2 || !same_place(x, w) || x->shape[x->ndim - 1] != w->shape[0]) { fail("op_linear: shape, dtype or device mismatch"); return nullptr; }
    if (bias && (bias->ndim != 1 || bias->shape[0] != w->shape[1] || !same_place(x, bias) || !rp_is_contiguous(bias))) { fail("op_linear: bias must be a dense vector of out_features"); return nullptr; }
    std::vector<int> shape(x->shape, x->shape + x->ndim);
    shape[x->ndim - 1] = w->shape[1];
    Tensor* out = empty_tensor(x->dtype, x->device_id, x->ndim, shape.data());
    if (!out) return nullptr;
    int bt; long long bs;
    Tensor* xx = batch_layout(x, &bt, &bs) ? tensor_retain(x) : rp_contiguous(x);
    int rc = xx ? device_gemm(out, xx, false, w, false, bias, 0) : -1;
    free_tensor(xx);
    if (rc != 0) { free_tensor(out); return nullptr; }
    if (needs_grad(x) || needs_grad(w) || needs_grad(bias)) {
        if (bias) attach(out, backward_linear_fn, {x, w, bias});
        else attach(out, backward_linear_fn, {x, w});
    }
    return out;
}

// O = softmax(scale · Q · Kᵀ) · V in one launch (extension; bfloat16, float16 or float32 with head dimension 32, 64 or
// 128).
// q: [..., sq, d], k and v: [..., sk, d] with equal leading dims.  Equals q.op_matmul(kᵀ).op_mul_scalar(scale)
// .op_softmax(-1).op_matmul(v) up to the roundings of the score matrix that the fused kernel does not make.
Tensor* op_attention(Tensor* q, Tensor* k, Tensor* v, double scale) {
    if (!q || !k || !v) return nullptr;
    const int nd = q->ndim;
    if (nd < 2 || k->ndim != nd || v->ndim != nd || !same_place(q, k) || !same_place(q, v)) { fail("op_attention: rank, dtype or device mismatch"); return nullptr; }
    if (q->dtype == DTYPE_FLOAT64) { fail("op_attention: bfloat16, float16 or float32 tensors"); return nullptr; }
    if (q->device_id == -1) { fail("op_attention on host tensors is not provided by this build; move the operands to a GPU"); return nullptr; }
    const int sq = q->shape[nd - 2], d = q->shape[nd - 1], sk = k->shape[nd - 2];
    bool shapes = k->shape[nd - 1] == d && v->shape[nd - 1] == d && v->shape[nd - 2] == sk;
    long long batch = 1;
    for (int i = 0; i < nd - 2; i++) { shapes = shapes && k->shape[i] == q->shape[i] && v->shape[i] == q->shape[i]; batch *= q->shape[i]; }
    if (!shapes || batch > 0x7fffffffll) { fail("op_attention: q [..., sq, d], k and v [..., sk, d] with equal leading dimensions"); return nullptr; }
    Tensor* qd = dense(q); Tensor* kd = dense(k); Tensor* vd = dense(v);
    Tensor* out = (qd && kd && vd) ? empty_tensor(q->dtype, q->device_id, nd, q->shape) : nullptr;
    const bool track = needs_grad(q) || needs_grad(k) || needs_grad(v);
    void* lse = nullptr;                                 // row-wise log-sum-exp, kept for the backward
    int rc = -1;
    if (out && on_device(q->device_id) && (!track || rp_hip_malloc(&lse, sizeof(float) * (size_t)batch * sq) == 0))
        rc = rp_hip_attention_forward(out->data, qd->data, kd->data, vd->data, (float*)lse, (int)batch, sq, sk, d,
                                      (long long)sq * d, d, (long long)sk * d, d, (long long)sk * d, d, (long long)sq * d, d, scale, q->dtype);
    if (rc != 0) { dev_fail("op_attention"); free_tensor(out); out = nullptr; if (lse) rp_hip_free(lse); lse = nullptr; }
    if (out && track) {
        GradFn* gf = attach(out, backward_attention_fn, {q, k, v});
        AttnSaved* sv = (AttnSaved*)malloc(sizeof(AttnSaved));
        sv->scale = scale; sv->lse = lse; sv->device_id = q->device_id;
        gf->saved_data = sv;
        gf->free_saved = free_attn_saved;
    }
    free_tensor(qd); free_tensor(kd); free_tensor(vd);
    return out;
}

// reference ops/ops.c:4723-4870.  input [N, C_in, H, W], weight [C_out, C_in, kH, kW], bias [C_out] or null.
Tensor* op_conv2d(Tensor* input, Tensor* weight, Tensor* bias, int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w) {
    if (!input || !weight) return nullptr;
    if (input->ndim != 4 || weight->ndim != 4 || weight->shape[1] != input->shape[1] || !same_place(input, weight)) { fail("op_conv2d: input [N, C, H, W] and weight [C_out, C, kH, kW] of one dtype and device"); return nullptr; }
    if (stride_h <= 0 || stride_w <= 0 || pad_h < 0 || pad_w < 0 || dilation_h <= 0 || dilation_w <= 0) { fail("op_conv2d: strides and dilations must be positive, paddings non-negative"); return nullptr; }
    if (bias && (bias->ndim != 1 || bias->shape[0] != weight->shape[0] || !same_place(input, bias) || !rp_is_contiguous(bias))) { fail("op_conv2d: bias must be a dense vector of C_out"); return nullptr; }
    if (input->device_id == -1) { fail("op_conv2d on host tensors is not provided by this build; move the operands to a GPU"); return nullptr; }
    ConvSaved c{stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, input->shape[0], input->shape[1], input->shape[2], input->shape[3],
                weight->shape[0], weight->shape[2], weight->shape[3], 0, 0};
    c.oH = (c.H + 2 * pad_h - dilation_h * (c.kH - 1) - 1) / stride_h + 1;
    c.oW = (c.W + 2 * pad_w - dilation_w * (c.kW - 1) - 1) / stride_w + 1;
    if (c.oH <= 0 || c.oW <= 0 || c.H + 2 * pad_h < dilation_h * (c.kH - 1) + 1 || c.W + 2 * pad_w < dilation_w * (c.kW - 1) + 1) { fail("op_conv2d: the kernel does not fit the padded input"); return nullptr; }
    const DType dt = input->dtype;
    const size_t esz = dtype_size(dt);
    const int rows = c.C * c.kH * c.kW, cols = c.oH * c.oW;
    const long long x_n = (long long)c.C * c.H * c.W, y_n = (long long)c.Co * cols, col_n = (long long)rows * cols;
    if (col_n >= (1ll << 31) || y_n >= (1ll << 31)) { fail("op_conv2d: one sample's lowered matrix exceeds 2^31 elements"); return nullptr; }
    int out_shape[4] = {c.N, c.Co, c.oH, c.oW};
    Tensor* xd = dense(input); Tensor* wd = dense(weight);
    Tensor* out = (xd && wd) ? empty_tensor(dt, input->device_id, 4, out_shape) : nullptr;
    const bool pointwise = conv_is_pointwise(c);
    const int chunk = conv_chunk(c, esz);
    void* col = nullptr;
    const bool direct = !pointwise && conv_direct(c, dt, c.C);
    bool ok = out && on_device(input->device_id) && (pointwise || direct || rp_hip_malloc(&col, (size_t)chunk * col_n * esz) == 0);
    if (ok && direct) {
        ok = rp_hip_conv2d_same_forward(out->data, xd->data, wd->data, bias ? bias->data : nullptr, c.N, c.C, c.H, c.W, c.Co, c.kH, c.kW, dt) == 0;   // adds the bias too
    }
    for (int n0 = 0; ok && !direct && n0 < c.N; n0 += chunk) {
        const int nb = c.N - n0 < chunk ? c.N - n0 : chunk;
        const char* x_nptr = (const char*)xd->data + n0 * x_n * esz;
        ok = (pointwise || conv_lower(col, x_nptr, nb, c, dt) == 0) &&
             rp_hip_gemm_strided_batched((char*)out->data + n0 * y_n * esz, wd->data, pointwise ? (const void*)x_nptr : col, nullptr, nb, c.Co, rows, cols,
                                         0, rows, 1, col_n, cols, 1, y_n, cols, 1, 0, dt) == 0;
    }
    if (ok && bias && !direct) ok = rp_hip_channel_bias_add(out->data, bias->data, c.N, c.Co, cols, dt) == 0;
    if (col) rp_hip_free(col);
    free_tensor(xd); free_tensor(wd);
    if (!ok) { dev_fail("op_conv2d"); free_tensor(out); return nullptr; }
    if (needs_grad(input) || needs_grad(weight) || needs_grad(bias)) {
        GradFn* gf = bias ? attach(out, backward_conv2d_fn, {input, weight, bias}) : attach(out, backward_conv2d_fn, {input, weight});
        ConvSaved* sv = (ConvSaved*)malloc(sizeof(ConvSaved));
        *sv = c;
        gf->saved_data = sv;
    }
    return out;
}

Tensor* op_slice(Tensor* x, int* start, int* stop, int* step) {        // reference ops/ops.h:51
    Tensor* out = rp_slice(x, start, stop, step);
    if (out && needs_grad(x)) {
        if (x->ndim > 8) { fail("op_slice: more than 8 dimensions"); free_tensor(out); return nullptr; }
        GradFn* gf = attach(out, backward_slice_fn, {x});
        SliceSaved* sv = (SliceSaved*)calloc(1, sizeof(SliceSaved));
        sv->ndim = x->ndim;
        for (int d = 0; d < x->ndim; d++) {
            int b = start ? start[d] : 0;
            sv->start[d] = b < 0 ? b + x->shape[d] : b;
            sv->step[d] = step ? step[d] : 1;
        }
        gf->saved_data = sv;
    }
    return out;
}

static bool cell_operands_ok(const char* op, Tensor* x, Tensor* h, Tensor* w_ih, Tensor* w_hh, Tensor* b_ih, Tensor* b_hh, int gates) {
    if (!x || !h || !w_ih || !w_hh) return false;
    const bool shapes = x->ndim == 2 && h->ndim == 2 && w_ih->ndim == 2 && w_hh->ndim == 2 && x->shape[0] == h->shape[0] && w_ih->shape[0] == x->shape[1] &&
                        w_hh->shape[0] == h->shape[1] && w_ih->shape[1] == gates * h->shape[1] && w_hh->shape[1] == gates * h->shape[1];
    if (!shapes || !same_place(x, h) || !same_place(x, w_ih) || !same_place(x, w_hh)) { fail("%s: x [B, I], h [B, H], w_ih [I, %dH], w_hh [H, %dH] of one dtype and device", op, gates, gates); return false; }
    if ((b_ih == nullptr) != (b_hh == nullptr)) { fail("%s: give both biases or neither", op); return false; }
    for (Tensor* b : {b_ih, b_hh})
        if (b && (b->ndim != 1 || b->shape[0] != gates * h->shape[1] || !same_place(x, b) || !rp_is_contiguous(b))) { fail("%s: biases must be dense vectors of %dH", op, gates); return false; }
    if (x->device_id == -1) { fail("%s on host tensors is not provided by this build; move the operands to a GPU", op); return false; }
    return true;
}

// One LSTM step (recpulse/module.py:281-300).  Returns hc [B, 2H] = h_next | c_next; the halves are taken with op_slice.
Tensor* op_lstm_cell(Tensor* x, Tensor* h, Tensor* c, Tensor* w_ih, Tensor* w_hh, Tensor* b_ih, Tensor* b_hh) {
    if (!cell_operands_ok("op_lstm_cell", x, h, w_ih, w_hh, b_ih, b_hh, 4)) return nullptr;
    if (!c || c->ndim != 2 || !same_shape(c, h) || !same_place(x, c)) { fail("op_lstm_cell: c must have h's shape, dtype and device"); return nullptr; }
    const int batch = x->shape[0], hidden = h->shape[1];
    int gshape[2] = {batch, 4 * hidden}, oshape[2] = {batch, 2 * hidden};
    Tensor* gates = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* act = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* hc = empty_tensor(x->dtype, x->device_id, 2, oshape);
    Tensor* cd = unit_columns(c);
    // x . W_ih, then h . W_hh on top of it (beta = 1): the reference's matmul, matmul, add as two launches
    bool ok = gates && act && hc && cd && device_gemm(gates, x, false, w_ih, false, nullptr, 0) == 0 && device_gemm(gates, h, false, w_hh, false, nullptr, 1) == 0 &&
              rp_hip_lstm_cell_forward(hc->data, act->data, gates->data, b_ih ? b_ih->data : nullptr, b_hh ? b_hh->data : nullptr, cd->data, cd->strides[0],
                                       batch, hidden, x->dtype) == 0;
    free_tensor(gates);
    if (!ok) { dev_fail("op_lstm_cell"); free_tensor(act); free_tensor(hc); free_tensor(cd); return nullptr; }
    bool track = needs_grad(x) || needs_grad(h) || needs_grad(c) || needs_grad(w_ih) || needs_grad(w_hh) || needs_grad(b_ih) || needs_grad(b_hh);
    if (track) {
        GradFn* gf = attach(hc, backward_lstm_cell_fn, {x, h, c, w_ih, w_hh, b_ih, b_hh});
        CellSaved* sv = (CellSaved*)calloc(1, sizeof(CellSaved));
        sv->act = act; sv->state = cd;
        gf->saved_data = sv;
        gf->free_saved = free_cell_saved;
    } else { free_tensor(act); free_tensor(cd); }
    return hc;
}

// One GRU step (recpulse/module.py:334-351).  Returns h_next [B, H].
Tensor* op_gru_cell(Tensor* x, Tensor* h, Tensor* w_ih, Tensor* w_hh, Tensor* b_ih, Tensor* b_hh) {
    if (!cell_operands_ok("op_gru_cell", x, h, w_ih, w_hh, b_ih, b_hh, 3)) return nullptr;
    const int batch = x->shape[0], hidden = h->shape[1];
    int gshape[2] = {batch, 3 * hidden};
    Tensor* gi = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* gh = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* act = empty_tensor(x->dtype, x->device_id, 2, gshape);
    Tensor* out = empty_tensor(x->dtype, x->device_id, 2, h->shape);
    Tensor* hd = unit_columns(h);
    bool ok = gi && gh && act && out && hd && device_gemm(gi, x, false, w_ih, false, b_ih, 0) == 0 && device_gemm(gh, h, false, w_hh, false, b_hh, 0) == 0 &&
              rp_hip_gru_cell_forward(out->data, act->data, gi->data, gh->data, hd->data, hd->strides[0], batch, hidden, x->dtype) == 0;
    free_tensor(gi);
    if (!ok) { dev_fail("op_gru_cell"); free_tensor(gh); free_tensor(act); free_tensor(out); free_tensor(hd); return nullptr; }
    bool track = needs_grad(x) || needs_grad(h) || needs_grad(w_ih) || needs_grad(w_hh) || needs_grad(b_ih) || needs_grad(b_hh);
    if (track) {
        GradFn* gf = attach(out, backward_gru_cell_fn, {x, h, w_ih, w_hh, b_ih, b_hh});
        CellSaved* sv = (CellSaved*)calloc(1, sizeof(CellSaved));
        sv->act = act; sv->pre = gh; sv->state = hd;
        gf->saved_data = sv;
        gf->free_saved = free_cell_saved;
    } else { free_tensor(act); free_tensor(gh); free_tensor(hd); }
    return out;
}

Tensor* op_add(Tensor* x1, Tensor* x2) {               // reference ops/ops.c:129-210
    if (!x1 || !x2) return nullptr;
    if (!same_place(x1, x2)) { fail("op_add: dtype or device mismatch"); return nullptr; }
    int nd = x1->ndim > x2->ndim ? x1->ndim : x2->ndim;
    if (nd > 8) { fail("op_add: more than 8 dimensions"); return nullptr; }
    std::vector<int> shape(nd);
    for (int i = 0; i < nd; i++) {                      // broadcast_shapes (reference ops/ops.c:6941-6968)
        int d1 = x1->ndim - nd + i, d2 = x2->ndim - nd + i;
        int s1 = d1 >= 0 ? x1->shape[d1] : 1, s2 = d2 >= 0 ? x2->shape[d2] : 1;
        if (s1 == s2) shape[i] = s1;
        else if (s1 == 1) shape[i] = s2;
        else if (s2 == 1) shape[i] = s1;
        else { fail("op_add: shapes do not broadcast"); return nullptr; }
    }
    Tensor* out = empty_tensor(x1->dtype, x1->device_id, nd, shape.data());
    if (!out) return nullptr;
    int rc;
    if (x1->device_id == -1) {
        // host tensors: both operands expanded to the output shape with stride-0 dimensions (functional/functional.c:1959-1966)
        // and added element by element in row-major order
        Tensor* e1 = rp_expand(x1, nd, shape.data());
        Tensor* e2 = rp_expand(x2, nd, shape.data());
        rc = (e1 && e2) ? 0 : -1;
        for (size_t i = 0; rc == 0 && i < out->size; i++) {
            size_t rem = i; long long o1 = 0, o2 = 0;
            for (int d = nd - 1; d >= 0; d--) { const long long c = (long long)(rem % shape[d]); rem /= shape[d]; o1 += c * e1->strides[d]; o2 += c * e2->strides[d]; }
            if (x1->dtype == DTYPE_FLOAT64) ((double*)out->data)[i] = ((const double*)e1->data)[o1] + ((const double*)e2->data)[o2];
            else host_store<float>(out->data, i, x1->dtype, host_load<float>(e1->data, (size_t)o1, x1->dtype) + host_load<float>(e2->data, (size_t)o2, x1->dtype));
        }
        free_tensor(e1); free_tensor(e2);
    }
    else if (!on_device(x1->device_id)) rc = -1;
    else if (same_shape(x1, x2) && rp_is_contiguous(x1) && rp_is_contiguous(x2)) rc = add_kernel_device(out->data, x1->data, x2->data, x1->size, x1->dtype);
    else {
        Tensor* e1 = rp_expand(x1, nd, shape.data());
        Tensor* e2 = rp_expand(x2, nd, shape.data());
        rc = (e1 && e2) ? add_strided_kernel_device(out->data, e1->data, e2->data, nd, shape.data(), e1->strides, e2->strides, out->size, x1->dtype) : -1;
        free_tensor(e1); free_tensor(e2);
    }
    if (rc != 0) { dev_fail("op_add"); free_tensor(out); return nullptr; }
    if (needs_grad(x1) || needs_grad(x2)) attach(out, backward_add_fn, {x1, x2});
    return out;
}

Tensor* op_relu(Tensor* x) {                           // reference ops/ops.c:2382-2431
    Tensor* out = unary_device_op(x, relu_kernel_device);
    if (out && needs_grad(x)) attach(out, backward_relu_fn, {x});
    return out;
}

static Tensor* softmax_any(Tensor* x, int dim, bool take_log, bool input_dead = false) {
    if (!x) return nullptr;
    if (dim < 0) dim += x->ndim;
    if (dim < 0 || dim >= x->ndim) { fail("softmax: dimension out of range"); return nullptr; }
    if (x->device_id == -1) { fail("softmax on host tensors is not provided by this build"); return nullptr; }
    Tensor* xd = dense(x);
    Tensor* out = xd ? empty_tensor(x->dtype, x->device_id, x->ndim, x->shape) : nullptr;
    size_t outer, d, inner;
    split_dims(x, dim, &outer, &d, &inner);
    int rc = -1;
    const void* src = nullptr;
    double sd = 1.0;
    if (out && !take_log && input_dead && xd == x && rp_hip_take_deferred(x->data, &src, &sd) == 1) {
        // x is a scalar multiple whose kernel has not been launched and whose values nobody will read: it never is
        const float sf = (float)sd;
        rc = on_device(x->device_id) ? rp_hip_scaled_softmax(out->data, src, x->dtype == DTYPE_FLOAT64 ? (const void*)&sd : (const void*)&sf, outer, d, inner, x->dtype) : -1;
    } else if (out && on_device(x->device_id)) {
        rc = take_log ? log_softmax_kernel_device(out->data, xd->data, outer, d, inner, x->dtype)
                      : softmax_kernel_device(out->data, xd->data, outer, d, inner, x->dtype);
    }
    free_tensor(xd);
    if (rc != 0) { dev_fail("softmax"); free_tensor(out); return nullptr; }
    if (needs_grad(x)) {
        GradFn* gf = attach(out, take_log ? backward_log_softmax_fn : backward_softmax_fn, {x});
        DimSaved* s = (DimSaved*)malloc(sizeof(DimSaved));
        s->dim = dim;
        gf->saved_data = s;
    }
    return out;
}

Tensor* op_softmax(Tensor* x, int dim) { return softmax_any(x, dim, false); }            // reference ops/ops.c:5721-5788
Tensor* op_softmax_consume(Tensor* x, int dim) { return softmax_any(x, dim, false, true); }
Tensor* op_log_softmax(Tensor* x, int dim) { return softmax_any(x, dim, true); }

Tensor* op_mul_scalar(Tensor* x, double scalar) {      // reference ops/ops.c:6022-6086
    if (!x) return nullptr;
    Tensor* xd = dense(x);
    Tensor* out = xd ? empty_tensor(x->dtype, x->device_id, x->ndim, x->shape) : nullptr;
    float sf = (float)scalar;                           // scalars are narrowed to float for every dtype but float64 (reference python/tensor_python.c:475-485)
    const void* sp = x->dtype == DTYPE_FLOAT64 ? (const void*)&scalar : (const void*)&sf;
    int rc = -1;
    // On the device the launch is left to the library's next call from this thread (which runs it first, whatever that
    // call is): if that call turns out to be a softmax whose caller lets the product die, the product is never written.
    if (out && x->device_id >= 0) rc = on_device(x->device_id) ? (rp_hip_mul_scalar_deferred(out->data, xd->data, sp, x->size, x->dtype) == 0 ? 0 : dev_fail("mul_scalar")) : dev_fail("set device");
    else if (out) rc = rp_mul_scalar(out->data, xd->data, sp, x->size, x->dtype, x->device_id);
    free_tensor(xd);
    if (rc != 0) { free_tensor(out); return nullptr; }
    if (needs_grad(x)) {
        GradFn* gf = attach(out, backward_mul_scalar_fn, {x});
        ScalarSaved* s = (ScalarSaved*)malloc(sizeof(ScalarSaved));
        s->s = scalar;
        gf->saved_data = s;
    }
    return out;
}

static Tensor* reduce_all(Tensor* x, bool mean) {      // result has shape [1] (reference ops/ops.c:3221-3222)
    if (!x) return nullptr;
    if (x->device_id == -1) { fail("reductions on host tensors are not provided by this build"); return nullptr; }
    Tensor* xd = dense(x);
    int one = 1;
    Tensor* out = xd ? empty_tensor(x->dtype, x->device_id, 1, &one) : nullptr;
    int rc = (out && on_device(x->device_id)) ? (mean ? mean_all_kernel_device(out->data, xd->data, x->size, x->dtype)
                                                      : sum_all_kernel_device(out->data, xd->data, x->size, x->dtype)) : -1;
    free_tensor(xd);
    if (rc != 0) { dev_fail("reduction"); free_tensor(out); return nullptr; }
    if (needs_grad(x)) {
        GradFn* gf = attach(out, backward_reduce_all_fn, {x});
        ScalarSaved* s = (ScalarSaved*)malloc(sizeof(ScalarSaved));
        s->s = mean ? 1.0 / (double)x->size : 1.0;
        gf->saved_data = s;
    }
    return out;
}

Tensor* op_sum_all(Tensor* x) { return reduce_all(x, false); }
Tensor* op_mean_all(Tensor* x) { return reduce_all(x, true); }

// reduction: 0 none, 1 mean, 2 sum as in the reference; this build provides mean on raw logits
// (reference ops/ops.c:5545-5643 with from_logits detection; out-of-range targets fail, :5547-5549).
Tensor* op_cross_entropy_loss(Tensor* input, const int* targets, int batch_size, int num_classes, int reduction, int from_logits) {
    if (!input || !targets) return nullptr;
    for (int b = 0; b < batch_size; b++) if (targets[b] < 0 || targets[b] >= num_classes) { fail("op_cross_entropy_loss: target out of range"); return nullptr; }
    if (input->ndim != 2 || input->shape[0] != batch_size || input->shape[1] != num_classes) { fail("op_cross_entropy_loss: input must be [batch, classes]"); return nullptr; }
    if (reduction < 0 || reduction > 2) { fail("op_cross_entropy_loss: reduction must be none (0), mean (1) or sum (2)"); return nullptr; }
    // -1: an input that came out of op_softmax holds probabilities, anything else logits (reference ops/ops.c:5553-5557)
    if (from_logits == -1) from_logits = !(input->metadata && input->metadata->grad_fn && input->metadata->grad_fn->backward == backward_softmax_fn);
    if (input->dtype != DTYPE_FLOAT32 && input->dtype != DTYPE_FLOAT64) { fail("op_cross_entropy_loss: float32 / float64 only"); return nullptr; }
    if (input->device_id == -1) { fail("op_cross_entropy_loss on host tensors is not provided by this build"); return nullptr; }
    if (!on_device(input->device_id)) { dev_fail("set device"); return nullptr; }
    void* tdev = nullptr;
    if (rp_hip_malloc(&tdev, sizeof(int) * batch_size) != 0 || rp_hip_memcpy_h2d(tdev, targets, sizeof(int) * batch_size) != 0) { dev_fail("targets upload"); if (tdev) rp_hip_free(tdev); return nullptr; }
    Tensor* xd = dense(input);
    int out_len = reduction == 0 ? batch_size : 1;                   // 'none' keeps one loss per row (reference ops/ops.c:5356-5360)
    Tensor* out = xd ? empty_tensor(input->dtype, input->device_id, 1, &out_len) : nullptr;
    int rc = out ? rp_hip_cross_entropy_forward(out->data, xd->data, (const int*)tdev, batch_size, num_classes, reduction, from_logits, input->dtype) : -1;
    free_tensor(xd);
    if (rc != 0) { dev_fail("cross entropy"); rp_hip_free(tdev); free_tensor(out); return nullptr; }
    if (needs_grad(input)) {
        GradFn* gf = attach(out, backward_cross_entropy_fn, {input});
        CESaved* s = (CESaved*)calloc(1, sizeof(CESaved));
        s->batch = batch_size; s->classes = num_classes; s->targets_dev = tdev; s->device_id = input->device_id;
        s->reduction = reduction; s->from_logits = from_logits;
        gf->saved_data = s;
        gf->free_saved = free_ce_saved;
    } else {
        rp_hip_free(tdev);
    }
    return out;
}

Tensor* op_transpose(Tensor* x, int dim0, int dim1) {  // reference ops/ops.c:8397-8451
    if (!x) return nullptr;
    if (dim0 < 0) dim0 += x->ndim;
    if (dim1 < 0) dim1 += x->ndim;
    Tensor* out = rp_transpose(x, dim0, dim1);
    if (out && needs_grad(x)) {
        GradFn* gf = attach(out, backward_permute_fn, {x});
        PermSaved* p = (PermSaved*)calloc(1, sizeof(PermSaved));
        p->ndim = x->ndim;
        for (int i = 0; i < x->ndim; i++) p->dims[i] = i;
        std::swap(p->dims[dim0], p->dims[dim1]);
        gf->saved_data = p;
    }
    return out;
}

Tensor* op_permute(Tensor* x, int* dims, int ndim) {   // reference ops/ops.c:8639-8697
    if (!x || ndim > 8) return nullptr;
    Tensor* out = rp_permute(x, dims, ndim);
    if (out && needs_grad(x)) {
        GradFn* gf = attach(out, backward_permute_fn, {x});
        PermSaved* p = (PermSaved*)calloc(1, sizeof(PermSaved));
        p->ndim = ndim;
        for (int i = 0; i < ndim; i++) p->dims[i] = dims[i] < 0 ? dims[i] + ndim : dims[i];
        gf->saved_data = p;
    }
    return out;
}

Tensor* op_reshape(Tensor* x, int ndim, int* shape) {
    if (!x) return nullptr;
    Tensor* out = rp_reshape(x, ndim, shape);
    if (out && needs_grad(x)) attach(out, backward_reshape_fn, {x});
    return out;
}

// ====================================================================== random
void rp_manual_seed(unsigned long long seed) { g_rng.seed(seed); }

static Tensor* random_tensor(DType dtype, int device_id, int ndim, int* shape, bool normal) {
    Tensor* host = empty_tensor(dtype, -1, ndim, shape);
    if (!host) return nullptr;
    std::normal_distribution<double> nd(0.0, 1.0);
    std::uniform_real_distribution<double> ud(0.0, 1.0);
    for (size_t i = 0; i < host->size; i++) {
        double v = normal ? nd(g_rng) : ud(g_rng);
        store_from_double(host->data, i, dtype, dtype == DTYPE_FLOAT64 ? v : (double)(float)v);
    }
    if (device_id == -1) return host;
    Tensor* dev = tensor_to(host, device_id, dtype, false);
    free_tensor(host);
    return dev;
}

Tensor* rp_randn(DType dtype, int device_id, int ndim, int* shape) { return random_tensor(dtype, device_id, ndim, shape, true); }
Tensor* rp_rand(DType dtype, int device_id, int ndim, int* shape) { return random_tensor(dtype, device_id, ndim, shape, false); }

}  // extern "C"
