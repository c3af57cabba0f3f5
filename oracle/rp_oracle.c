/*
 * rp_oracle.c — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C restatement of the RecPulse reference's CPU arithmetic for the
 * matmul path and its callers' lowering (im2col / col2im of conv2d).  It exists to check the HIP kernels and to time a CPU baseline.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load it; nothing in the shipped library links, imports or calls it.
 *
 * Build: gcc -O3 -std=c11 -fPIC -shared -ffp-contract=off (see Makefile).  The
 * reference builds its host files with `gcc -O3 -fPIC -std=c11` and no -march
 * (reference Makefile:55), so there is no FMA contraction and no
 * reassociation; -ffp-contract=off keeps that true on any host.
 *
 * Each function names the reference file:line it follows.  Pins (what proves
 * each restatement right without trusting this file) live in
 * tests/test_oracle.py: the reference tests' known answers, bit-equality with
 * the reference's own host kernels compiled into oracle/_ref, numpy float64
 * closed forms, and exhaustive converter sweeps.
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* dtype codes: reference core/tensor.h:7-13 */
enum { ORC_F32 = 0, ORC_F64 = 1, ORC_F16 = 2, ORC_BF16 = 3 };

static size_t orc_elem_size(int dtype) {
    /* reference core/half_precision.h:10-18 */
    switch (dtype) {
        case ORC_F32: return 4;
        case ORC_F64: return 8;
        case ORC_F16: return 2;
        case ORC_BF16: return 2;
        default: return 0;
    }
}

/* ---------------------------------------------------------------------------
 * 16-bit converters.  reference core/half_precision.h:20-97.
 * Widening is exact.  Narrowing adds the first dropped mantissa bit to the
 * truncated pattern (round half away from zero on the magnitude), which is
 * NOT round-to-nearest-even; bf16 narrowing has no NaN special case.
 * ------------------------------------------------------------------------- */
float orc_f16_to_f32(uint16_t h) {
    /* reference core/half_precision.h:20-48 */
    uint32_t s = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t f = h & 0x3FFu;
    uint32_t w;
    float out;
    if (e == 0) {
        if (f == 0) {
            w = s;
            memcpy(&out, &w, 4);
            return out;
        }
        /* subnormal: f * 2^-10 * 2^-14, both factors exact in fp32 */
        out = ((float)f / 1024.0f) * (1.0f / 16384.0f);
        return s ? -out : out;
    }
    if (e == 0x1Fu) {
        w = s | 0x7F800000u | (f << 13);
    } else {
        w = s | ((e + 112u) << 23) | (f << 13);
    }
    memcpy(&out, &w, 4);
    return out;
}

uint16_t orc_f32_to_f16(float x) {
    /* reference core/half_precision.h:50-83 */
    uint32_t w;
    memcpy(&w, &x, 4);
    uint32_t s = (w >> 16) & 0x8000u;
    uint32_t e32 = (w >> 23) & 0xFFu;
    uint32_t f = w & 0x7FFFFFu;
    int32_t e = (int32_t)e32 - 127 + 15;

    if (e32 == 0xFFu) {
        if (f) return (uint16_t)(s | 0x7C00u | (f >> 13) | 1u);
        return (uint16_t)(s | 0x7C00u);
    }
    if (e <= 0) {
        if (e < -10) return (uint16_t)s;
        f |= 0x800000u;
        int sh = 14 - e;
        uint32_t rb = (f >> (sh - 1)) & 1u;
        return (uint16_t)((uint16_t)(s | (f >> sh)) + (uint16_t)rb);
    }
    if (e >= 0x1F) return (uint16_t)(s | 0x7C00u);
    {
        uint32_t rb = (f >> 12) & 1u;
        return (uint16_t)((uint16_t)(s | ((uint32_t)e << 10) | (f >> 13)) + (uint16_t)rb);
    }
}

float orc_bf16_to_f32(uint16_t h) {
    /* reference core/half_precision.h:85-90 */
    uint32_t w = (uint32_t)h << 16;
    float out;
    memcpy(&out, &w, 4);
    return out;
}

uint16_t orc_f32_to_bf16(float x) {
    /* reference core/half_precision.h:92-97 */
    uint32_t w;
    memcpy(&w, &x, 4);
    return (uint16_t)((w >> 16) + ((w >> 15) & 1u));
}

void orc_widen(const void* src, float* dst, size_t n, int dtype) {
    /* reference core/half_precision.h:115-120 */
    const uint16_t* s = (const uint16_t*)src;
    if (dtype == ORC_F16) for (size_t i = 0; i < n; i++) dst[i] = orc_f16_to_f32(s[i]);
    else                  for (size_t i = 0; i < n; i++) dst[i] = orc_bf16_to_f32(s[i]);
}

void orc_narrow(const float* src, void* dst, size_t n, int dtype) {
    /* reference core/half_precision.h:122-127 */
    uint16_t* d = (uint16_t*)dst;
    if (dtype == ORC_F16) for (size_t i = 0; i < n; i++) d[i] = orc_f32_to_f16(src[i]);
    else                  for (size_t i = 0; i < n; i++) d[i] = orc_f32_to_bf16(src[i]);
}

/* ---------------------------------------------------------------------------
 * Dense 2-D matmul.  reference functional/functional_host.c:780-806.
 * i-j-l order, C[i,j] zeroed then accumulated in place, in the output type,
 * multiply then add (two roundings), sequential in l.
 * ------------------------------------------------------------------------- */
int orc_matmul_f32(float* C, const float* A, const float* B, int m, int k, int n) {
    if (!C || !A || !B || m <= 0 || k <= 0 || n <= 0) return -1;
    for (int i = 0; i < m; i++) {
        const float* arow = A + (size_t)i * k;
        for (int j = 0; j < n; j++) {
            float acc = 0.0f;
            const float* bcol = B + j;
            for (int l = 0; l < k; l++) acc += arow[l] * bcol[(size_t)l * n];
            C[(size_t)i * n + j] = acc;
        }
    }
    return 0;
}

int orc_matmul_f64(double* C, const double* A, const double* B, int m, int k, int n) {
    if (!C || !A || !B || m <= 0 || k <= 0 || n <= 0) return -1;
    for (int i = 0; i < m; i++) {
        const double* arow = A + (size_t)i * k;
        for (int j = 0; j < n; j++) {
            double acc = 0.0;
            const double* bcol = B + j;
            for (int l = 0; l < k; l++) acc += arow[l] * bcol[(size_t)l * n];
            C[(size_t)i * n + j] = acc;
        }
    }
    return 0;
}

/* dtype dispatch.  reference functional/functional.c:978-1001.
 * fp16/bf16: widen A and B to fp32, run the fp32 loop, narrow C once. */
int orc_matmul(void* C, const void* A, const void* B, int m, int k, int n, int dtype) {
    if (!C || !A || !B || m <= 0 || k <= 0 || n <= 0) return -1;
    if (dtype == ORC_F32) return orc_matmul_f32((float*)C, (const float*)A, (const float*)B, m, k, n);
    if (dtype == ORC_F64) return orc_matmul_f64((double*)C, (const double*)A, (const double*)B, m, k, n);
    if (dtype == ORC_F16 || dtype == ORC_BF16) {
        size_t na = (size_t)m * k, nb = (size_t)k * n, nc = (size_t)m * n;
        float* a = (float*)malloc(na * 4);
        float* b = (float*)malloc(nb * 4);
        float* c = (float*)malloc(nc * 4);
        int rc = -1;
        if (a && b && c) {
            orc_widen(A, a, na, dtype);
            orc_widen(B, b, nb, dtype);
            rc = orc_matmul_f32(c, a, b, m, k, n);
            if (rc == 0) orc_narrow(c, C, nc, dtype);
        }
        free(a); free(b); free(c);
        return rc;
    }
    return -1;
}

/* ---------------------------------------------------------------------------
 * Flat and broadcasting add.  reference functional/functional.c:58-74 (flat,
 * 16-bit through the fp32 pivot) and functional/functional_host.c:106-134
 * (strided: out is dense row-major, operands indexed by per-dim strides).
 * ------------------------------------------------------------------------- */
static void* orc_load_as_compute(const void* x, size_t n, int dtype) {
    /* 16-bit → fresh fp32 array; f32/f64 → NULL (use x in place) */
    if (dtype == ORC_F16 || dtype == ORC_BF16) {
        float* w = (float*)malloc((n ? n : 1) * 4);
        if (w) orc_widen(x, w, n, dtype);
        return w;
    }
    return NULL;
}

int orc_add(void* out, const void* x1, const void* x2, size_t n, int dtype) {
    if (!out || !x1 || !x2 || n == 0) return -1;
    if (dtype == ORC_F32) {
        for (size_t i = 0; i < n; i++) ((float*)out)[i] = ((const float*)x1)[i] + ((const float*)x2)[i];
        return 0;
    }
    if (dtype == ORC_F64) {
        for (size_t i = 0; i < n; i++) ((double*)out)[i] = ((const double*)x1)[i] + ((const double*)x2)[i];
        return 0;
    }
    float* a = (float*)orc_load_as_compute(x1, n, dtype);
    float* b = (float*)orc_load_as_compute(x2, n, dtype);
    if (!a || !b) { free(a); free(b); return -1; }
    for (size_t i = 0; i < n; i++) a[i] = a[i] + b[i];
    orc_narrow(a, out, n, dtype);
    free(a); free(b);
    return 0;
}

int orc_add_strided(void* out, const void* x1, const void* x2, int ndim, const int* out_shape,
                    const int* s1, const int* s2, size_t out_size, int dtype) {
    /* reference functional/functional_host.c:106-134; 16-bit operands are read
     * through the fp32 pivot like every other host binary op */
    if (!out || !x1 || !x2 || out_size == 0 || ndim <= 0 || ndim > 16) return -1;
    size_t pitch[16];
    pitch[ndim - 1] = 1;
    for (int d = ndim - 2; d >= 0; d--) pitch[d] = pitch[d + 1] * (size_t)out_shape[d + 1];
    for (size_t i = 0; i < out_size; i++) {
        size_t rem = i, i1 = 0, i2 = 0;
        for (int d = 0; d < ndim; d++) {
            size_t c = rem / pitch[d];
            rem %= pitch[d];
            i1 += c * (size_t)s1[d];
            i2 += c * (size_t)s2[d];
        }
        switch (dtype) {
            case ORC_F32: ((float*)out)[i] = ((const float*)x1)[i1] + ((const float*)x2)[i2]; break;
            case ORC_F64: ((double*)out)[i] = ((const double*)x1)[i1] + ((const double*)x2)[i2]; break;
            case ORC_F16:
                ((uint16_t*)out)[i] = orc_f32_to_f16(orc_f16_to_f32(((const uint16_t*)x1)[i1]) +
                                                     orc_f16_to_f32(((const uint16_t*)x2)[i2]));
                break;
            case ORC_BF16:
                ((uint16_t*)out)[i] = orc_f32_to_bf16(orc_bf16_to_f32(((const uint16_t*)x1)[i1]) +
                                                      orc_bf16_to_f32(((const uint16_t*)x2)[i2]));
                break;
            default: return -1;
        }
    }
    return 0;
}

/* x * scalar.  reference functional/functional.c:241-258; the scalar arrives as
 * float for every dtype but float64 (python/tensor_python.c:475-485). */
int orc_mul_scalar(void* out, const void* x, double scalar, size_t n, int dtype) {
    if (!out || !x || n == 0) return -1;
    if (dtype == ORC_F64) {
        for (size_t i = 0; i < n; i++) ((double*)out)[i] = ((const double*)x)[i] * scalar;
        return 0;
    }
    float s = (float)scalar;
    if (dtype == ORC_F32) {
        for (size_t i = 0; i < n; i++) ((float*)out)[i] = ((const float*)x)[i] * s;
        return 0;
    }
    float* a = (float*)orc_load_as_compute(x, n, dtype);
    if (!a) return -1;
    for (size_t i = 0; i < n; i++) a[i] = a[i] * s;
    orc_narrow(a, out, n, dtype);
    free(a);
    return 0;
}

/* relu and its VJP.  reference functional/functional_host.c:514-528,
 * ops/grad_host.c:589-620. */
int orc_relu(void* out, const void* x, size_t n, int dtype) {
    if (!out || !x || n == 0) return -1;
    if (dtype == ORC_F32) {
        for (size_t i = 0; i < n; i++) { float v = ((const float*)x)[i]; ((float*)out)[i] = v > 0.0f ? v : 0.0f; }
        return 0;
    }
    if (dtype == ORC_F64) {
        for (size_t i = 0; i < n; i++) { double v = ((const double*)x)[i]; ((double*)out)[i] = v > 0.0 ? v : 0.0; }
        return 0;
    }
    float* a = (float*)orc_load_as_compute(x, n, dtype);
    if (!a) return -1;
    for (size_t i = 0; i < n; i++) a[i] = a[i] > 0.0f ? a[i] : 0.0f;
    orc_narrow(a, out, n, dtype);
    free(a);
    return 0;
}

int orc_backwards_relu(const void* grad_c, const void* x, void* grad_x, size_t n, int dtype) {
    if (!grad_c || !x || !grad_x) return -1;
    if (dtype == ORC_F32) {
        for (size_t i = 0; i < n; i++)
            ((float*)grad_x)[i] = ((const float*)x)[i] > 0.0f ? ((const float*)grad_c)[i] : 0.0f;
        return 0;
    }
    if (dtype == ORC_F64) {
        for (size_t i = 0; i < n; i++)
            ((double*)grad_x)[i] = ((const double*)x)[i] > 0.0 ? ((const double*)grad_c)[i] : 0.0;
        return 0;
    }
    float* g = (float*)orc_load_as_compute(grad_c, n, dtype);
    float* a = (float*)orc_load_as_compute(x, n, dtype);
    if (!g || !a) { free(g); free(a); return -1; }
    for (size_t i = 0; i < n; i++) g[i] = a[i] > 0.0f ? g[i] : 0.0f;
    orc_narrow(g, grad_x, n, dtype);
    free(g); free(a);
    return 0;
}

/* softmax / log-softmax along the middle axis of [outer, dim, inner].
 * reference functional/functional_host.c:1050-1140 (three serial passes per
 * row: max, exp+sum, divide), 16-bit through the fp32 pivot
 * (functional/functional.c:556-600). */
static void orc_softmax_f32(float* out, const float* x, size_t outer, size_t dim, size_t inner, int take_log) {
    for (size_t o = 0; o < outer; o++) for (size_t i = 0; i < inner; i++) {
        size_t base = o * dim * inner + i;
        float mx = -FLT_MAX;
        for (size_t d = 0; d < dim; d++) { float v = x[base + d * inner]; if (v > mx) mx = v; }
        float sum = 0.0f;
        if (!take_log) {
            for (size_t d = 0; d < dim; d++) { float e = expf(x[base + d * inner] - mx); out[base + d * inner] = e; sum += e; }
            for (size_t d = 0; d < dim; d++) out[base + d * inner] /= sum;
        } else {
            for (size_t d = 0; d < dim; d++) sum += expf(x[base + d * inner] - mx);
            float lse = logf(sum);
            for (size_t d = 0; d < dim; d++) out[base + d * inner] = x[base + d * inner] - mx - lse;
        }
    }
}

static void orc_softmax_f64(double* out, const double* x, size_t outer, size_t dim, size_t inner, int take_log) {
    for (size_t o = 0; o < outer; o++) for (size_t i = 0; i < inner; i++) {
        size_t base = o * dim * inner + i;
        double mx = -DBL_MAX;
        for (size_t d = 0; d < dim; d++) { double v = x[base + d * inner]; if (v > mx) mx = v; }
        double sum = 0.0;
        if (!take_log) {
            for (size_t d = 0; d < dim; d++) { double e = exp(x[base + d * inner] - mx); out[base + d * inner] = e; sum += e; }
            for (size_t d = 0; d < dim; d++) out[base + d * inner] /= sum;
        } else {
            for (size_t d = 0; d < dim; d++) sum += exp(x[base + d * inner] - mx);
            double lse = log(sum);
            for (size_t d = 0; d < dim; d++) out[base + d * inner] = x[base + d * inner] - mx - lse;
        }
    }
}

static int orc_softmax_any(void* out, const void* x, size_t outer, size_t dim, size_t inner, int dtype, int take_log) {
    if (!out || !x) return -1;
    size_t n = outer * dim * inner;
    if (dtype == ORC_F32) { orc_softmax_f32((float*)out, (const float*)x, outer, dim, inner, take_log); return 0; }
    if (dtype == ORC_F64) { orc_softmax_f64((double*)out, (const double*)x, outer, dim, inner, take_log); return 0; }
    float* a = (float*)orc_load_as_compute(x, n, dtype);
    float* r = (float*)malloc((n ? n : 1) * 4);
    if (!a || !r) { free(a); free(r); return -1; }
    orc_softmax_f32(r, a, outer, dim, inner, take_log);
    orc_narrow(r, out, n, dtype);
    free(a); free(r);
    return 0;
}

int orc_softmax(void* out, const void* x, size_t outer, size_t dim, size_t inner, int dtype) {
    return orc_softmax_any(out, x, outer, dim, inner, dtype, 0);
}

int orc_log_softmax(void* out, const void* x, size_t outer, size_t dim, size_t inner, int dtype) {
    return orc_softmax_any(out, x, outer, dim, inner, dtype, 1);
}

/* softmax VJP: gx = y * (g - sum_d g*y).  reference ops/grad_host.c:1360-1426. */
int orc_backwards_softmax(const void* grad_c, const void* y, void* grad_x,
                          size_t outer, size_t dim, size_t inner, int dtype) {
    if (!grad_c || !y || !grad_x) return -1;
    size_t n = outer * dim * inner;
    if (dtype == ORC_F64) {
        const double* g = (const double*)grad_c; const double* s = (const double*)y; double* r = (double*)grad_x;
        for (size_t o = 0; o < outer; o++) for (size_t i = 0; i < inner; i++) {
            size_t base = o * dim * inner + i;
            double dot = 0.0;
            for (size_t d = 0; d < dim; d++) dot += g[base + d * inner] * s[base + d * inner];
            for (size_t d = 0; d < dim; d++) r[base + d * inner] = s[base + d * inner] * (g[base + d * inner] - dot);
        }
        return 0;
    }
    float* gw = (float*)orc_load_as_compute(grad_c, n, dtype);
    float* sw = (float*)orc_load_as_compute(y, n, dtype);
    int half = (dtype == ORC_F16 || dtype == ORC_BF16);
    if (half && (!gw || !sw)) { free(gw); free(sw); return -1; }
    const float* g = half ? gw : (const float*)grad_c;
    const float* s = half ? sw : (const float*)y;
    float* r = half ? (float*)malloc((n ? n : 1) * 4) : (float*)grad_x;
    if (!r) { free(gw); free(sw); return -1; }
    for (size_t o = 0; o < outer; o++) for (size_t i = 0; i < inner; i++) {
        size_t base = o * dim * inner + i;
        float dot = 0.0f;
        for (size_t d = 0; d < dim; d++) dot += g[base + d * inner] * s[base + d * inner];
        for (size_t d = 0; d < dim; d++) r[base + d * inner] = s[base + d * inner] * (g[base + d * inner] - dot);
    }
    if (half) { orc_narrow(r, grad_x, n, dtype); free(r); }
    free(gw); free(sw);
    return 0;
}

/* sum of all elements, sequential.  reference functional/functional_host.c:
 * 700-716 and functional/functional.c:444-470 (16-bit: widen, fp32 sum,
 * narrow the one result). */
int orc_sum_all(void* out, const void* x, size_t n, int dtype) {
    if (!out || !x || n == 0) return -1;
    if (dtype == ORC_F64) {
        double s = 0.0;
        for (size_t i = 0; i < n; i++) s += ((const double*)x)[i];
        *(double*)out = s;
        return 0;
    }
    float s = 0.0f;
    if (dtype == ORC_F32) {
        for (size_t i = 0; i < n; i++) s += ((const float*)x)[i];
        *(float*)out = s;
        return 0;
    }
    float* a = (float*)orc_load_as_compute(x, n, dtype);
    if (!a) return -1;
    for (size_t i = 0; i < n; i++) s += a[i];
    free(a);
    orc_narrow(&s, out, 1, dtype);
    return 0;
}

/* Bias gradient: reduce a dense [rows, cols] grad over rows into [cols].
 * reference ops/ops.c:6970-7101 (reduce_grad_to_shape) specialised to the
 * Linear case target_shape = [cols]: elements are visited in row-major order
 * and added into res[col], so each column is summed top to bottom; fp32
 * accumulator for f32/f16/bf16 (:7027-7067), fp64 for f64 (:7068-7086). */
int orc_reduce_rows(void* out, const void* grad, int rows, int cols, int dtype) {
    if (!out || !grad || rows <= 0 || cols <= 0) return -1;
    size_t n = (size_t)rows * cols;
    if (dtype == ORC_F64) {
        double* r = (double*)out; const double* g = (const double*)grad;
        for (int j = 0; j < cols; j++) r[j] = 0.0;
        for (size_t i = 0; i < n; i++) r[i % cols] += g[i];
        return 0;
    }
    float* gw = (float*)orc_load_as_compute(grad, n, dtype);
    int half = (dtype == ORC_F16 || dtype == ORC_BF16);
    if (half && !gw) return -1;
    const float* g = half ? gw : (const float*)grad;
    float* r = half ? (float*)calloc(cols, 4) : (float*)out;
    if (!r) { free(gw); return -1; }
    if (!half) for (int j = 0; j < cols; j++) r[j] = 0.0f;
    for (size_t i = 0; i < n; i++) r[i % cols] += g[i];
    if (half) { orc_narrow(r, out, cols, dtype); free(r); }
    free(gw);
    return 0;
}

/* Gather a strided view into dense row-major memory.
 * reference functional/functional_host.c:880-942. */
int orc_contiguous_copy(void* out, const void* in, int ndim, const int* shape, const long long* strides, int dtype) {
    if (!out || !in || ndim <= 0 || ndim > 16) return -1;
    size_t es = orc_elem_size(dtype), total = 1;
    if (!es) return -1;
    for (int d = 0; d < ndim; d++) total *= (size_t)shape[d];
    for (size_t i = 0; i < total; i++) {
        size_t rem = i; long long off = 0;
        for (int d = ndim - 1; d >= 0; d--) { off += (long long)(rem % shape[d]) * strides[d]; rem /= shape[d]; }
        memcpy((char*)out + i * es, (const char*)in + off * (long long)es, es);
    }
    return 0;
}

/* ---------------------------------------------------------------------------
 * Strided, batched GEMM with the Linear epilogue, expressed the only way the
 * reference can express it: per batch slice, densify both operands
 * (ops/ops.c:6830-6831), run the 2-D matmul (ops/ops.c:6838), then — when a
 * bias is given — the broadcasting add of recpulse/module.py:110-114 →
 * ops/ops.c:129-210, and — when accumulate is set — the grad-accumulation add
 * of ops/ops.c:6781-6788.  For 16-bit dtypes every one of those steps narrows
 * its result (three roundings), exactly as the chain of reference ops does.
 * Strides are in elements; C may be strided too.
 * ------------------------------------------------------------------------- */
int orc_gemm_strided_batched(void* C, const void* A, const void* B, const void* bias,
                             int batch, int m, int k, int n,
                             long long a_bs, long long a_rs, long long a_cs,
                             long long b_bs, long long b_rs, long long b_cs,
                             long long c_bs, long long c_rs, long long c_cs,
                             int accumulate, int dtype) {
    size_t es = orc_elem_size(dtype);
    if (!C || !A || !B || !es || batch <= 0 || m <= 0 || k <= 0 || n <= 0) return -1;
    void* a = malloc((size_t)m * k * es);
    void* b = malloc((size_t)k * n * es);
    void* c = malloc((size_t)m * n * es);
    void* t = malloc((size_t)m * n * es);
    int rc = -1;
    if (!a || !b || !c || !t) goto done;
    for (int z = 0; z < batch; z++) {
        int shp_a[2] = {m, k}, shp_b[2] = {k, n}, shp_c[2] = {m, n};
        long long st_a[2] = {a_rs, a_cs}, st_b[2] = {b_rs, b_cs}, st_c[2] = {c_rs, c_cs};
        const char* Az = (const char*)A + (long long)z * a_bs * (long long)es;
        const char* Bz = (const char*)B + (long long)z * b_bs * (long long)es;
        char* Cz = (char*)C + (long long)z * c_bs * (long long)es;
        orc_contiguous_copy(a, Az, 2, shp_a, st_a, dtype);
        orc_contiguous_copy(b, Bz, 2, shp_b, st_b, dtype);
        if (orc_matmul(c, a, b, m, k, n, dtype) != 0) goto done;
        if (bias) {
            int s1[2] = {n, 1}, s2[2] = {0, 1};
            if (orc_add_strided(t, c, bias, 2, shp_c, s1, s2, (size_t)m * n, dtype) != 0) goto done;
            memcpy(c, t, (size_t)m * n * es);
        }
        if (accumulate) {
            orc_contiguous_copy(t, Cz, 2, shp_c, st_c, dtype);
            if (orc_add(c, t, c, (size_t)m * n, dtype) != 0) goto done;
        }
        for (int i = 0; i < m; i++) for (int j = 0; j < n; j++)
            memcpy(Cz + ((long long)i * c_rs + (long long)j * c_cs) * (long long)es,
                   (const char*)c + ((size_t)i * n + j) * es, es);
    }
    rc = 0;
done:
    free(a); free(b); free(c); free(t);
    return rc;
}

/* ---------------------------------------------------------------------------
 * Cross-entropy on logits [batch, classes], reduction = mean, f32 and f64.
 * reference ops/ops.c:5545-5643 (forward = log_softmax then NLL) with
 * ops/ops.c:5318-5352 (NLL: fp64 running sum of -logp[target]; the f32 result
 * is that sum narrowed to float and then divided by batch in float) and
 * ops/ops.c:5412-5543 (backward = ((softmax - onehot) * (1/batch)) * upstream,
 * each step rounded in the tensor dtype).
 * The reference's NLL reads 16-bit log-probabilities through a float pointer
 * (ops/ops.c:5344), so it defines no usable 16-bit result; 16-bit is refused.
 * ------------------------------------------------------------------------- */
int orc_cross_entropy_mean(void* loss_out, void* grad_logits, const void* logits, const int* targets,
                           int batch, int classes, double upstream, int dtype) {
    if (!logits || !targets || batch <= 0 || classes <= 0) return -1;
    if (dtype != ORC_F32 && dtype != ORC_F64) return -1;
    for (int b = 0; b < batch; b++) if (targets[b] < 0 || targets[b] >= classes) return -1;
    size_t n = (size_t)batch * classes, es = orc_elem_size(dtype);
    void* lp = malloc(n * es);
    void* sm = malloc(n * es);
    int rc = -1;
    if (!lp || !sm) goto done;
    orc_log_softmax(lp, logits, (size_t)batch, (size_t)classes, 1, dtype);
    orc_softmax(sm, logits, (size_t)batch, (size_t)classes, 1, dtype);
    if (loss_out) {
        double s64 = 0.0;
        for (int b = 0; b < batch; b++) {
            size_t off = (size_t)b * classes + targets[b];
            if (dtype == ORC_F64) s64 -= ((const double*)lp)[off];
            else s64 -= (double)((const float*)lp)[off];
        }
        if (dtype == ORC_F64) *(double*)loss_out = s64 / (double)batch;
        else { float s32 = (float)s64; s32 /= (float)batch; *(float*)loss_out = s32; }
    }
    if (grad_logits) {
        if (dtype == ORC_F64) {
            double* g = (double*)grad_logits; const double* s = (const double*)sm;
            for (size_t i = 0; i < n; i++) g[i] = s[i];
            for (int b = 0; b < batch; b++) g[(size_t)b * classes + targets[b]] -= 1.0;
            double sc = 1.0 / (double)batch;
            for (size_t i = 0; i < n; i++) g[i] *= sc;
            for (size_t i = 0; i < n; i++) g[i] = g[i] * upstream;
        } else {
            float* g = (float*)grad_logits; const float* s = (const float*)sm;
            for (size_t i = 0; i < n; i++) g[i] = s[i];
            for (int b = 0; b < batch; b++) g[(size_t)b * classes + targets[b]] -= 1.0f;
            float sc = 1.0f / (float)batch;
            for (size_t i = 0; i < n; i++) g[i] *= sc;
            float up = (float)upstream;
            for (size_t i = 0; i < n; i++) g[i] = g[i] * up;
        }
    }
    rc = 0;
done:
    free(lp); free(sm);
    return rc;
}

/* ---------------------------------------------------------------------------
 * Cross-entropy with every reduction and both input kinds.
 * reference ops/ops.c:5545-5643 (op_cross_entropy_loss), 5318-5400 (op_nll_loss),
 * 5412-5543 (backward_cross_entropy_loss_fn); reduction codes ops/ops.h:109-111
 * (0 none, 1 mean, 2 sum).
 *   from_logits != 0: log_probs = log_softmax(x), the saved probabilities = softmax(x);
 *   from_logits == 0: x already holds probabilities, log_probs = log(x) (rp_log, element-wise).
 * Forward: NLL terms -log_probs[b, target_b]; 'none' returns them, otherwise they are
 * summed in batch order in double, narrowed to float for float32, and 'mean' then divides
 * by (float)batch in the tensor's type.
 * Backward: grad = p - onehot (logits) or -1 / p at the target and 0 elsewhere
 * (probabilities); 'mean' multiplies by 1 / batch; then by the upstream gradient, one
 * element for 'mean' / 'sum', one per row for 'none' (rp_mul_strided with strides {1, 0}).
 * float32 / float64 only, as orc_cross_entropy_mean.
 * ------------------------------------------------------------------------- */
int orc_cross_entropy(void* loss_out, void* grad_x, const void* x, const int* targets, int batch, int classes,
                      int reduction, int from_logits, const void* upstream, int dtype) {
    if (!x || !targets || batch <= 0 || classes <= 0 || reduction < 0 || reduction > 2) return -1;
    if (dtype != ORC_F32 && dtype != ORC_F64) return -1;
    for (int b = 0; b < batch; b++) if (targets[b] < 0 || targets[b] >= classes) return -1;
    size_t n = (size_t)batch * classes, es = orc_elem_size(dtype);
    void* lp = malloc(n * es);
    void* sm = malloc(n * es);
    int rc = -1;
    if (!lp || !sm) goto done;
    if (from_logits) {
        orc_log_softmax(lp, x, (size_t)batch, (size_t)classes, 1, dtype);
        orc_softmax(sm, x, (size_t)batch, (size_t)classes, 1, dtype);
    } else {
        if (dtype == ORC_F64) for (size_t i = 0; i < n; i++) ((double*)lp)[i] = log(((const double*)x)[i]);
        else for (size_t i = 0; i < n; i++) ((float*)lp)[i] = logf(((const float*)x)[i]);
        memcpy(sm, x, n * es);
    }
    if (loss_out) {
        if (reduction == 0) {
            for (int b = 0; b < batch; b++) {
                size_t off = (size_t)b * classes + targets[b];
                if (dtype == ORC_F64) ((double*)loss_out)[b] = -((const double*)lp)[off];
                else ((float*)loss_out)[b] = -((const float*)lp)[off];
            }
        } else {
            double s64 = 0.0;
            for (int b = 0; b < batch; b++) {
                size_t off = (size_t)b * classes + targets[b];
                if (dtype == ORC_F64) s64 -= ((const double*)lp)[off];
                else s64 -= (double)((const float*)lp)[off];
            }
            float s32 = (float)s64;
            if (reduction == 1) { s32 /= (float)batch; s64 /= (double)batch; }
            if (dtype == ORC_F64) *(double*)loss_out = s64; else *(float*)loss_out = s32;
        }
    }
    if (grad_x) {
        if (!upstream) goto done;
        if (dtype == ORC_F64) {
            double* g = (double*)grad_x; const double* s = (const double*)sm; const double* up = (const double*)upstream;
            if (from_logits) {
                for (size_t i = 0; i < n; i++) g[i] = s[i];
                for (int b = 0; b < batch; b++) g[(size_t)b * classes + targets[b]] -= 1.0;
            } else {
                for (size_t i = 0; i < n; i++) g[i] = 0.0;
                for (int b = 0; b < batch; b++) { size_t ti = (size_t)b * classes + targets[b]; g[ti] = -1.0 / s[ti]; }
            }
            if (reduction == 1) { double sc = 1.0 / (double)batch; for (size_t i = 0; i < n; i++) g[i] *= sc; }
            for (size_t i = 0; i < n; i++) g[i] = g[i] * (reduction == 0 ? up[i / (size_t)classes] : up[0]);
        } else {
            float* g = (float*)grad_x; const float* s = (const float*)sm; const float* up = (const float*)upstream;
            if (from_logits) {
                for (size_t i = 0; i < n; i++) g[i] = s[i];
                for (int b = 0; b < batch; b++) g[(size_t)b * classes + targets[b]] -= 1.0f;
            } else {
                for (size_t i = 0; i < n; i++) g[i] = 0.0f;
                for (int b = 0; b < batch; b++) { size_t ti = (size_t)b * classes + targets[b]; g[ti] = -1.0f / s[ti]; }
            }
            if (reduction == 1) { float sc = 1.0f / (float)batch; for (size_t i = 0; i < n; i++) g[i] *= sc; }
            for (size_t i = 0; i < n; i++) g[i] = g[i] * (reduction == 0 ? up[i / (size_t)classes] : up[0]);
        }
    }
    rc = 0;
done:
    free(lp); free(sm);
    return rc;
}

/* gradient of log_softmax: gx = g - exp(y) * sum_d g, the sum in index order in the compute type.
 * reference ops/grad_host.c:1428-1500 (16-bit through the fp32 pivot, one narrowing). */
int orc_backwards_log_softmax(const void* grad_c, const void* y, void* grad_x,
                              size_t outer, size_t dim, size_t inner, int dtype) {
    if (!grad_c || !y || !grad_x) return -1;
    size_t n = outer * dim * inner;
    if (dtype == ORC_F64) {
        const double* g = (const double*)grad_c; const double* l = (const double*)y; double* r = (double*)grad_x;
        for (size_t o = 0; o < outer; o++) for (size_t i = 0; i < inner; i++) {
            size_t base = o * dim * inner + i;
            double sum = 0.0;
            for (size_t d = 0; d < dim; d++) sum += g[base + d * inner];
            for (size_t d = 0; d < dim; d++) r[base + d * inner] = g[base + d * inner] - exp(l[base + d * inner]) * sum;
        }
        return 0;
    }
    float* gw = (float*)orc_load_as_compute(grad_c, n, dtype);
    float* lw = (float*)orc_load_as_compute(y, n, dtype);
    int half = (dtype == ORC_F16 || dtype == ORC_BF16);
    if (half && (!gw || !lw)) { free(gw); free(lw); return -1; }
    const float* g = half ? gw : (const float*)grad_c;
    const float* l = half ? lw : (const float*)y;
    float* r = half ? (float*)malloc((n ? n : 1) * 4) : (float*)grad_x;
    if (!r) { free(gw); free(lw); return -1; }
    for (size_t o = 0; o < outer; o++) for (size_t i = 0; i < inner; i++) {
        size_t base = o * dim * inner + i;
        float sum = 0.0f;
        for (size_t d = 0; d < dim; d++) sum += g[base + d * inner];
        for (size_t d = 0; d < dim; d++) r[base + d * inner] = g[base + d * inner] - expf(l[base + d * inner]) * sum;
    }
    if (half) { orc_narrow(r, grad_x, n, dtype); free(r); }
    free(gw); free(lw);
    return 0;
}

/* ---------------------------------------------------------------------------
 * conv2d lowering.  reference functional/functional_host.c:1237-1262 (im2col)
 * and 1291-1313 (col2im, which ADDS into im); 16-bit through the fp32 pivot with
 * one narrowing at the end (functional/functional.c:866-879, 896-911).
 * Written as a gather per destination element rather than the reference's
 * five nested loops; for col2im the contributions to one pixel still arrive in
 * ascending (kh, kw) order, which is the order the reference's loops visit them.
 * ------------------------------------------------------------------------- */
#define ORC_IM2COL(NAME, TYPE)                                                                          \
    static void NAME(TYPE* col, const TYPE* im, int C, int H, int W, int kH, int kW, int sh, int sw,   \
                     int ph, int pw, int dh, int dw, int oH, int oW) {                                  \
        size_t cols = (size_t)oH * oW;                                                                  \
        for (int r = 0; r < C * kH * kW; r++) {                                                         \
            int kw = r % kW, kh = (r / kW) % kH, c = r / (kW * kH);                                     \
            for (int oh = 0; oh < oH; oh++)                                                             \
                for (int ow = 0; ow < oW; ow++) {                                                       \
                    int h = oh * sh + kh * dh - ph, w = ow * sw + kw * dw - pw;                         \
                    int inside = h >= 0 && h < H && w >= 0 && w < W;                                    \
                    col[r * cols + (size_t)oh * oW + ow] = inside ? im[((size_t)c * H + h) * W + w] : (TYPE)0; \
                }                                                                                       \
        }                                                                                               \
    }
ORC_IM2COL(orc_im2col_f32, float)
ORC_IM2COL(orc_im2col_f64, double)

#define ORC_COL2IM(NAME, TYPE)                                                                          \
    static void NAME(TYPE* im, const TYPE* col, int C, int H, int W, int kH, int kW, int sh, int sw,   \
                     int ph, int pw, int dh, int dw, int oH, int oW) {                                  \
        size_t cols = (size_t)oH * oW;                                                                  \
        for (int c = 0; c < C; c++)                                                                     \
            for (int h = 0; h < H; h++)                                                                 \
                for (int w = 0; w < W; w++) {                                                           \
                    TYPE acc = im[((size_t)c * H + h) * W + w];                                         \
                    for (int kh = 0; kh < kH; kh++)                                                     \
                        for (int kw = 0; kw < kW; kw++) {                                               \
                            int hh = h + ph - kh * dh, ww = w + pw - kw * dw;                           \
                            if (hh < 0 || ww < 0 || hh % sh || ww % sw) continue;                       \
                            int oh = hh / sh, ow = ww / sw;                                             \
                            if (oh >= oH || ow >= oW) continue;                                         \
                            acc += col[((size_t)(c * kH + kh) * kW + kw) * cols + (size_t)oh * oW + ow]; \
                        }                                                                               \
                    im[((size_t)c * H + h) * W + w] = acc;                                              \
                }                                                                                       \
    }
ORC_COL2IM(orc_col2im_f32, float)
ORC_COL2IM(orc_col2im_f64, double)

int orc_im2col(void* col, const void* im, int C, int H, int W, int kH, int kW, int sh, int sw,
               int ph, int pw, int dh, int dw, int oH, int oW, int dtype) {
    if (!col || !im) return -1;
    size_t nim = (size_t)C * H * W, ncol = (size_t)C * kH * kW * oH * oW;
    if (dtype == ORC_F32) { orc_im2col_f32((float*)col, (const float*)im, C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW); return 0; }
    if (dtype == ORC_F64) { orc_im2col_f64((double*)col, (const double*)im, C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW); return 0; }
    if (dtype != ORC_F16 && dtype != ORC_BF16) return -1;
    float* a = (float*)malloc(nim * 4);
    float* b = (float*)malloc(ncol * 4);
    if (!a || !b) { free(a); free(b); return -1; }
    orc_widen(im, a, nim, dtype);
    orc_im2col_f32(b, a, C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW);
    orc_narrow(b, col, ncol, dtype);
    free(a); free(b);
    return 0;
}

int orc_col2im(void* im, const void* col, int C, int H, int W, int kH, int kW, int sh, int sw,
               int ph, int pw, int dh, int dw, int oH, int oW, int dtype) {
    if (!col || !im) return -1;
    size_t nim = (size_t)C * H * W, ncol = (size_t)C * kH * kW * oH * oW;
    if (dtype == ORC_F32) { orc_col2im_f32((float*)im, (const float*)col, C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW); return 0; }
    if (dtype == ORC_F64) { orc_col2im_f64((double*)im, (const double*)col, C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW); return 0; }
    if (dtype != ORC_F16 && dtype != ORC_BF16) return -1;
    float* a = (float*)malloc(nim * 4);
    float* b = (float*)malloc(ncol * 4);
    if (!a || !b) { free(a); free(b); return -1; }
    orc_widen(im, a, nim, dtype);
    orc_widen(col, b, ncol, dtype);
    orc_col2im_f32(a, b, C, H, W, kH, kW, sh, sw, ph, pw, dh, dw, oH, oW);
    orc_narrow(a, im, nim, dtype);
    free(a); free(b);
    return 0;
}

/* ---------------------------------------------------------------------------
 * sigmoid and tanh, the nonlinearities of the LSTM / GRU cells.
 * reference functional/functional_host.c:498-545 (tanhf / tanh; 1/(1+expf(-x)) / 1/(1+exp(-x)));
 * 16-bit through the fp32 pivot with one narrowing (functional/functional.c, same pattern as add).
 * ------------------------------------------------------------------------- */
static int orc_unary(void* out, const void* x, size_t n, int dtype, int is_tanh) {
    if (!out || !x || n == 0) return -1;
    if (dtype == ORC_F64) {
        const double* a = (const double*)x; double* o = (double*)out;
        for (size_t i = 0; i < n; i++) o[i] = is_tanh ? tanh(a[i]) : 1.0 / (1.0 + exp(-a[i]));
        return 0;
    }
    float* w = (float*)orc_load_as_compute(x, n, dtype);
    const float* a = w ? w : (const float*)x;
    float* o = (dtype == ORC_F32) ? (float*)out : (float*)malloc(n * 4);
    if (!o || (dtype != ORC_F32 && !w)) { free(w); if (dtype != ORC_F32) free(o); return -1; }
    for (size_t i = 0; i < n; i++) o[i] = is_tanh ? tanhf(a[i]) : 1.0f / (1.0f + expf(-a[i]));
    if (dtype != ORC_F32) { orc_narrow(o, out, n, dtype); free(o); }
    free(w);
    return 0;
}
int orc_sigmoid(void* out, const void* x, size_t n, int dtype) { return orc_unary(out, x, n, dtype, 0); }
int orc_tanh(void* out, const void* x, size_t n, int dtype) { return orc_unary(out, x, n, dtype, 1); }

