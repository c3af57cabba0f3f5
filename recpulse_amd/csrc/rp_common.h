// Shared helpers of the gfx950 device layer: error reporting, the per-thread
// stream, dtype traits and the reference's 16-bit rounding on the device.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/rp_hip.h"

namespace rp {

// ---- host side ------------------------------------------------------------
void set_error(const char* fmt, ...);
hipStream_t current_stream();
bool check_hip(hipError_t e, const char* what);          // false (and error text) on failure
bool check_launch(const char* what);                     // hipGetLastError after a launch
bool stream_is_capturing();                              // the calling thread's stream is recording a graph
int device_cu_count();                                   // compute units of the current device (0 when it cannot be read)
// Kernel families can be switched off for cross-checks and same-machine comparisons: RP_HIP_DISABLE holds a comma-separated
// list of names (read once per process).  The dispatcher then takes what it would take if that kernel did not exist.
bool path_disabled(const char* name);
// True when, on the current device, workgroups of a one-dimensional grid whose linear ids are equal modulo 8 were
// observed to run on one XCD (one L2).  Measured once per device with a short kernel and a blocking read-back; a
// first query made while the calling thread's stream records a graph answers false and measures later.
bool workgroups_share_xcd_by_residue();
// Launches the calling thread's postponed scalar multiply, if there is one (rp_hip_mul_scalar_deferred).  current_stream()
// calls it, so every launch and stream-ordered copy is preceded by it; entry points that reach the device without asking
// for the stream call it themselves.  deferred_touches: the postponed multiply reads or writes a buffer starting at ptr.
void flush_deferred();
bool deferred_touches(const void* ptr);

inline size_t dtype_size(int dtype) {                    // reference core/half_precision.h:10-18
    switch (dtype) {
        case RP_DTYPE_FLOAT32: return 4;
        case RP_DTYPE_FLOAT64: return 8;
        case RP_DTYPE_FLOAT16: return 2;
        case RP_DTYPE_BFLOAT16: return 2;
        default: return 0;
    }
}

// ---- device side ----------------------------------------------------------
// Storage types.  16-bit values are carried as raw bit patterns so that the
// reference's own rounding (not the hardware's round-to-nearest-even) decides
// every narrowing.
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };

template <typename T> struct traits;
template <> struct traits<float>  { using acc = float;  static constexpr int code = RP_DTYPE_FLOAT32; };
template <> struct traits<double> { using acc = double; static constexpr int code = RP_DTYPE_FLOAT64; };
template <> struct traits<f16_t>  { using acc = float;  static constexpr int code = RP_DTYPE_FLOAT16; };
template <> struct traits<bf16_t> { using acc = float;  static constexpr int code = RP_DTYPE_BFLOAT16; };

__device__ __forceinline__ float widen(float x) { return x; }
__device__ __forceinline__ double widen(double x) { return x; }
__device__ __forceinline__ float widen(bf16_t x) { return __uint_as_float((uint32_t)x.bits << 16); }
__device__ __forceinline__ float widen(f16_t x) {
    // every fp16 value (subnormals included) is exact in fp32; the hardware
    // conversion is exact too and keeps NaN payload bits in place
    _Float16 h = __builtin_bit_cast(_Float16, x.bits);
    return (float)h;
}

// fp32 -> bf16: truncate and add the first dropped bit (reference
// core/half_precision.h:92-97; no NaN special case there either).
__device__ __forceinline__ uint16_t narrow_bf16_bits(float f) {
    uint32_t w = __float_as_uint(f);
    return (uint16_t)((w >> 16) + ((w >> 15) & 1u));
}

// fp32 -> fp16 with the same "add the first dropped bit" rule, including the subnormal and overflow branches
// (reference core/half_precision.h:50-83).  Adding the first dropped bit and truncating is truncating
// |x| + half an fp16 ulp: the half ulp is 2^(E-11) for an fp16-normal result and 2^-25 below that, the sum is
// exact in fp32 up to a carry that cannot reach the truncation point, and the hardware's round-toward-zero
// conversion does the truncation, subnormal results included.  Magnitudes below 2^-25 are the reference's zero
// (their sum could round up to 2^-24, so they are cleared first); sums of 65536 or more, infinities included,
// are its infinity; a NaN stays a NaN (the hardware's quiet NaN; the reference keeps the top payload bits).
// Straight-line code on the magnitude, the sign is put back at the end.
__device__ __forceinline__ uint16_t narrow_f16_bits(float x) {
    const uint32_t w = __float_as_uint(x);
    uint32_t a = w & 0x7FFFFFFFu;
    a = a < 0x33000000u ? 0u : a;                                                  // below 2^-25
    const uint32_t he = (a & 0x7F800000u) - (11u << 23);                           // exponent field of 2^(E-11); wraps for tiny a,
    const uint32_t hb = (int32_t)he > (int32_t)(102u << 23) ? he : (102u << 23);   // which the signed maximum with 2^-25 absorbs
    const float sum = __uint_as_float(a) + __uint_as_float(hb);
    uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(sum, 0.f));     // upper half: +0
    bits = sum >= 65536.f ? 0x7C00u : bits;
    return (uint16_t)(bits | ((w >> 16) & 0x8000u));
}

// The same narrowing for values whose result is a normal fp16 number (2^-14 <= |x| < 65520): there the first dropped
// bit is bit 12 of the fp32 pattern, adding it to the pattern carries into the kept bits exactly when it is set (into
// the exponent too, which is the next power of two), and the hardware's truncating conversion drops the rest: two
// instructions instead of twelve.  f16_range_key(x) is below F16_NORMAL_SPAN exactly for those values (NaN, infinities,
// zeros and subnormal results are not), so a wave takes this path for a tile after one unsigned maximum over its keys.
constexpr uint32_t F16_NORMAL_SPAN = (0x477FF000u << 1) - (0x38800000u << 1);
__device__ __forceinline__ uint32_t f16_range_key(float x) { return (__float_as_uint(x) << 1) - (0x38800000u << 1); }
__device__ __forceinline__ uint16_t narrow_f16_normal_bits(float x) {
    const float bumped = __uint_as_float(__float_as_uint(x) + 0x1000u);
    return (uint16_t)__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bumped, 0.f));
}

template <typename T> __device__ __forceinline__ T narrow(typename traits<T>::acc v);
template <> __device__ __forceinline__ float narrow<float>(float v) { return v; }
template <> __device__ __forceinline__ double narrow<double>(double v) { return v; }
template <> __device__ __forceinline__ bf16_t narrow<bf16_t>(float v) { bf16_t r; r.bits = narrow_bf16_bits(v); return r; }
template <> __device__ __forceinline__ f16_t narrow<f16_t>(float v) { f16_t r; r.bits = narrow_f16_bits(v); return r; }

// The GEMM epilogue: one narrowing per reference op in the chain
//   matmul (ops/ops.c:6838) -> bias add (ops/ops.c:162) -> grad accumulation (ops/ops.c:6785).
template <typename T>
__device__ __forceinline__ T finish(typename traits<T>::acc acc, bool has_bias, T bias, bool accumulate, T old) {
    T y = narrow<T>(acc);
    if (has_bias) y = narrow<T>(widen(y) + widen(bias));
    if (accumulate) y = narrow<T>(widen(old) + widen(y));
    return y;
}

}  // namespace rp

#define RP_DISPATCH_DTYPE(dtype, ...)                                              \
    switch (dtype) {                                                               \
        case RP_DTYPE_FLOAT32:  { using T = float;       __VA_ARGS__; break; }     \
        case RP_DTYPE_FLOAT64:  { using T = double;      __VA_ARGS__; break; }     \
        case RP_DTYPE_FLOAT16:  { using T = rp::f16_t;   __VA_ARGS__; break; }     \
        case RP_DTYPE_BFLOAT16: { using T = rp::bf16_t;  __VA_ARGS__; break; }     \
        default: rp::set_error("unsupported dtype %d", (int)(dtype)); return -1;   \
    }
