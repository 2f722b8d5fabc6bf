// Shared helpers for the gfx950 kernels: error plumbing, dtype traits, wavefront reductions.
#ifndef TNN_ROCM_CSRC_COMMON_H_
#define TNN_ROCM_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "tnn_rocm.h"

namespace tnn_rocm {

constexpr int kWave = 64;  // CDNA wavefront width

void set_error(const char *fmt, ...);

#define TR_CHECK_HIP(expr)                                                                     \
    do {                                                                                       \
        hipError_t _e = (expr);                                                                \
        if (_e != hipSuccess) {                                                                \
            ::tnn_rocm::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),       \
                                  __FILE__, __LINE__);                                         \
            return (int)_e;                                                                    \
        }                                                                                      \
    } while (0)

#define TR_REQUIRE(cond, code, ...)                                                            \
    do {                                                                                       \
        if (!(cond)) {                                                                         \
            ::tnn_rocm::set_error(__VA_ARGS__);                                                \
            return (code);                                                                     \
        }                                                                                      \
    } while (0)

// Launch check: reports configuration errors of the launch just issued.
#define TR_CHECK_LAUNCH() TR_CHECK_HIP(hipGetLastError())

typedef _Float16 half_t;
typedef uint16_t bf16_bits;

__device__ __forceinline__ float bf16_to_float(bf16_bits v) {
    return __uint_as_float(((uint32_t)v) << 16);
}
__device__ __forceinline__ bf16_bits float_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return (bf16_bits)((u >> 16) | 0x40);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);           // round to nearest even
    return (bf16_bits)(u >> 16);
}

// Element load/store as float for the three floating dtypes.
template <int DT> struct Elem;
template <> struct Elem<TNN_ROCM_F32> {
    typedef float type;
    static __device__ __forceinline__ float ld(const float *p) { return *p; }
    static __device__ __forceinline__ void st(float *p, float v) { *p = v; }
};
template <> struct Elem<TNN_ROCM_F16> {
    typedef half_t type;
    static __device__ __forceinline__ float ld(const half_t *p) { return (float)*p; }
    static __device__ __forceinline__ void st(half_t *p, float v) { *p = (half_t)v; }
};
template <> struct Elem<TNN_ROCM_BF16> {
    typedef bf16_bits type;
    static __device__ __forceinline__ float ld(const bf16_bits *p) { return bf16_to_float(*p); }
    static __device__ __forceinline__ void st(bf16_bits *p, float v) { *p = float_to_bf16(v); }
};

// Round half away from zero exactly as the reference's float2int8: add +-0.5f in fp32 (one
// rounding), clamp in fp32, truncate.  The translation units are compiled with -ffp-contract=off
// so the add is never fused with the multiply that produced v.
__device__ __forceinline__ int8_t float2int8_ref(float v) {
    float t = __fadd_rn(v, v >= 0.f ? 0.5f : -0.5f);
    t       = fminf(t, 127.0f);
    t       = fmaxf(t, -128.0f);
    return (int8_t)(int)t;
}

// erf GELU in fp32, the product kept un-contracted in the reference's operand order.
__device__ __forceinline__ float gelu_erf(float x) {
    float e = erff(__fmul_rn(x, 0.707106793288165f));
    return __fmul_rn(__fmul_rn(0.5f, x), __fadd_rn(e, 1.0f));
}

// erf GELU for results that are rounded to fp16/bf16.  With q = erfc(|x|/sqrt2)/2 = Phi(-|x|):
// gelu(x) = x - x*q for x >= 0 and x*q for x < 0 (no cancellation in the negative tail).  q comes from the rational
// approximation 7.1.26 of Abramowitz & Stegun (|error| <= 1.5e-7 in erf), with the 1/2 folded into the
// coefficients and 1/sqrt2 into the two constants: one reciprocal, one exp2 and ten plain operations instead
// of the ~40-instruction erff; the rounded fp16 result differs from the exact one by at most one ulp.
// fp32 outputs keep gelu_erf.
__device__ __forceinline__ float gelu_erf_fast(float x) {
    float t  = __builtin_amdgcn_rcpf(fmaf(0.231641888f, fabsf(x), 1.0f));
    float p  = fmaf(fmaf(fmaf(fmaf(0.5307027145f, t, -0.7265760135f), t, 0.7107068705f), t, -0.142248368f), t, 0.127414796f);
    float e  = __builtin_amdgcn_exp2f(x * x * -0.72134752f);
    // p*t*e = Phi(-|x|), and x*Phi(x) = max(x, 0) - |x| * Phi(-|x|) for either sign
    return fmaf(-fabsf(x), p * t * e, fmaxf(x, 0.f));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

static inline bool is_float_dtype(int dt) {
    return dt == TNN_ROCM_F32 || dt == TNN_ROCM_F16 || dt == TNN_ROCM_BF16;
}
static inline size_t dtype_bytes(int dt) {
    switch (dt) {
        case TNN_ROCM_F32: return 4;
        case TNN_ROCM_F16: return 2;
        case TNN_ROCM_I8: return 1;
        case TNN_ROCM_I32: return 4;
        case TNN_ROCM_BF16: return 2;
        default: return 0;
    }
}

}  // namespace tnn_rocm
#endif
