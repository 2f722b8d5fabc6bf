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
// ---- result stores --------------------------------------------------------------------------------------------------
// When a kernel ends, the dirty lines of the eight L2s are written back before the next kernel of the stream may start
// (the L2s are not coherent with each other, so this is what makes one kernel's results visible to the next).  A GEMM
// that leaves 18 MB of results dirty pays about 1.8 us for that between its last instruction and its successor's first.
// Stores issued at device scope (sc1) go through the L2 to the memory side as they are made, under the kernel's own
// remaining work, and leave nothing to write back; they still allocate in the memory-side cache, where the consumer
// finds them (stores with the non-temporal hint do not, which costs the consumer more than the write-back saved).
// The compiler has no spelling for a 16-byte store at device scope, hence the assembly; a store of more than 8 bytes
// needs two wait states before its data registers may be overwritten, which the hazard recognizer cannot see through
// an asm statement, so they are part of it.  No memory clobber: nothing in these kernels reads what they store.
// The switch (one copy per translation unit, set together by tnn_rocm_debug_set_store_through) is there for A/B runs.
typedef unsigned int store_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int store_u32x2 __attribute__((ext_vector_type(2)));
static __constant__ int g_dev_store_through = 1;
#define TR_DEFINE_STORE_THROUGH_SETTER(name)                                                          \
    int name(int on) { return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_dev_store_through), &on, sizeof(int)); }

__device__ __forceinline__ void store_out16(void *p, store_u32x4 v) {
    if (g_dev_store_through)
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v));
    else
        *reinterpret_cast<store_u32x4 *>(p) = v;
}
__device__ __forceinline__ void store_out8(void *p, store_u32x2 v) {
    if (g_dev_store_through)
        asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(p), "v"(v));
    else
        *reinterpret_cast<store_u32x2 *>(p) = v;
}
__device__ __forceinline__ void store_out8(float2 *p, float2 v) {
    store_out8((void *)p, store_u32x2{__float_as_uint(v.x), __float_as_uint(v.y)});
}
__device__ __forceinline__ void store_out4(void *p, uint32_t v) {
    if (g_dev_store_through)
        asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v));
    else
        *reinterpret_cast<uint32_t *>(p) = v;
}
__device__ __forceinline__ void store_out2(void *p, uint16_t v) {
    if (g_dev_store_through)
        asm volatile("global_store_short %0, %1, off sc1" ::"v"(p), "v"((uint32_t)v));
    else
        *reinterpret_cast<uint16_t *>(p) = v;
}

template <int DT> struct Elem;
template <> struct Elem<TNN_ROCM_F32> {
    typedef float type;
    static __device__ __forceinline__ float ld(const float *p) { return *p; }
    static __device__ __forceinline__ void st(float *p, float v) { *p = v; }
    static __device__ __forceinline__ void st_out(float *p, float v) { store_out4(p, __float_as_uint(v)); }
};
template <> struct Elem<TNN_ROCM_F16> {
    typedef half_t type;
    static __device__ __forceinline__ float ld(const half_t *p) { return (float)*p; }
    static __device__ __forceinline__ void st(half_t *p, float v) { *p = (half_t)v; }
    static __device__ __forceinline__ void st_out(half_t *p, float v) {
        const half_t h = (half_t)v;
        store_out2(p, *reinterpret_cast<const uint16_t *>(&h));
    }
};
template <> struct Elem<TNN_ROCM_BF16> {
    typedef bf16_bits type;
    static __device__ __forceinline__ float ld(const bf16_bits *p) { return bf16_to_float(*p); }
    static __device__ __forceinline__ void st(bf16_bits *p, float v) { *p = float_to_bf16(v); }
    static __device__ __forceinline__ void st_out(bf16_bits *p, float v) { store_out2(p, float_to_bf16(v)); }
};

// Round half away from zero exactly as the reference's float2int8: add +-0.5f in fp32 (one
// rounding), clamp in fp32, truncate.  The translation units are compiled with -ffp-contract=off
// so the add is never fused with the multiply that produced v.
// (+-0.5 taken from the sign bit and the clamp as one med3 give the same result for every value that is not a NaN --
// -0.0 lands on 0 either way -- in three instructions instead of seven.  A NaN comes out as -128: the median of three
// with a NaN operand is the minimum of the other two, and -128 is also what the reference's x86 path makes of a NaN,
// whose truncating conversion yields INT_MIN before the saturating pack, x86_compute_int8.cc:31-39.)
__device__ __forceinline__ int8_t float2int8_ref(float v) {
    float t = __fadd_rn(v, __builtin_copysignf(0.5f, v));
    t       = __builtin_amdgcn_fmed3f(t, -128.0f, 127.0f);
    return (int8_t)(int)t;
}

// erf GELU for fp32 results, evaluated as the reference's CPU path compiles (cpu_gelu_layer_acc.cc:42-45 includes
// only <cmath>, so its unqualified erf is the double one): x*0.7071f and 0.5f*x are fp32 products, erf, the +1 and the
// final product are double, and the store rounds once to fp32.  erff would differ in the last ulp, which is enough
// to move a value across a rounding boundary of a quantiser that follows.
__device__ __forceinline__ float gelu_erf(float x) {
    const float hv = __fmul_rn(0.5f, x);
    const double e = erf((double)__fmul_rn(x, 0.707106793288165f)) + 1.0;
    return (float)((double)hv * e);
}

// erf GELU for results that are rounded to fp16/bf16.  With a = |x| and Phi(-a) = erfc(a/sqrt2)/2:
// gelu(x) = x*Phi(x) = max(x, 0) - a*Phi(-a) for either sign (no cancellation in the negative tail).
// -log2(Phi(-a)) is smooth and nearly quadratic, so Phi(-a) = exp2(-q(a)) with a degree-6 polynomial q, q(0) = 1
// (minimax fit of the relative error on [0, 9]: 2e-5, i.e. 3e-6 absolute in a*Phi(-a); beyond 9 the term is below
// 1e-18 and a is clamped so the polynomial stays inside its fitted range).  Six fused multiply-adds, one clamp, one
// exp2, one max and the final multiply-add: 13 issue slots against 19 for the rational form 7.1.26 of Abramowitz &
// Stegun used before and ~40 for erff.  Against the correctly rounded fp16 result 0.4 % of the values differ, by one
// ulp (2.8 % for the rational form).  fp32 outputs keep gelu_erf.
// max(x, 0) is formed as x/2 + |x/2|: exact for every finite x (halving and the sum of equal or opposite halves do not
// round), and unlike the maximum instruction, which returns its other operand for a NaN, it hands a NaN through, as the
// reference's GELU does (and gives NaN for -inf, where the reference's 0.5 x (erf + 1) is -inf times 0).  An overflow
// upstream therefore stays visible in the output instead of turning into zeros.
__device__ __forceinline__ float max_with_zero(float x) {
    const float h = __fmul_rn(0.5f, x);
    return __fadd_rn(h, fabsf(h));
}

__device__ __forceinline__ float gelu_erf_fast(float x) {
    // med3 instead of fmin / fmax: one instruction each, where the minimum / maximum forms first quiet their operand
    const float a = __builtin_amdgcn_fmed3f(fabsf(x), 0.f, 9.0f);
    float q       = -2.8009472064e-05f;
    q             = fmaf(q, a, 6.8930927528e-04f);
    q             = fmaf(q, a, -7.6513012845e-03f);
    q             = fmaf(q, a, 5.2408451099e-02f);
    q             = fmaf(q, a, 4.5977897954e-01f);
    q             = fmaf(q, a, 1.1508630942e+00f);
    q             = fmaf(q, a, 1.0f);
    const float e = __builtin_amdgcn_exp2f(-q);  // Phi(-a)
    // the clamped a: a*Phi(-a) is below 1e-18 past 9, and +inf stays +inf
    return fmaf(-a, e, max_with_zero(x));
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
