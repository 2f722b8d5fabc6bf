// MFMA GEMM for gfx950: C = A * op(B) with fused epilogues, for fp32 / fp16 / bf16 / int8 inputs.
//
// Tiling (64-wide wavefronts): a workgroup of WM x WN waves computes a BM x BN macro tile; each
// wave owns a (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks.  Operand panels are staged
// through LDS in k-slabs of 64 bytes per row, double buffered: the global loads of slab k+1 are
// issued into registers before the MFMAs of slab k and written to the other LDS buffer afterwards,
// so one barrier per slab suffices.  Both LDS panels are stored "row x k" (k contiguous), which is
// the order the MFMA operands want: a lane supplies 16 contiguous bytes of k for one row/column.
//
//   fp16 : v_mfma_f32_32x32x16_f16   (8 halfs per lane per operand)
//   bf16 : v_mfma_f32_32x32x16_bf16
//   int8 : v_mfma_i32_32x32x32_i8    (16 bytes per lane per operand), exact int32 accumulation
//   fp32 : 4 x v_mfma_f32_32x32x2f32 per 16-byte operand read
//
// The contraction index inside one MFMA is symmetric between the two operands, so any fixed
// assignment of k-values to (lane half, vector element) gives the same sum; both panels use the
// same one.
//
// Output layout of a 32x32 block: lane l holds column (l % 32); accumulator register r holds row
// 8*(r/4) + 4*(l/32) + (r%4).
#include <atomic>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "common.h"

using namespace tnn_rocm;

// Hook for scratch builds that include this file to time the tiled kernel from inside: TR_TL(i) marks point i of a
// workgroup's life (0 entry, 5 first slabs requested, 6 row sums added up, 1 first slab landed, 2 main loop done,
// 3 C stored, 4 kernel end).  The library itself compiles it to nothing.
#ifndef TR_TL
#define TR_TL(i)
#endif

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kSlabBytes  = 64;               // bytes of k per row per LDS slab
constexpr int kLdsStride  = kSlabBytes + 16;  // padded row stride in bytes (bank spread for b128 reads)

template <int DT> struct GemmTraits;
template <> struct GemmTraits<TNN_ROCM_F16> {
    typedef half_t elem;
    typedef f32x16 acc;
    static __device__ __forceinline__ void mma(const uint4 &a, const uint4 &b, acc &c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                   0);
    }
};
template <> struct GemmTraits<TNN_ROCM_BF16> {
    typedef bf16_bits elem;
    typedef f32x16 acc;
    static __device__ __forceinline__ void mma(const uint4 &a, const uint4 &b, acc &c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                    0, 0);
    }
};
template <> struct GemmTraits<TNN_ROCM_I8> {
    typedef int8_t elem;
    typedef i32x16 acc;
    static __device__ __forceinline__ void mma(const uint4 &a, const uint4 &b, acc &c) {
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a), __builtin_bit_cast(i32x4, b), c, 0, 0,
                                                  0);
    }
};
template <> struct GemmTraits<TNN_ROCM_F32> {
    typedef float elem;
    typedef f32x16 acc;
    static __device__ __forceinline__ void mma(const uint4 &a, const uint4 &b, acc &c) {
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
    }
};


// ---- epilogues ----------------------------------------------------------------------------------
// Optional abilities of an epilogue type, false where the type does not name them:
//   kEmitsRowSums  the epilogue's store8 returns the sum and the sum of squares of the eight values it stored, and the
//                  kernel leaves per tile column and row their totals over the tile's columns (LnResidualEpilogue)
//   kTakesRowSums  a LayerNorm-folding epilogue that is handed such sums by the kernel that produced its A operand,
//                  instead of taking them from the A fragments in the main loop
template <typename E, typename = void> struct EmitsRowSums : std::false_type {};
template <typename E> struct EmitsRowSums<E, typename std::enable_if<E::kEmitsRowSums>::type> : std::true_type {};
template <typename E, typename = void> struct TakesRowSums : std::false_type {};
template <typename E> struct TakesRowSums<E, typename std::enable_if<E::kTakesRowSums>::type> : std::true_type {};
//   kColArrays     the epilogue reads that many per-column float arrays (col_src(k, n)) in store8.  The tiled kernel
//                  copies the tile's columns of each into LDS once, after the main loop, and store8 takes them from
//                  there (cl[k * cs + j] for column j of the item): an item then waits for two LDS reads instead of
//                  for global loads that cannot be moved above the previous item's stores
//   kRowIn         likewise for one float2 per row (row_src(m)), handed to store8 by value
template <typename E, typename = void> struct ColArrays : std::integral_constant<int, 0> {};
template <typename E> struct ColArrays<E, typename std::enable_if<(E::kColArrays > 0)>::type> : std::integral_constant<int, E::kColArrays> {};
template <typename E, typename = void> struct RowIn : std::false_type {};
template <typename E> struct RowIn<E, typename std::enable_if<E::kRowIn>::type> : std::true_type {};
constexpr int kMaxRowSumBlocks = TNN_ROCM_MAX_ROW_SUM_BLOCKS;
template <typename E, typename = void> struct SumBlocks : std::integral_constant<int, 1> {};
template <typename E> struct SumBlocks<E, typename std::enable_if<E::kTakesRowSums>::type> : std::integral_constant<int, E::kSumBlocks> {};  // tile columns of a producer a consumer can add up (768 columns of 32)


template <int DT> struct FloatEpilogue {
    typedef typename Elem<DT>::type T;
    static constexpr bool kRowStats = false;
    int flags;
    const float *bias;
    const T *residual;
    long ldr;
    T *C;
    long ldc;
    long batch_stride_c;
    long batch_stride_r;
    __device__ __forceinline__ void set_batch(int b) {
        C += (size_t)b * batch_stride_c;
        if (residual)
            residual += (size_t)b * batch_stride_r;
    }
    __device__ __forceinline__ float col_const(int n) const { return (flags & TNN_ROCM_EPI_BIAS) ? bias[n] : 0.f; }
    __device__ __forceinline__ void store(int m, int n, float acc, float bias_n) const {
        float v = acc;
        if (flags & TNN_ROCM_EPI_BIAS)
            v = v + bias_n;
        if (flags & TNN_ROCM_EPI_GELU)
            v = gelu_erf(v);
        if (flags & TNN_ROCM_EPI_RESIDUAL)
            v = v + Elem<DT>::ld(&residual[(size_t)m * ldr + n]);
        Elem<DT>::st(&C[(size_t)m * ldc + n], v);
    }
    // true: this workgroup's columns go to a transposed layout, so the epilogue hands out rows to consecutive lanes
    __device__ __forceinline__ bool direct(int) const { return false; }
    // eight consecutive columns n..n+7 of row m (n % 8 == 0, n + 7 < N, rows 16-byte aligned): whole 16-byte
    // (half) / 32-byte (fp32) pieces, so that the lanes of one row together write full cache lines
    static constexpr int kColArrays = 1;  // bias
    __device__ __forceinline__ float col_src(int, int n) const { return (flags & TNN_ROCM_EPI_BIAS) ? bias[n] : 0.f; }
    // cl = the item's eight columns of the bias in LDS
    __device__ __forceinline__ void store8(int m, int n, const float (&acc)[8], const float *cl, int) const {
        float v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)
            v[t] = acc[t];
        if (flags & TNN_ROCM_EPI_BIAS) {
            float4 b0 = *reinterpret_cast<const float4 *>(cl), b1 = *reinterpret_cast<const float4 *>(cl + 4);
            v[0] += b0.x, v[1] += b0.y, v[2] += b0.z, v[3] += b0.w;
            v[4] += b1.x, v[5] += b1.y, v[6] += b1.z, v[7] += b1.w;
        }
        if (flags & TNN_ROCM_EPI_GELU) {
#pragma unroll
            for (int t = 0; t < 8; ++t)
                v[t] = (DT == TNN_ROCM_F32) ? gelu_erf(v[t]) : gelu_erf_fast(v[t]);
        }
        constexpr int NV = 8 * sizeof(T) / 16;  // 16-byte vectors per eight elements
        u32x4 packed[NV];
        T *pe = reinterpret_cast<T *>(packed);
        if (flags & TNN_ROCM_EPI_RESIDUAL) {
            const u32x4 *rp = reinterpret_cast<const u32x4 *>(residual + (size_t)m * ldr + n);
#pragma unroll
            for (int q = 0; q < NV; ++q)
                packed[q] = rp[q];
#pragma unroll
            for (int t = 0; t < 8; ++t)
                v[t] += Elem<DT>::ld(&pe[t]);
        }
#pragma unroll
        for (int t = 0; t < 8; ++t)
            Elem<DT>::st(&pe[t], v[t]);
        u32x4 *cp = reinterpret_cast<u32x4 *>(C + (size_t)m * ldc + n);
#pragma unroll
        for (int q = 0; q < NV; ++q)
            store_out16(&cp[q], packed[q]);
    }
};

// Where key s goes inside its V^T row.  sh = 0: at s.  sh = 1: inside every group of 16 keys the blocks of four
// k4-7 and k8-11 change places ([k0-3 | k8-11 | k4-7 | k12-15]), the order in which the lane halves of the attention
// kernel hold a tile's probabilities, so that kernel feeds them to its second MFMA without exchanging registers.
__device__ __forceinline__ int key_slot(int s, int sh) { return (s & ~12) | ((s & 4) << sh) | ((s & 8) >> sh); }

// QKV projection epilogue: columns [0,2H) -> qk[T,2H]; columns [2H,3H) -> V^T[b][head][d][s]
template <int DT> struct QkvSplitEpilogue {
    typedef typename Elem<DT>::type T;
    static constexpr bool kRowStats = false;
    const float *bias;
    T *qk;
    T *vt;
    int H, S, heads;
    int vt_sh;  // 0: V^T keys in natural order; 1: bits 2 and 3 of the key index change places (see key_slot)
    __device__ __forceinline__ void set_batch(int) {}
    __device__ __forceinline__ float col_const(int n) const { return bias ? bias[n] : 0.f; }
    __device__ __forceinline__ void store(int m, int n, float acc, float bias_n) const {
        float v = acc + bias_n;
        if (n < 2 * H) {
            Elem<DT>::st(&qk[(size_t)m * 2 * H + n], v);
        } else {
            int c = n - 2 * H, b = m / S, s = key_slot(m - b * S, vt_sh);
            Elem<DT>::st(&vt[(((size_t)b * heads + (c >> 6)) * 64 + (c & 63)) * S + s], v);
        }
    }
    // the V^T columns are written with consecutive lanes along s; Q|K rows with consecutive lanes along the row
    __device__ __forceinline__ bool direct(int n0) const { return n0 >= 2 * H; }
    static constexpr int kColArrays = 1;  // bias
    __device__ __forceinline__ float col_src(int, int n) const { return bias ? bias[n] : 0.f; }
    __device__ __forceinline__ void store8(int m, int n, const float (&acc)[8], const float *cl, int) const {
        float v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)
            v[t] = acc[t];
        if (bias) {
            float4 b0 = *reinterpret_cast<const float4 *>(cl), b1 = *reinterpret_cast<const float4 *>(cl + 4);
            v[0] += b0.x, v[1] += b0.y, v[2] += b0.z, v[3] += b0.w;
            v[4] += b1.x, v[5] += b1.y, v[6] += b1.z, v[7] += b1.w;
        }
        if (n < 2 * H) {
            constexpr int NV = 8 * sizeof(T) / 16;
            u32x4 packed[NV];
            T *pe = reinterpret_cast<T *>(packed);
#pragma unroll
            for (int t = 0; t < 8; ++t)
                Elem<DT>::st(&pe[t], v[t]);
            u32x4 *cp = reinterpret_cast<u32x4 *>(qk + (size_t)m * 2 * H + n);
#pragma unroll
            for (int q = 0; q < NV; ++q)
                store_out16(&cp[q], packed[q]);
        } else {
            int c = n - 2 * H, b = m / S, s_ = key_slot(m - b * S, vt_sh);
            T *dst = vt + (((size_t)b * heads + (c >> 6)) * 64 + (c & 63)) * S + s_;
#pragma unroll
            for (int t = 0; t < 8; ++t)
                Elem<DT>::st_out(dst + (size_t)t * S, v[t]);
        }
    }
};

// ---- LayerNorm folded into the projection that reads it ------------------------------------------------------------
// y = LayerNorm(t) over the last axis (cpu_layer_norm_layer_acc.cc:86-135: per row mean and variance,
// (t - mean) * rstd * gamma + beta) followed by y W^T + b, as one GEMM on the raw t:
//     y W^T + b = rstd * (t W'^T - mean * colsum) + b',   W' = gamma (.) W,  colsum[n] = sum_k W'[n,k],  b' = b + W beta.
// K is the normalised width, so every workgroup streams whole rows of t through LDS anyway: the row sums and sums of
// squares are taken from the A fragments the waves already hold for the MFMAs (two dot2 instructions per four
// values), reduced over the workgroup after the main loop, and applied to the accumulators in the epilogue.
// Other readers of y (the residual additions) still need the tensor: the workgroup of tile column j writes
// y for the j-th share of the columns of its rows, so the LayerNorm launch disappears without y disappearing.
std::atomic<int> g_ln_y_ahead{1};  // experiment hook, see tnn_rocm_debug_set_ln_y_ahead

struct LnFold {
    float inv_cols, eps;
    const float *colsum;        // [N]
    const float *gamma, *beta;  // [K], for the y side output
    void *y;                    // [M, K] in the compute type, or nullptr
    int y_ahead;                // 1: the source vectors of y are requested under the epilogue (0 for experiments)
    float2 *stats;              // [M] {rstd, mean} for a later kernel that rebuilds LayerNorm(t) itself, or nullptr
    const float2 *row_sums;     // kTakesRowSums: [sum_blocks][M] {sum, sum of squares} over a block of columns of t
    int sum_blocks;
};

// row sum and sum of squares of the eight values of an A fragment register quad
template <int DT> __device__ __forceinline__ void ln_accumulate(const uint4 &frag, float &s1, float &s2) {
    const uint32_t w[4] = {frag.x, frag.y, frag.z, frag.w};
    if constexpr (DT == TNN_ROCM_F16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 one = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            h2 v = __builtin_bit_cast(h2, w[t]);
            s1   = __builtin_amdgcn_fdot2(v, one, s1, false);
            s2   = __builtin_amdgcn_fdot2(v, v, s2, false);
        }
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            float lo = __uint_as_float(w[t] << 16), hi = __uint_as_float(w[t] & 0xffff0000u);
            s1 += lo + hi;
            s2 = fmaf(lo, lo, fmaf(hi, hi, s2));
        }
    }
}

// Element offset of (row m, column n) in a row-major matrix of leading dimension ld, for the epilogues whose entry
// points have checked rows < 2^24, ld < 2^24 and rows * ld < 2^31: one full-rate 24-bit multiply where the 64-bit
// product m * ld costs two v_mul_lo_u32 and a v_mad_u64_u32 (quarter rate each) per item.
__device__ __forceinline__ unsigned elem_offset24(int m, unsigned ld, int n) {
    return __umul24((unsigned)m, ld) + (unsigned)n;
}

// SUMS: 0 = the statistics come from the A fragments; else the most row-sum blocks the kernel is handed (12 or 24: that
// many register pairs hold them while they are in flight)
template <int DT, int SUMS = 0> struct LnFloatEpilogue {
    typedef typename Elem<DT>::type T;
    static constexpr bool kRowStats = true;
    static constexpr bool kTakesRowSums = SUMS > 0;
    static constexpr int kSumBlocks     = SUMS;
    int flags;
    const float *bias;  // b' (always present)
    const T *residual;
    T *C;
    long ldc;
    LnFold ln;
    __device__ __forceinline__ void set_batch(int) {}
    __device__ __forceinline__ float col_const(int) const { return 0.f; }
    __device__ __forceinline__ void store(int, int, float, float) const {}  // N % 8 == 0 is required at launch
    __device__ __forceinline__ bool direct(int) const { return false; }
    static constexpr int kColArrays = 2;  // colsum, b'
    __device__ __forceinline__ float col_src(int k, int n) const { return k == 0 ? ln.colsum[n] : bias[n]; }
    // st = {rstd, mean} of row m; cl = the item's eight columns of the two arrays in LDS, cs apart
    __device__ __forceinline__ void store8(int m, int n, const float (&acc)[8], float2 st, const float *cl, int cs) const {
        float4 g0 = *reinterpret_cast<const float4 *>(cl), g1 = *reinterpret_cast<const float4 *>(cl + 4);
        float4 b0 = *reinterpret_cast<const float4 *>(cl + cs), b1 = *reinterpret_cast<const float4 *>(cl + cs + 4);
        const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        float v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)
            v[t] = fmaf(st.x, fmaf(-st.y, g[t], acc[t]), b[t]);
        if (flags & TNN_ROCM_EPI_GELU) {
#pragma unroll
            for (int t = 0; t < 8; ++t)
                v[t] = gelu_erf_fast(v[t]);
        }
        // the two forms each end in their own conversion and store: joined behind the branch, the form without a
        // residual pays eight register copies per item for the join
        if (flags & TNN_ROCM_EPI_RESIDUAL) {
            constexpr int NV = 8 * sizeof(T) / 16;
            u32x4 packed[NV];
            const T *pe      = reinterpret_cast<const T *>(packed);
            const u32x4 *rp = reinterpret_cast<const u32x4 *>(residual + elem_offset24(m, (unsigned)ldc, n));
#pragma unroll
            for (int q = 0; q < NV; ++q)
                packed[q] = rp[q];
            float w[8];
#pragma unroll
            for (int t = 0; t < 8; ++t)
                w[t] = v[t] + Elem<DT>::ld(&pe[t]);
            convert_and_store(m, n, w);
        } else {
            convert_and_store(m, n, v);
        }
    }
    __device__ __forceinline__ void convert_and_store(int m, int n, const float (&v)[8]) const {
        constexpr int NV = 8 * sizeof(T) / 16;
        u32x4 packed[NV];
        T *pe = reinterpret_cast<T *>(packed);
#pragma unroll
        for (int t = 0; t < 8; ++t)
            Elem<DT>::st(&pe[t], v[t]);
        u32x4 *cp = reinterpret_cast<u32x4 *>(C + elem_offset24(m, (unsigned)ldc, n));
#pragma unroll
        for (int q = 0; q < NV; ++q)
            store_out16(&cp[q], packed[q]);
    }
};

// QKV projection of LayerNorm(t): QkvSplitEpilogue's layout with the folded-LayerNorm correction on the accumulators
template <int DT, int SUMS = 0> struct LnQkvSplitEpilogue {
    typedef typename Elem<DT>::type T;
    static constexpr bool kRowStats = true;
    static constexpr bool kTakesRowSums = SUMS > 0;
    static constexpr int kSumBlocks     = SUMS;
    const float *bias;
    T *qk;
    T *vt;
    int H, S, heads;
    int vt_sh;  // 0: V^T keys in natural order; 1: bits 2 and 3 of the key index change places (see key_slot)
    LnFold ln;
    __device__ __forceinline__ void set_batch(int) {}
    __device__ __forceinline__ float col_const(int) const { return 0.f; }
    __device__ __forceinline__ void store(int, int, float, float) const {}
    __device__ __forceinline__ bool direct(int n0) const { return n0 >= 2 * H; }
    static constexpr int kColArrays = 2;  // colsum, b'
    __device__ __forceinline__ float col_src(int k, int n) const { return k == 0 ? ln.colsum[n] : bias[n]; }
    __device__ __forceinline__ void store8(int m, int n, const float (&acc)[8], float2 st, const float *cl, int cs) const {
        float4 g0 = *reinterpret_cast<const float4 *>(cl), g1 = *reinterpret_cast<const float4 *>(cl + 4);
        float4 b0 = *reinterpret_cast<const float4 *>(cl + cs), b1 = *reinterpret_cast<const float4 *>(cl + cs + 4);
        const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        float v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)
            v[t] = fmaf(st.x, fmaf(-st.y, g[t], acc[t]), b[t]);
        if (n < 2 * H) {
            constexpr int NV = 8 * sizeof(T) / 16;
            u32x4 packed[NV];
            T *pe = reinterpret_cast<T *>(packed);
#pragma unroll
            for (int t = 0; t < 8; ++t)
                Elem<DT>::st(&pe[t], v[t]);
            u32x4 *cp = reinterpret_cast<u32x4 *>(qk + elem_offset24(m, 2u * (unsigned)H, n));
#pragma unroll
            for (int q = 0; q < NV; ++q)
                store_out16(&cp[q], packed[q]);
        } else {
            // B * S * 3H < 2^31 is checked at launch: 32-bit offsets throughout
            int c = n - 2 * H, bb = m / S, s_ = key_slot(m - bb * S, vt_sh);
            T *dst = vt + (unsigned)(((bb * heads + (c >> 6)) * 64 + (c & 63)) * S + s_);
#pragma unroll
            for (int t = 0; t < 8; ++t)
                Elem<DT>::st_out(dst + (unsigned)(t * S), v[t]);
        }
    }
};

// Projection whose residual operand is LayerNorm(t) of a tensor whose row statistics an earlier kernel left behind
// (LnFold::stats): C = act(x W^T + b) + ((t - mean) * rstd * gamma + beta).  The normalised tensor is rebuilt from t in
// registers, in the LayerNorm kernel's half-precision form x * rstd * gamma + (beta - mean * rstd * gamma), and never
// stored.  N is the normalised width.
template <int DT, bool SUMS = false> struct LnResidualEpilogue {
    typedef typename Elem<DT>::type T;
    static constexpr bool kRowStats = false;
    static constexpr bool kEmitsRowSums = SUMS;
    float2 *row_sums;  // kEmitsRowSums: [tile columns][M] {sum, sum of squares} of the stored values of C
    int flags;  // TNN_ROCM_EPI_BIAS, TNN_ROCM_EPI_GELU
    const float *bias;
    const T *t;                 // [M, N]
    const float2 *st;           // [M] {rstd, mean}
    const float *gamma, *beta;  // [N]
    T *C;
    long ldc;
    __device__ __forceinline__ void set_batch(int) {}
    __device__ __forceinline__ float col_const(int n) const { return (flags & TNN_ROCM_EPI_BIAS) ? bias[n] : 0.f; }
    __device__ __forceinline__ void store(int m, int n, float acc, float bias_n) const {
        float v = acc;
        if (flags & TNN_ROCM_EPI_BIAS)
            v = v + bias_n;
        if (flags & TNN_ROCM_EPI_GELU)
            v = gelu_erf(v);
        const float2 s = st[m];
        const float mrs = s.y * s.x;
        v = v + (Elem<DT>::ld(&t[(size_t)m * ldc + n]) * s.x * gamma[n] + (beta[n] - mrs * gamma[n]));
        Elem<DT>::st(&C[(size_t)m * ldc + n], v);
    }
    __device__ __forceinline__ bool direct(int) const { return false; }
    static constexpr int kColArrays = 3;  // bias (zeros without one), gamma, beta
    static constexpr bool kRowIn    = true;  // {rstd, mean} of the rows of t
    __device__ __forceinline__ float col_src(int k, int n) const {
        return k == 0 ? ((flags & TNN_ROCM_EPI_BIAS) ? bias[n] : 0.f) : k == 1 ? gamma[n] : beta[n];
    }
    __device__ __forceinline__ float2 row_src(int m) const { return st[m]; }
    // cl = the item's eight columns of the three arrays in LDS, cs apart; s = {rstd, mean} of row m
    __device__ __forceinline__ float2 store8(int m, int n, const float (&acc)[8], const float *cl, int cs, float2 s) const {
        static_assert(sizeof(T) == 2, "half-precision blobs only");
        const unsigned off = elem_offset24(m, (unsigned)ldc, n);
        u32x4 packed = *reinterpret_cast<const u32x4 *>(t + off);
        float v[8];
        {
            float4 b0 = *reinterpret_cast<const float4 *>(cl), b1 = *reinterpret_cast<const float4 *>(cl + 4);
            v[0] = acc[0] + b0.x, v[1] = acc[1] + b0.y, v[2] = acc[2] + b0.z, v[3] = acc[3] + b0.w;
            v[4] = acc[4] + b1.x, v[5] = acc[5] + b1.y, v[6] = acc[6] + b1.z, v[7] = acc[7] + b1.w;
        }
        if (flags & TNN_ROCM_EPI_GELU) {
#pragma unroll
            for (int q = 0; q < 8; ++q)
                v[q] = gelu_erf_fast(v[q]);
        }
        T *pe = reinterpret_cast<T *>(&packed);
        const float mrs = s.y * s.x;
        float4 k0 = *reinterpret_cast<const float4 *>(cl + cs), k1 = *reinterpret_cast<const float4 *>(cl + cs + 4);
        float4 e0 = *reinterpret_cast<const float4 *>(cl + 2 * cs), e1 = *reinterpret_cast<const float4 *>(cl + 2 * cs + 4);
        const float kk[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
        const float ee[8] = {e0.x, e0.y, e0.z, e0.w, e1.x, e1.y, e1.z, e1.w};
#pragma unroll
        for (int q = 0; q < 8; ++q)
            v[q] += Elem<DT>::ld(&pe[q]) * s.x * kk[q] + (ee[q] - mrs * kk[q]);
#pragma unroll
        for (int q = 0; q < 8; ++q)
            Elem<DT>::st(&pe[q], v[q]);
        store_out16(C + off, packed);
        float2 sums = make_float2(0.f, 0.f);
        if constexpr (SUMS) {  // of the values as stored (rounded to the blob type): what the next GEMM reads
            ln_accumulate<DT>(__builtin_bit_cast(uint4, packed), sums.x, sums.y);
        }
        return sums;
    }
};

struct Int8Epilogue {
    static constexpr bool kRowStats = false;
    // optional 256-entry table applied to the requantised value (index q + 128): an int8 -> int8 function that
    // followed the layer (dequantise, GELU, quantise) folded into this epilogue.  The tiled kernel keeps a copy in LDS.
    const int8_t *lut;
    const int32_t *bias;
    const float *scale;
    int8_t *out;
    int32_t *acc_out;
    long ldo;
    void *out_f;
    int out_f_dtype;
    float dq;
    const void *residual;  // optional, type and leading dimension of out_f: out_f = q * dq + residual
    __device__ __forceinline__ void set_batch(int) {}
    struct ColConst {
        int32_t bias;
        float scale;
    };
    __device__ __forceinline__ ColConst col_const(int n) const {
        ColConst c;
        c.bias  = bias ? bias[n] : 0;
        c.scale = scale ? scale[n] : 0.f;
        return c;
    }
    __device__ __forceinline__ void store(int m, int n, int acc, const ColConst &cc) const {
        int a = acc + cc.bias;
        if (acc_out)
            acc_out[(size_t)m * ldo + n] = a;
        if (out || out_f) {
            // (float)int32 rounds to nearest even, one fp32 multiply, then the +-0.5 add: three
            // separately rounded steps as on the CPU paths.
            float f  = __fmul_rn((float)a, cc.scale);
            int8_t q = float2int8_ref(f);
            if (lut)
                q = lut[(int)q + 128];
            if (out)
                out[(size_t)m * ldo + n] = q;
            if (out_f) {
                float d = __fmul_rn((float)q, dq);
                if (out_f_dtype == TNN_ROCM_F32) {
                    if (residual)
                        d = __fadd_rn(d, ((const float *)residual)[(size_t)m * ldo + n]);
                    ((float *)out_f)[(size_t)m * ldo + n] = d;
                } else {
                    if (residual)
                        d = __fadd_rn(d, (float)((const half_t *)residual)[(size_t)m * ldo + n]);
                    ((half_t *)out_f)[(size_t)m * ldo + n] = (half_t)d;
                }
            }
        }
    }
    __device__ __forceinline__ bool direct(int) const { return false; }
    // eight consecutive columns (n % 8 == 0, n + 7 < N, ldo % 8 == 0): same arithmetic as store(), vector accesses
    static constexpr int kColArrays = 2;  // bias (its int32 bits), scale
    __device__ __forceinline__ float col_src(int k, int n) const {
        return k == 0 ? (bias ? __int_as_float(bias[n]) : 0.f) : (scale ? scale[n] : 0.f);
    }
    // cl = the item's eight columns of the two arrays in LDS, cs apart
    __device__ __forceinline__ void store8(int m, int n, const int (&acc)[8], const int8_t *lut_lds, const float *cl, int cs) const {
        int a[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)
            a[t] = acc[t];
        if (bias) {
            i32x4 b0 = *reinterpret_cast<const i32x4 *>(cl), b1 = *reinterpret_cast<const i32x4 *>(cl + 4);
#pragma unroll
            for (int t = 0; t < 4; ++t)
                a[t] += b0[t], a[4 + t] += b1[t];
        }
        const size_t o = (size_t)m * ldo + n;
        if (acc_out) {
            i32x4 *ap = reinterpret_cast<i32x4 *>(acc_out + o);
            ap[0] = i32x4{a[0], a[1], a[2], a[3]};
            ap[1] = i32x4{a[4], a[5], a[6], a[7]};
        }
        if (out || out_f) {
            float sc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (scale) {
                float4 s0 = *reinterpret_cast<const float4 *>(cl + cs), s1 = *reinterpret_cast<const float4 *>(cl + cs + 4);
                sc[0] = s0.x, sc[1] = s0.y, sc[2] = s0.z, sc[3] = s0.w, sc[4] = s1.x, sc[5] = s1.y, sc[6] = s1.z, sc[7] = s1.w;
            }
            int8_t q[8];
#pragma unroll
            for (int t = 0; t < 8; ++t)
                q[t] = float2int8_ref(__fmul_rn((float)a[t], sc[t]));
            if (lut_lds) {
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    q[t] = lut_lds[(int)q[t] + 128];
            }
            if (out)
                store_out8(out + o, *reinterpret_cast<const store_u32x2 *>(q));
            if (out_f) {
                float d[8];
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    d[t] = __fmul_rn((float)q[t], dq);
                if (out_f_dtype == TNN_ROCM_F32) {
                    if (residual) {
                        const float4 *rp = reinterpret_cast<const float4 *>((const float *)residual + o);
                        float4 r0 = rp[0], r1 = rp[1];
                        d[0] = __fadd_rn(d[0], r0.x), d[1] = __fadd_rn(d[1], r0.y), d[2] = __fadd_rn(d[2], r0.z),
                        d[3] = __fadd_rn(d[3], r0.w), d[4] = __fadd_rn(d[4], r1.x), d[5] = __fadd_rn(d[5], r1.y),
                        d[6] = __fadd_rn(d[6], r1.z), d[7] = __fadd_rn(d[7], r1.w);
                    }
                    float4 *fp = reinterpret_cast<float4 *>((float *)out_f + o);
                    store_out16(fp, store_u32x4{__float_as_uint(d[0]), __float_as_uint(d[1]), __float_as_uint(d[2]),
                                                __float_as_uint(d[3])});
                    store_out16(fp + 1, store_u32x4{__float_as_uint(d[4]), __float_as_uint(d[5]), __float_as_uint(d[6]),
                                                    __float_as_uint(d[7])});
                } else {
                    half_t h[8];
                    if (residual) {
                        *reinterpret_cast<u32x4 *>(h) = *reinterpret_cast<const u32x4 *>((const half_t *)residual + o);
#pragma unroll
                        for (int t = 0; t < 8; ++t)
                            d[t] = __fadd_rn(d[t], (float)h[t]);
                    }
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        h[t] = (half_t)d[t];
                    store_out16((half_t *)out_f + o, *reinterpret_cast<const u32x4 *>(h));
                }
            }
        }
    }
};

// Quantised QKV projection for the attention layer: the int8 outputs of the three QuantizedInnerProduct layers are
// formed in registers (requantisation with scale[n] = w_scale[n] / o_scale of the column's section) and written
// already dequantised (q * dequant[n], the value the following Reformat layer produces) in the layout of
// QkvSplitEpilogue: columns [0,2H) -> qk[T,2H]; columns [2H,3H) -> V^T[b][head][d][s].
template <int DT> struct Int8QkvSplitEpilogue {
    typedef typename Elem<DT>::type T;
    static constexpr bool kRowStats = false;
    const int32_t *bias;
    const float *scale;
    const float *dequant;
    T *qk;
    T *vt;
    int H, S, heads;
    int vt_sh;  // 0: V^T keys in natural order; 1: bits 2 and 3 of the key index change places (see key_slot)
    __device__ __forceinline__ void set_batch(int) {}
    struct ColConst {
        int32_t bias;
        float scale, dq;
    };
    __device__ __forceinline__ ColConst col_const(int n) const {
        ColConst c;
        c.bias  = bias ? bias[n] : 0;
        c.scale = scale[n];
        c.dq    = dequant[n];
        return c;
    }
    __device__ __forceinline__ void store(int m, int n, int acc, const ColConst &cc) const {
        int8_t q = float2int8_ref(__fmul_rn((float)(acc + cc.bias), cc.scale));
        float v  = __fmul_rn((float)q, cc.dq);
        if (n < 2 * H) {
            Elem<DT>::st(&qk[(size_t)m * 2 * H + n], v);
        } else {
            int c = n - 2 * H, b = m / S, s = key_slot(m - b * S, vt_sh);
            Elem<DT>::st(&vt[(((size_t)b * heads + (c >> 6)) * 64 + (c & 63)) * S + s], v);
        }
    }
    __device__ __forceinline__ bool direct(int n0) const { return n0 >= 2 * H; }
    static constexpr int kColArrays = 3;  // bias (its int32 bits), scale, dequant
    __device__ __forceinline__ float col_src(int k, int n) const {
        return k == 0 ? (bias ? __int_as_float(bias[n]) : 0.f) : k == 1 ? scale[n] : dequant[n];
    }
    __device__ __forceinline__ void store8(int m, int n, const int (&acc)[8], const float *cl, int cs) const {
        // the item's eight columns of the three arrays, from LDS
        const i32x4 b0 = *reinterpret_cast<const i32x4 *>(cl), b1 = *reinterpret_cast<const i32x4 *>(cl + 4);
        const float4 s0 = *reinterpret_cast<const float4 *>(cl + cs), s1 = *reinterpret_cast<const float4 *>(cl + cs + 4);
        const float4 d0 = *reinterpret_cast<const float4 *>(cl + 2 * cs), d1 = *reinterpret_cast<const float4 *>(cl + 2 * cs + 4);
        const int bb[8]   = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
        const float sc[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        const float dq[8] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
        float v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            int8_t q = float2int8_ref(__fmul_rn((float)(acc[t] + bb[t]), sc[t]));
            v[t]     = __fmul_rn((float)q, dq[t]);
        }
        if (n < 2 * H) {
            constexpr int NV = 8 * sizeof(T) / 16;
            u32x4 packed[NV];
            T *pe = reinterpret_cast<T *>(packed);
#pragma unroll
            for (int t = 0; t < 8; ++t)
                Elem<DT>::st(&pe[t], v[t]);
            u32x4 *cp = reinterpret_cast<u32x4 *>(qk + (size_t)m * 2 * H + n);
#pragma unroll
            for (int q = 0; q < NV; ++q)
                store_out16(&cp[q], packed[q]);
        } else {
            int c = n - 2 * H, b = m / S, s_ = key_slot(m - b * S, vt_sh);
            T *dst = vt + (((size_t)b * heads + (c >> 6)) * 64 + (c & 63)) * S + s_;
#pragma unroll
            for (int t = 0; t < 8; ++t)
                Elem<DT>::st_out(dst + (size_t)t * S, v[t]);
        }
    }
};

// 16-byte panel fetch with zero fill outside [0,rows) x [0,K).  `row_major_k` panels have k
// contiguous in memory.
template <typename T, bool ALIGNED>
__device__ __forceinline__ uint4 fetch_k_contig(const T *__restrict__ base, long ld, int row, int rows, int k, int K) {
    constexpr int VEC = 16 / sizeof(T);
    uint4 r           = make_uint4(0, 0, 0, 0);
    if (row < rows) {
        const T *p = base + (size_t)row * ld + k;
        if (ALIGNED) {
            if (k < K)
                r = *reinterpret_cast<const uint4 *>(p);
        } else {
            T *e = reinterpret_cast<T *>(&r);
#pragma unroll
            for (int t = 0; t < VEC; ++t)
                if (k + t < K)
                    e[t] = p[t];
        }
    }
    return r;
}

// B given as [K,N] (n contiguous): fetch 16 bytes along n at row k.
template <typename T, bool ALIGNED>
__device__ __forceinline__ uint4 fetch_n_contig(const T *__restrict__ base, long ld, int k, int K, int n, int N) {
    constexpr int VEC = 16 / sizeof(T);
    uint4 r           = make_uint4(0, 0, 0, 0);
    if (k < K) {
        const T *p = base + (size_t)k * ld + n;
        if (ALIGNED) {
            if (n < N)
                r = *reinterpret_cast<const uint4 *>(p);
        } else {
            T *e = reinterpret_cast<T *>(&r);
#pragma unroll
            for (int t = 0; t < VEC; ++t)
                if (n + t < N)
                    e[t] = p[t];
        }
    }
    return r;
}

template <int DT, int BM, int BN, int WM, int WN, bool B_NK, bool ALIGNED, typename Epi>
__global__ void __launch_bounds__(WM *WN * 64)
    gemm_kernel(const typename GemmTraits<DT>::elem *__restrict__ A, const typename GemmTraits<DT>::elem *__restrict__ B,
                int M, int N, int K, long lda, long ldb, int batch_a, int batch_b, long stride_a, long stride_b,
                int tiles_m, int tiles_n, Epi epi) {
    typedef typename GemmTraits<DT>::elem T;
    typedef typename GemmTraits<DT>::acc Acc;
    constexpr int NT      = WM * WN * 64;
    constexpr int VEC     = 16 / sizeof(T);
    constexpr int KB      = kSlabBytes / sizeof(T);  // k elements per slab
    constexpr int MT      = BM / WM / 32;
    constexpr int NTL     = BN / WN / 32;
    constexpr int A_VECS  = BM * 4 / NT;  // 16-byte vectors of the A slab per thread
    constexpr int B_VECS  = BN * 4 / NT;
    static_assert(BM * 4 % NT == 0 && BN * 4 % NT == 0, "slab must divide evenly over the workgroup");
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be a multiple of 32x32");

    __shared__ __attribute__((aligned(16))) unsigned char lds_a[2][BM * kLdsStride];
    __shared__ __attribute__((aligned(16))) unsigned char lds_b[2][BN * kLdsStride];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm   = wave / WN;
    const int wn   = wave % WN;

    // XCD-aware tile order: workgroups are dealt round-robin to the 8 XCDs, so give each XCD a
    // contiguous run of tiles (shared A row panels stay in one L2).
    int pid           = blockIdx.x;
    const int n_tiles = tiles_m * tiles_n;
    if ((n_tiles & 7) == 0) {
        pid = (pid & 7) * (n_tiles >> 3) + (pid >> 3);
    }
    const int tm = pid / tiles_n;
    const int tn = pid % tiles_n;
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const int bz = blockIdx.y;
    A += (size_t)(bz % batch_a) * stride_a;
    B += (size_t)(bz % batch_b) * stride_b;
    epi.set_batch(bz);

    uint4 ra[A_VECS], rb[B_VECS];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_VECS; ++i) {
            int v   = tid + i * NT;
            int row = v >> 2, kc = (v & 3) * VEC;
            ra[i] = fetch_k_contig<T, ALIGNED>(A, lda, m0 + row, M, k0 + kc, K);
        }
        if (B_NK) {
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) {
                int v   = tid + i * NT;
                int row = v >> 2, kc = (v & 3) * VEC;
                rb[i] = fetch_k_contig<T, ALIGNED>(B, ldb, n0 + row, N, k0 + kc, K);
            }
        } else {
            // slab is KB rows (k) x BN columns (n): BN/VEC vectors per k row
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) {
                int v  = tid + i * NT;
                int kr = v / (BN / VEC), nc = (v % (BN / VEC)) * VEC;
                rb[i] = fetch_n_contig<T, ALIGNED>(B, ldb, k0 + kr, K, n0 + nc, N);
            }
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_VECS; ++i) {
            int v   = tid + i * NT;
            int row = v >> 2, kc = (v & 3);
            *reinterpret_cast<uint4 *>(&lds_a[buf][row * kLdsStride + kc * 16]) = ra[i];
        }
        if (B_NK) {
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) {
                int v   = tid + i * NT;
                int row = v >> 2, kc = (v & 3);
                *reinterpret_cast<uint4 *>(&lds_b[buf][row * kLdsStride + kc * 16]) = rb[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) {
                int v  = tid + i * NT;
                int kr = v / (BN / VEC), nc = (v % (BN / VEC)) * VEC;
                const T *e = reinterpret_cast<const T *>(&rb[i]);
#pragma unroll
                for (int t = 0; t < VEC; ++t)
                    *reinterpret_cast<T *>(&lds_b[buf][(nc + t) * kLdsStride + kr * (int)sizeof(T)]) = e[t];
            }
        }
    };

    Acc acc[MT][NTL];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NTL; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0;

    const int nk = (K + KB - 1) / KB;
    load_global(0);
    store_lds(0);
    __syncthreads();

    const int frag_row = lane & 31;
    const int frag_off = (lane >> 5) * 16;

    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk)
            load_global((kt + 1) * KB);
#pragma unroll
        for (int kk = 0; kk < kSlabBytes / 32; ++kk) {
            uint4 fa[MT], fb[NTL];
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                int row = wm * (BM / WM) + i * 32 + frag_row;
                fa[i]   = *reinterpret_cast<const uint4 *>(&lds_a[buf][row * kLdsStride + kk * 32 + frag_off]);
            }
#pragma unroll
            for (int j = 0; j < NTL; ++j) {
                int row = wn * (BN / WN) + j * 32 + frag_row;
                fb[j]   = *reinterpret_cast<const uint4 *>(&lds_b[buf][row * kLdsStride + kk * 32 + frag_off]);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NTL; ++j)
                    GemmTraits<DT>::mma(fa[i], fb[j], acc[i][j]);
        }
        if (kt + 1 < nk)
            store_lds(buf ^ 1);
        __syncthreads();
    }

    // epilogue: lane = column, registers = rows
#pragma unroll
    for (int j = 0; j < NTL; ++j) {
        int n = n0 + wn * (BN / WN) + j * 32 + (lane & 31);
        if (n < N) {
            auto cc = epi.col_const(n);
#pragma unroll
            for (int i = 0; i < MT; ++i) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    int m = m0 + wm * (BM / WM) + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    if (m < M)
                        epi.store(m, n, acc[i][j][r], cc);
                }
            }
        }
    }
}


// ---- tiled, pipelined kernel for the aligned x * W^T case ----------------------------------------------
// One workgroup of four or eight waves (one or two per SIMD) per output tile.  The waves form a WGM x WGN x WGK grid: a wave
// owns a (32*TM) x (32*TN) block of the tile and, when WGK > 1, every WGK-th 32-byte k-step of each slab
// (the partial sums of the WGK waves are added in the epilogue).  Tile = (32*TM*WGM) x (32*TN*WGN).
//   * the launcher picks the shape so that the tile count is at most (or a multiple of) the CU count with
//     tiles as large as registers allow: fewer bytes per flop from L2 and LDS, no second partial round;
//   * k-slabs of SLAB bytes per row; two slabs in flight in registers in addition to the one being consumed
//     from LDS (global loads for slab k+2 are issued before the MFMAs of slab k);
//   * the MFMA operands are swapped (the W panel is the "A" operand), so a lane owns one output ROW and
//     four consecutive columns per accumulator group;
//   * the epilogue turns the accumulators through LDS into a row-contiguous layout, so C, bias and residual
//     move as whole cache lines.
// LDS is dynamic: max(2 buffers x (BM + BN) rows x (SLAB + 16) bytes, 4 x 32 x (32*TN + 4) words of staging).
// NSTAGE = 0: slabs travel global -> registers -> LDS (padded rows, two LDS buffers).
// NSTAGE = 2 or 3: slabs travel global -> LDS directly (global_load_lds_dwordx4: no staging registers and no LDS
//     store instructions), into NSTAGE un-padded buffers whose 16-byte chunks are XOR-swizzled per row so that the
//     fragment reads stay free of bank conflicts; loads run NSTAGE-1 slabs ahead of the MFMAs.
template <int TM_, int TN_, int WGM_, int WGN_, int WGK_, int SLAB_, int NSTAGE_ = 0> struct TileCfg {
    static constexpr int TM = TM_, TN = TN_, WGM = WGM_, WGN = WGN_, WGK = WGK_, SLAB = SLAB_, NSTAGE = NSTAGE_;
    static constexpr int BM = 32 * TM * WGM, BN = 32 * TN * WGN;
    static constexpr int STRIDE = NSTAGE_ ? SLAB : SLAB + 16;
    static constexpr int SSTR   = 32 * TN + 4;  // staged row stride in 32-bit words
    static constexpr size_t slab_bytes  = (size_t)(NSTAGE_ ? NSTAGE_ : 2) * (BM + BN) * STRIDE;
    static constexpr size_t stage_bytes = (size_t)WGM_ * WGN_ * WGK_ * 32 * SSTR * 4;
    static constexpr size_t lds_bytes   = slab_bytes > stage_bytes ? slab_bytes : stage_bytes;
    // where an epilogue that leaves row sums keeps its BM x BN / 8 pairs: in the part of the slab area the staging does
    // not reach when that is large enough (dead by then), else behind everything
    static constexpr size_t sums_bytes  = (size_t)BM * BN;
    static constexpr size_t sums_offset = (slab_bytes >= stage_bytes + sums_bytes) ? stage_bytes : lds_bytes;
    static constexpr int NW = WGM * WGN * WGK, NT = 64 * NW;  // waves and threads per workgroup
    static_assert(NW == 4 || NW == 8, "four or eight waves per workgroup");
    static_assert((SLAB / 32) % WGK == 0, "k-steps of a slab must split evenly over the k-waves");
    static_assert((BM * (SLAB / 16)) % NT == 0 && (BN * (SLAB / 16)) % NT == 0, "slab must divide over the workgroup");
    static_assert(NSTAGE_ == 0 || NSTAGE_ == 2 || NSTAGE_ == 3, "register-staged, or two / three direct-to-LDS stages");
};

// Dynamic LDS of one (tile shape, epilogue) pair, for the kernel and its launcher alike: the slab / staging area, what
// the epilogue keeps behind it, and at the very end the tile's columns of the epilogue's per-column arrays followed by
// its per-row pairs.
template <typename CFG, typename Epi> struct EpiLds {
    static constexpr size_t lut_need   = CFG::stage_bytes + 256;  // Int8Epilogue's table behind the staging area
    static constexpr size_t stats_need = CFG::stage_bytes + (size_t)CFG::BM * 8 * (1 + 2 * CFG::WGK * CFG::WGN);
    static constexpr size_t base0 = std::is_same<Epi, Int8Epilogue>::value && lut_need > CFG::lds_bytes ? lut_need : CFG::lds_bytes;
    // row statistics and the partial-sum buffer sit behind the staging area; handed-over sums park {rstd, mean} per row
    // behind the slabs before the main loop
    static constexpr size_t base1 = TakesRowSums<Epi>::value ? CFG::lds_bytes + (size_t)CFG::BM * 8
                                    : (Epi::kRowStats && stats_need > base0) ? stats_need : base0;
    // without / with the row-sum side output (eight bytes per eight columns and row)
    static constexpr size_t plain     = base1;
    static constexpr size_t with_sums = CFG::sums_offset + CFG::sums_bytes > base1 ? CFG::sums_offset + CFG::sums_bytes : base1;
    static constexpr size_t front      = EmitsRowSums<Epi>::value ? with_sums : plain;
    static constexpr size_t col_offset = (front + 15) & ~(size_t)15;
    static constexpr size_t row_offset = col_offset + (size_t)ColArrays<Epi>::value * CFG::BN * 4;
    static constexpr size_t side_bytes = (size_t)ColArrays<Epi>::value * CFG::BN * 4 + (RowIn<Epi>::value ? (size_t)CFG::BM * 8 : 0);
    static constexpr size_t total      = col_offset + side_bytes;
};

// s_waitcnt that waits only for the vector-memory counter to drop to n (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4 and lgkmcnt 11:8 left at their maxima)
#define TR_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt((((n)&0xF) | ((((n) >> 4) & 3) << 14) | (0x7 << 4) | (0xF << 8)))

template <int DT, typename CFG, typename Epi>
__global__ void __launch_bounds__(CFG::NT)
    gemm_nk_tiled_kernel(const typename GemmTraits<DT>::elem *__restrict__ A,
                         const typename GemmTraits<DT>::elem *__restrict__ B, int M, int N, int K, long lda, long ldb,
                         int tiles_m, int tiles_n, int group_m, Epi epi) {
    typedef typename GemmTraits<DT>::elem T;
    typedef typename GemmTraits<DT>::acc Acc;
    constexpr int TM = CFG::TM, TN = CFG::TN, WGN = CFG::WGN, WGK = CFG::WGK, SLAB = CFG::SLAB;
    constexpr int BM = CFG::BM, BN = CFG::BN, STRIDE = CFG::STRIDE;
    constexpr int NT     = CFG::NT;
    constexpr int VEC    = 16 / sizeof(T);
    constexpr int KB     = SLAB / sizeof(T);
    constexpr int VPR    = SLAB / 16;  // 16-byte vectors per slab row
    constexpr int A_VECS = BM * VPR / NT;
    constexpr int B_VECS = BN * VPR / NT;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_dyn[];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wk   = wave % WGK;
    const int wn   = (wave / WGK) % WGN;
    const int wm   = wave / (WGK * WGN);

    // Tile order.  Workgroups are dealt round-robin to the 8 XCDs, each with its own 4 MB L2, and run roughly in
    // launch order.  Every XCD takes a contiguous run of a "grouped" tile order (group_m tile rows at a time, down
    // the rows first, then the next tile column), so the tiles that are resident together on one XCD form a
    // compact block of the tile grid: their A and W panels fit that L2 and are fetched from HBM once, instead of
    // the whole W panel streaming through every L2 once per tile row.
    TR_TL(0);  // entry
    const int n_tiles = tiles_m * tiles_n;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int vid     = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (vid >= n_tiles)
        return;  // the grid is padded to a multiple of 8; whole workgroups leave before any barrier
    const int group_sz = group_m * tiles_n;
    const int grp      = vid / group_sz;
    const int first_m  = grp * group_m;
    const int rows_g   = tiles_m - first_m < group_m ? tiles_m - first_m : group_m;
    const int in_grp   = vid - grp * group_sz;
    const int m0       = (first_m + in_grp % rows_g) * BM;
    const int n0       = (in_grp / rows_g) * BN;

    Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0;

    const int frag_row = lane & 31;
    const int frag_off = (lane >> 5) * 16;
    const int nk       = K / KB;

    // LayerNorm-folding epilogues: this lane's share of sum / sum of squares of A row (wm * TM + i) * 32 + frag_row
    float ln_s1[TM], ln_s2[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
        ln_s1[i] = ln_s2[i] = 0.f;

    if constexpr (CFG::NSTAGE > 0) {
        // Direct-to-LDS pipeline.  One load instruction of a wave fills 1024 contiguous LDS bytes (lane L writes
        // bytes 16L..16L+15), i.e. RPL whole slab rows; the lane picks WHICH 16 global bytes land there, so the
        // swizzle is applied on the global side: physical chunk p of LDS row r holds logical chunk p ^ f(r),
        // f(r) = (r / rows per 256 bytes) mod VPR.  Sixteen consecutive rows reading the same logical chunk then
        // touch sixteen different 16-byte bank groups.
        constexpr int NS    = CFG::NSTAGE;
        constexpr int RPL   = 1024 / SLAB;        // slab rows per wave-load
        constexpr int R256  = 256 / SLAB > 0 ? 256 / SLAB : 1;
        constexpr int A_LD  = BM / RPL / CFG::NW;  // wave-loads of A per wave and slab
        constexpr int B_LD  = BN / RPL / CFG::NW;
        constexpr int STAGE = (BM + BN) * SLAB;
        static_assert(BM % (RPL * CFG::NW) == 0 && BN % (RPL * CFG::NW) == 0, "slab rows must divide over the waves");
        static_assert((NS - 1) * (A_LD + B_LD) < 64, "look-ahead must fit the vmcnt counter");
        uint32_t a_off[A_LD], b_off[B_LD];
        const int lrow = lane / VPR, lpos = lane % VPR;
#pragma unroll
        for (int i = 0; i < A_LD; ++i) {
            const int r = (wave + i * CFG::NW) * RPL + lrow;
            int row     = m0 + r;
            row         = row < M ? row : M - 1;
            a_off[i]    = (uint32_t)row * (uint32_t)lda + (uint32_t)((lpos ^ ((r / R256) % VPR)) * VEC);
        }
#pragma unroll
        for (int i = 0; i < B_LD; ++i) {
            const int r = (wave + i * CFG::NW) * RPL + lrow;
            int row     = n0 + r;
            row         = row < N ? row : N - 1;
            b_off[i]    = (uint32_t)row * (uint32_t)ldb + (uint32_t)((lpos ^ ((r / R256) % VPR)) * VEC);
        }
        // The load is spelled as inline assembly on purpose: for the compiler's own global_load_lds builtin the
        // wait-count pass puts vmcnt(0) in front of every later LDS read (it cannot tell the stages apart), which
        // serialises the pipeline.  Here the waits are placed by hand (TR_WAIT_VMCNT below); the kernel issues no
        // other vector-memory operation until the loop has drained.  m0 carries the wave-uniform LDS address and
        // needs one wait state before the load.
        const uint32_t lds_base = (uint32_t)(uintptr_t)lds_dyn;  // generic -> LDS offset (low 32 bits of the aperture address)
        const uint32_t wave_dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_base + (uint32_t)wave * 1024u));
        auto load16 = [](const T *base, uint32_t byte_off, uint32_t lds_addr) {
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :
                         : "v"(byte_off), "s"(base), "s"(lds_addr)
                         : "memory", "m0");
        };
        auto issue = [&](int slab, int stage) {
            const uint32_t dst = wave_dst + (uint32_t)(stage * STAGE);
            const T *ga = A + (size_t)slab * KB, *gb = B + (size_t)slab * KB;
#pragma unroll
            for (int i = 0; i < A_LD; ++i)
                load16(ga, a_off[i] * (uint32_t)sizeof(T), dst + i * CFG::NW * 1024);
#pragma unroll
            for (int i = 0; i < B_LD; ++i)
                load16(gb, b_off[i] * (uint32_t)sizeof(T), dst + BM * SLAB + i * CFG::NW * 1024);
        };
        // byte offset of this lane's fragment chunk inside a slab row, per k-step of the slab
        const int fswz = (frag_row / R256) % VPR;
        const int frow = frag_row * SLAB;
        auto compute = [&](int stage) {
            const unsigned char *sa = lds_dyn + stage * STAGE, *sb = sa + BM * SLAB;
#pragma unroll
            for (int kk = wk; kk < SLAB / 32; kk += WGK) {
                const int chunk = ((kk * 2 + (lane >> 5)) ^ fswz) * 16;
                uint4 fa[TM], fb[TN];
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    fa[i] = *reinterpret_cast<const uint4 *>(sa + (wm * TM + i) * 32 * SLAB + frow + chunk);
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    fb[j] = *reinterpret_cast<const uint4 *>(sb + (wn * TN + j) * 32 * SLAB + frow + chunk);
                if constexpr (Epi::kRowStats && !TakesRowSums<Epi>::value) {
                    // the WGN waves that hold the same A rows take turns over the row groups and k-steps
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        if ((i + kk / WGK) % WGN == wn)
                            ln_accumulate<DT>(fa[i], ln_s1[i], ln_s2[i]);
                }
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        GemmTraits<DT>::mma(fb[j], fa[i], acc[i][j]);
            }
        };
        constexpr int LPW = A_LD + B_LD;
        // A folding epilogue that is handed the row sums of A: the first BM threads request their row's sums (one
        // 8-byte load per tile column of the kernel that wrote A), add them up and park {rstd, mean} behind everything
        // else in LDS, where the epilogue finds them.  In the early form the loads are spelled as assembly like the
        // slab loads and the wait is placed by hand: the compiler knows nothing of the slabs in flight, and the wait it
        // would place itself (everything outstanding) would also wait for the slabs requested after the sums.  In the
        // late form they are ordinary loads.  When:
        //   late  (tile shapes that have a CU to themselves, hence registers to spare, and any shape when at most twelve
        //         blocks are handed over: 24 registers): once the last slab is in LDS.
        //         Nothing stands between the kernel's entry and its first slabs, the loads' latency passes under the
        //         last slab's MFMAs, and the sums are added up after the loop while the other waves are on their way
        //         to the barrier that follows it.  They are the youngest loads of the kernel: wait for all.
        //   early (shapes that share a CU, with up to 24 blocks: the 48 registers the sums would occupy through the last
        //         slab would cost a resident workgroup): before the first slabs, added up while those are on their way.  Older than
        //         every slab load, they are complete once at most the slab loads are outstanding.
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        constexpr int NSUM      = SumBlocks<Epi>::value;
        constexpr bool kLateSums = TakesRowSums<Epi>::value && (EpiLds<CFG, Epi>::total > 80 * 1024 || NSUM <= 12);
        f32x2 early[NSUM];
        auto request_sums = [&]() __attribute__((always_inline)) {
            if constexpr (TakesRowSums<Epi>::value) {
                if (tid < BM) {
                    const int m = m0 + tid < M ? m0 + tid : M - 1;
#pragma unroll
                    for (int q = 0; q < NSUM; ++q) {
                        early[q] = f32x2{0.f, 0.f};
                        if (q < epi.ln.sum_blocks) {
                            if constexpr (kLateSums)
                                // ordinary loads: they are the youngest of the kernel, so the wait the compiler puts in
                                // front of their first use (everything outstanding) is the wait that is wanted, and
                                // the compiler knows the registers are not valid before it
                                early[q] = *reinterpret_cast<const f32x2 *>(
                                    reinterpret_cast<const char *>(epi.ln.row_sums) + ((size_t)q * M + m) * sizeof(float2));
                            else
                                asm volatile("global_load_dwordx2 %0, %1, %2"
                                             : "=v"(early[q])
                                             : "v"((uint32_t)(((size_t)q * M + m) * sizeof(float2))), "s"(epi.ln.row_sums)
                                             : "memory");
                        }
                    }
                }
            }
        };
        // slab_loads_behind: slab loads requested after the sums that may still be outstanding when the sums are read
        auto finish_sums = [&](int slab_loads_behind) __attribute__((always_inline)) {
            if constexpr (TakesRowSums<Epi>::value) {
                if (tid < BM) {
                    if constexpr (!kLateSums) {
                        if (slab_loads_behind >= 2)
                            TR_WAIT_VMCNT(2 * LPW);
                        else if (slab_loads_behind == 1)
                            TR_WAIT_VMCNT(LPW);
                        else
                            TR_WAIT_VMCNT(0);
                    }
                    // The other waves wait at a barrier while these do this, so it is kept short: the block sums (fp32)
                    // are added up in double in a fixed order (the sum of squares of a row that sits far from zero
                    // would lose the variance's digits in fp32), the variance is formed as a difference of doubles,
                    // and its reciprocal root is taken in single precision with one Newton step.
                    double f1 = 0.0, f2 = 0.0;
#pragma unroll
                    for (int q = 0; q < NSUM; ++q) {
                        if constexpr (!kLateSums)
                            asm volatile("" : "+v"(early[q]));  // not to be read before the wait above
                        if (q < epi.ln.sum_blocks) {
                            f1 += (double)early[q].x;
                            f2 += (double)early[q].y;
                        }
                    }
                    const double mean = f1 * (double)epi.ln.inv_cols;
                    // fp32 block sums can leave E[x^2] - mean^2 a hair below zero for rows whose spread is tiny next to
                    // their mean; the variance is clamped there (with eps = 1e-12 the root would otherwise be NaN)
                    const double var  = f2 * (double)epi.ln.inv_cols - mean * mean;
                    const float ve    = (float)((var > 0.0 ? var : 0.0) + (double)epi.ln.eps);
                    float r           = __builtin_amdgcn_rsqf(ve);
                    r                 = r * (1.5f - 0.5f * ve * r * r);
                    reinterpret_cast<float2 *>(lds_dyn + CFG::lds_bytes)[tid] = make_float2(r, (float)mean);
                }
            }
        };
        if constexpr (TakesRowSums<Epi>::value && !kLateSums)
            request_sums();
        int issued = 0;
#pragma unroll
        for (int p = 0; p < NS - 1; ++p)
            if (p < nk)
                issue(p, p), ++issued;
        TR_TL(5);  // first slabs requested
        if constexpr (TakesRowSums<Epi>::value && !kLateSums) {
            finish_sums(issued);
            TR_TL(6);  // handed-over row sums added up
        }
        int stage = 0, fill = NS - 1;  // stage of slab kt; stage that slab kt + NS - 1 goes to
        // one slab; with_sums (the last slab in the late form) also requests the row sums
        auto step = [&](int kt, auto with_sums) __attribute__((always_inline)) {
            // slab kt has landed once at most the loads of the slabs issued after it are outstanding
            if (NS == 3 && kt + 1 < nk)
                TR_WAIT_VMCNT(LPW);
            else
                TR_WAIT_VMCNT(0);
            // everyone's part of slab kt is in LDS, and everyone is done reading slab kt - 1 (its fragments were
            // consumed by MFMAs already issued).  A bare barrier: __syncthreads() adds a fence that waits for
            // every outstanding load, the look-ahead ones included.
            __builtin_amdgcn_s_barrier();
            if (kt == 0)
                TR_TL(1);  // first slab landed
            asm volatile("" ::: "memory");  // no LDS access may be moved across the barrier by the compiler
            if (kt + NS - 1 < nk)
                issue(kt + NS - 1, fill);
            if constexpr (decltype(with_sums)::value)
                request_sums();
            compute(stage);
            stage = stage + 1 == NS ? 0 : stage + 1;
            fill  = fill + 1 == NS ? 0 : fill + 1;
        };
        if constexpr (kLateSums) {
            // the last slab apart, so that the requested sums cross no loop edge on their way to the wait
            for (int kt = 0; kt + 1 < nk; ++kt)
                step(kt, std::false_type());
            step(nk - 1, std::true_type());
            finish_sums(0);
            TR_TL(6);  // handed-over row sums added up
        } else {
            for (int kt = 0; kt < nk; ++kt)
                step(kt, std::false_type());
        }
    } else {
    u32x4 ra0[A_VECS], rb0[B_VECS], ra1[A_VECS], rb1[B_VECS];

    // Loads carry no bounds branches: rows past the matrix edge are clamped to the last row (their products
    // land in accumulators that the epilogue never stores) and K is a whole number of slabs (checked by the
    // launcher), so every global load of a slab can be in flight at once.
    // vector v = tid + i*NT sits in slab row v / VPR at 16-byte column v % VPR; NT is a multiple of VPR, so
    // the column is the same for every i and the row advances by NT / VPR
    constexpr int ROW_STEP = NT / VPR;
    const int vrow = tid / VPR, vcol = tid % VPR;
    uint32_t a_off[A_VECS], b_off[B_VECS];  // element offsets (the launcher checks they fit 32 bits)
#pragma unroll
    for (int i = 0; i < A_VECS; ++i) {
        int row  = m0 + vrow + i * ROW_STEP;
        row      = row < M ? row : M - 1;
        a_off[i] = (uint32_t)row * (uint32_t)lda + (uint32_t)(vcol * VEC);
    }
#pragma unroll
    for (int i = 0; i < B_VECS; ++i) {
        int row  = n0 + vrow + i * ROW_STEP;
        row      = row < N ? row : N - 1;
        b_off[i] = (uint32_t)row * (uint32_t)ldb + (uint32_t)(vcol * VEC);
    }
// The three pipeline stages are macros on purpose: passing the register arrays through lambdas kept them in
// scratch memory (the compiler did not promote them), which costs more than the prefetch gains.
#define TR_LOAD_GLOBAL(RA, RB, K0)                                                                                    \
    {                                                                                                                 \
        _Pragma("unroll") for (int i = 0; i < A_VECS; ++i) RA[i] =                                                    \
            *reinterpret_cast<const u32x4 *>(A + a_off[i] + (K0));                                                    \
        _Pragma("unroll") for (int i = 0; i < B_VECS; ++i) RB[i] =                                                    \
            *reinterpret_cast<const u32x4 *>(B + b_off[i] + (K0));                                                    \
    }
#define TR_STORE_LDS(BUF, RA, RB)                                                                                     \
    {                                                                                                                 \
        _Pragma("unroll") for (int i = 0; i < A_VECS; ++i) *reinterpret_cast<u32x4 *>(                                \
            lds_a##BUF + (vrow + i * ROW_STEP) * STRIDE + vcol * 16) = RA[i];                                         \
        _Pragma("unroll") for (int i = 0; i < B_VECS; ++i) *reinterpret_cast<u32x4 *>(                                \
            lds_b##BUF + (vrow + i * ROW_STEP) * STRIDE + vcol * 16) = RB[i];                                         \
    }
#define TR_COMPUTE(BUF)                                                                                               \
    {                                                                                                                 \
        _Pragma("unroll") for (int kk = wk; kk < SLAB / 32; kk += WGK) {                                              \
            uint4 fa[TM], fb[TN];                                                                                     \
            _Pragma("unroll") for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const uint4 *>(                  \
                lds_a##BUF + ((wm * TM + i) * 32 + frag_row) * STRIDE + kk * 32 + frag_off);                          \
            _Pragma("unroll") for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const uint4 *>(                  \
                lds_b##BUF + ((wn * TN + j) * 32 + frag_row) * STRIDE + kk * 32 + frag_off);                          \
            _Pragma("unroll") for (int i = 0; i < TM; ++i) _Pragma("unroll") for (int j = 0; j < TN; ++j)             \
                GemmTraits<DT>::mma(fb[j], fa[i], acc[i][j]); /* rows of D = n, lanes of D = m */                     \
        }                                                                                                             \
    }

    unsigned char *const lds_a0 = lds_dyn, *const lds_b0 = lds_dyn + BM * STRIDE;
    unsigned char *const lds_a1 = lds_dyn + (BM + BN) * STRIDE, *const lds_b1 = lds_a1 + BM * STRIDE;

    // Slab schedule (two slabs in flight in registers, one in LDS being consumed).  The loop body is branch
    // free: look-ahead loads past the last slab are clamped to it and their LDS copy is never consumed.
    // (Forcing the look-ahead loads to the top of each phase with sched_barrier was measured slower: the
    // compiler's own interleaving of loads, LDS traffic and MFMAs is kept.)
    const int last = (nk - 1) * KB;
#define TR_CLAMPK(SLABIDX) (((SLABIDX)*KB) < last ? ((SLABIDX)*KB) : last)
    TR_LOAD_GLOBAL(ra0, rb0, 0);
    TR_LOAD_GLOBAL(ra1, rb1, TR_CLAMPK(1));
    TR_STORE_LDS(0, ra0, rb0);
    __syncthreads();
    for (int kt = 0; kt + 2 <= nk; kt += 2) {
        TR_LOAD_GLOBAL(ra0, rb0, TR_CLAMPK(kt + 2));
        TR_COMPUTE(0);
        TR_STORE_LDS(1, ra1, rb1);
        __syncthreads();
        TR_LOAD_GLOBAL(ra1, rb1, TR_CLAMPK(kt + 3));
        TR_COMPUTE(1);
        TR_STORE_LDS(0, ra0, rb0);
        __syncthreads();
    }
    if (nk & 1)
        TR_COMPUTE(0);
#undef TR_LOAD_GLOBAL
#undef TR_STORE_LDS
#undef TR_COMPUTE
#undef TR_CLAMPK
    }

    typedef typename std::remove_reference<decltype(acc[0][0][0])>::type AccT;
    // Row-contiguous epilogue.  In the accumulator layout one store instruction touches 32 rows with 16 bytes
    // each, i.e. 32 partial cache lines; the L2 then sees eight times as many write requests as there are lines.
    // For each 32-row group every wave writes its 32 x CW accumulator block to its own LDS region (the slab
    // buffers are free after the main loop); the workgroup then walks the staged rows with eight columns per
    // thread, adds the WGK partial sums and applies the epilogue, so a store instruction covers whole lines of C
    // and bias/residual are read in the same coalesced shape.
    constexpr int CW   = TN * 32;       // columns per wave
    constexpr int SSTR = CFG::SSTR;     // staged row stride in 32-bit words (16-byte pad spreads the b128 banks)
    constexpr int CPR  = CW / 8;        // 8-column pieces per staged row
    constexpr int POS  = CFG::NW / WGK;  // wave positions (wm, wn) in the tile
    constexpr int ITEMS = POS * 32 * CPR;
    typedef AccT acc4 __attribute__((ext_vector_type(4)));
    AccT *const stage_all = reinterpret_cast<AccT *>(lds_dyn);
    AccT *const stage_me  = stage_all + wave * (32 * SSTR);  // wave = (wm*WGN + wn)*WGK + wk
    const bool by_rows = epi.direct(n0);
    const int tid_piece = tid % CPR, tid_rowpos = tid / CPR;
    __syncthreads();  // every wave is done reading the slabs
    TR_TL(2);         // main loop done
    // LayerNorm-folding epilogues: reduce the lanes' partial row sums over the two k-halves of a fragment and the WGK
    // k-waves (fixed order), giving {rstd, mean} per tile row; both arrays sit behind the staging area
    float2 *const row_st   = reinterpret_cast<float2 *>(lds_dyn + (TakesRowSums<Epi>::value ? CFG::lds_bytes : CFG::stage_bytes));  // [BM]
    float2 *const row_part = row_st + BM;                                             // [WGK * WGN * 2][BM]
    int8_t *const lut_lds = reinterpret_cast<int8_t *>(lds_dyn + CFG::stage_bytes);  // Int8Epilogue's table, 256 bytes
    if constexpr (std::is_same<Epi, Int8Epilogue>::value) {
        if (epi.lut && tid < 64)
            reinterpret_cast<uint32_t *>(lut_lds)[tid] = reinterpret_cast<const uint32_t *>(epi.lut)[tid];
        // read after the first staging barrier below
    }
    // the tile's columns of the epilogue's per-column arrays, and its rows' pairs: read after the first staging barrier
    float *const col_lds        = reinterpret_cast<float *>(lds_dyn + EpiLds<CFG, Epi>::col_offset);
    const float2 *const row_lds = reinterpret_cast<const float2 *>(lds_dyn + EpiLds<CFG, Epi>::row_offset);
    if constexpr (ColArrays<Epi>::value > 0) {
#pragma unroll
        for (int q = 0; q < (ColArrays<Epi>::value * BN + NT - 1) / NT; ++q) {
            const int e = q * NT + tid;
            if (e < ColArrays<Epi>::value * BN) {
                const int c = e % BN;
                col_lds[e]  = n0 + c < N ? epi.col_src(e / BN, n0 + c) : 0.f;
            }
        }
    }
    if constexpr (RowIn<Epi>::value) {
        if (tid < BM)
            reinterpret_cast<float2 *>(lds_dyn + EpiLds<CFG, Epi>::row_offset)[tid] =
                m0 + tid < M ? epi.row_src(m0 + tid) : make_float2(0.f, 0.f);
    }
    if constexpr (Epi::kRowStats && TakesRowSums<Epi>::value) {
        // {rstd, mean} were parked in LDS before the main loop (the barrier above orders that write); hand them on
        if (epi.ln.stats && n0 == 0 && tid < BM && m0 + tid < M)
            store_out8(&epi.ln.stats[m0 + tid], row_st[tid]);
    }
    if constexpr (Epi::kRowStats && !TakesRowSums<Epi>::value) {
        static_assert(CFG::NSTAGE > 0, "LayerNorm-folding epilogues run on the direct-to-LDS pipeline");
#pragma unroll
        for (int i = 0; i < TM; ++i)
            row_part[((wk * WGN + wn) * 2 + (lane >> 5)) * BM + (wm * TM + i) * 32 + frag_row] = make_float2(ln_s1[i], ln_s2[i]);
        __syncthreads();
        if (tid < BM) {
            double s1 = 0.0, s2 = 0.0;
            for (int q = 0; q < WGK * WGN * 2; ++q) {
                float2 v = row_part[q * BM + tid];
                s1 += (double)v.x;
                s2 += (double)v.y;
            }
            const double mean = s1 * (double)epi.ln.inv_cols;
            const double var  = s2 * (double)epi.ln.inv_cols - mean * mean;
            const float2 st   = make_float2((float)(1.0 / sqrt(var + (double)epi.ln.eps)), (float)mean);
            row_st[tid]       = st;
            if (epi.ln.stats && n0 == 0 && m0 + tid < M)  // every tile column holds them; the first one hands them on
                store_out8(&epi.ln.stats[m0 + tid], st);
        }
        // row_st is read after the first staging barrier below
    }
    // The LayerNorm output y is written at the very end from this tile's own share of its rows of A; the vectors it
    // needs are requested here, once the last accumulators have been staged, so their latency hides under the
    // remaining epilogue instead of standing alone at the kernel's tail.
    constexpr int YPRE = 3;  // vectors a thread holds ahead (192 x 192 tiles: 12 rows x K/8 groups over 512 threads)
    u32x4 y_pre[Epi::kRowStats ? YPRE : 1];
    int y_r0 = 0, y_items = 0, y_groups = 1;
    if constexpr (Epi::kRowStats) {
        if (epi.ln.y) {
            const int tn = n0 / BN;
            y_groups     = K / 8;
            y_r0         = (int)((long)tn * BM / tiles_n);
            y_items      = ((int)((long)(tn + 1) * BM / tiles_n) - y_r0) * y_groups;
        }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4)
                *reinterpret_cast<acc4 *>(stage_me + (lane & 31) * SSTR + j * 32 + 8 * r4 + 4 * (lane >> 5)) =
                    acc4{acc[i][j][r4 * 4 + 0], acc[i][j][r4 * 4 + 1], acc[i][j][r4 * 4 + 2], acc[i][j][r4 * 4 + 3]};
        if constexpr (Epi::kRowStats) {
            if (i == TM - 1) {
#pragma unroll
                for (int q = 0; q < YPRE; ++q) {
                    const int item = tid + q * NT;
                    if (epi.ln.y_ahead && item < y_items) {
                        const int m = m0 + y_r0 + item / y_groups;
                        if (m < M)
                            y_pre[q] = *reinterpret_cast<const u32x4 *>(A + (size_t)m * lda + (item % y_groups) * 8);
                    }
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < (ITEMS + NT - 1) / NT; ++it) {
            const int item = it * NT + tid;
            if (ITEMS % NT != 0 && item >= ITEMS)
                break;
            // consecutive threads walk along a row of C, or down the rows where the epilogue writes a transposed
            // layout (consecutive rows are then consecutive in memory)
            // item % CPR and item / CPR: where CPR is not a power of two (96-column wave tiles) the thread index is
            // split once and every item adds its constant share, instead of a multiply-high sequence per item
            int piece, rowpos;
            if constexpr ((CPR & (CPR - 1)) != 0) {
                const int c     = tid_piece + (it * NT) % CPR;
                const int carry = c >= CPR ? 1 : 0;
                piece           = c - carry * CPR;
                rowpos          = tid_rowpos + (it * NT) / CPR + carry;
            } else {
                piece  = item % CPR;
                rowpos = item / CPR;
            }
            const int c8  = by_rows ? ((item >> 5) % CPR) * 8 : piece * 8;
            const int row = by_rows ? (item & 31) : rowpos % 32;
            const int pos = rowpos / 32;  // = item / (CPR * 32) = pm * WGN + pn
            const AccT *src = stage_all + (pos * WGK) * (32 * SSTR) + row * SSTR + c8;
            acc4 lo = *reinterpret_cast<const acc4 *>(src);
            acc4 hi = *reinterpret_cast<const acc4 *>(src + 4);
#pragma unroll
            for (int q = 1; q < WGK; ++q) {
                lo += *reinterpret_cast<const acc4 *>(src + q * (32 * SSTR));
                hi += *reinterpret_cast<const acc4 *>(src + q * (32 * SSTR) + 4);
            }
            const int m = m0 + ((pos / WGN) * TM + i) * 32 + row;
            const int n = n0 + (pos % WGN) * CW + c8;
            const int nl = (pos % WGN) * CW + c8;  // column inside the tile
            if constexpr (Epi::kRowStats) {
                if (m < M && n + 7 < N) {  // N is a multiple of 8 for these epilogues (checked at launch)
                    AccT v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    epi.store8(m, n, v, row_st[m - m0], col_lds + nl, BN);
                }
            } else if constexpr (EmitsRowSums<Epi>::value) {
                // N is a multiple of 8 for these epilogues (checked at launch); every item leaves its eight columns'
                // sums, zero where nothing is stored, so that the totals below see a fully written array
                float2 sm = make_float2(0.f, 0.f);
                if (m < M && n + 7 < N) {
                    AccT v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    sm = epi.store8(m, n, v, col_lds + nl, BN, row_lds[m - m0]);
                }
                reinterpret_cast<float2 *>(lds_dyn + CFG::sums_offset)[(((pos / WGN) * TM + i) * 32 + row) * (BN / 8) +
                                                                     ((pos % WGN) * CW + c8) / 8] = sm;
            } else if (m < M) {
                AccT v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                if (n + 7 < N) {
                    if constexpr (std::is_same<Epi, Int8Epilogue>::value)
                        epi.store8(m, n, v, epi.lut ? lut_lds : nullptr, col_lds + nl, BN);
                    else if constexpr (RowIn<Epi>::value)
                        (void)epi.store8(m, n, v, col_lds + nl, BN, row_lds[m - m0]);
                    else if constexpr (ColArrays<Epi>::value > 0)
                        epi.store8(m, n, v, col_lds + nl, BN);
                    else
                        epi.store8(m, n, v);
                } else {
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        if (n + t < N)
                            epi.store(m, n + t, v[t], epi.col_const(n + t));
                }
            }
        }
        if (i + 1 < TM)
            __syncthreads();
    }
    TR_TL(3);  // C stored
    if constexpr (EmitsRowSums<Epi>::value) {
        // this tile's share of every row's sum and sum of squares, added up in a fixed order, for the folding GEMM
        // that reads C next
        __syncthreads();
        if (tid < BM && m0 + tid < M) {
            const float2 *part = reinterpret_cast<const float2 *>(lds_dyn + CFG::sums_offset) + tid * (BN / 8);
            float s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int q = 0; q < BN / 8; ++q)
                s1 += part[q].x, s2 += part[q].y;
            store_out8(&epi.row_sums[(size_t)(n0 / BN) * M + m0 + tid], make_float2(s1, s2));
        }
    }
    if constexpr (Epi::kRowStats) {
        // y = LayerNorm(t) for this tile's share of its rows (the BM rows are dealt out evenly over the tile columns, so
        // every workgroup writes whole rows), in the LayerNorm kernel's half-precision form
        // x * rstd * gamma + (beta - mean * rstd * gamma)
        if (epi.ln.y) {
            typedef typename GemmTraits<DT>::elem TY;
            const int groups = y_groups, r0 = y_r0;
            int q = 0;
            for (int item = tid; item < y_items; item += NT, ++q) {
                const int row = r0 + item / groups, c = (item % groups) * 8, m = m0 + row;
                if (m >= M)
                    continue;
                const float2 st = row_st[row];
                const float mrs = st.y * st.x;
                float4 k0 = *reinterpret_cast<const float4 *>(epi.ln.gamma + c), k1 = *reinterpret_cast<const float4 *>(epi.ln.gamma + c + 4);
                float4 e0 = *reinterpret_cast<const float4 *>(epi.ln.beta + c), e1 = *reinterpret_cast<const float4 *>(epi.ln.beta + c + 4);
                const float kk[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
                const float ee[8] = {e0.x, e0.y, e0.z, e0.w, e1.x, e1.y, e1.z, e1.w};
                u32x4 raw;
                if (epi.ln.y_ahead && q == 0)
                    raw = y_pre[0];
                else if (epi.ln.y_ahead && q == 1 && YPRE > 1)
                    raw = y_pre[YPRE > 1 ? 1 : 0];
                else if (epi.ln.y_ahead && q == 2 && YPRE > 2)
                    raw = y_pre[YPRE > 2 ? 2 : 0];
                else
                    raw = *reinterpret_cast<const u32x4 *>(A + (size_t)m * lda + c);
                TY *pe = reinterpret_cast<TY *>(&raw);
#pragma unroll
                for (int t = 0; t < 8; ++t)
                    Elem<DT>::st(&pe[t], Elem<DT>::ld(&pe[t]) * st.x * kk[t] + (ee[t] - mrs * kk[t]));
                *reinterpret_cast<u32x4 *>(reinterpret_cast<TY *>(epi.ln.y) + (size_t)m * K + c) = raw;
            }
        }
    }
    TR_TL(4);  // kernel end
}

// tuning override for experiments: 0 = heuristic, otherwise a configuration code of the tiled kernel
// the hooks may be set while other threads launch: atomics, and a lock around the tuning table
std::atomic<int> g_gemm_force_cfg{0};
std::atomic<int> g_gemm_group_m{0};  // 0 = derived from the tile count; otherwise forced

inline int tune_override(int N, int K, int *group_m);
// internal: the chosen tile shape leaves no LDS for the row-sum side output; the caller launches the plain form
constexpr int kTileTooLargeForSums = -12345;
thread_local int t_last_tiles_n = 0;  // tile columns of this thread's last tiled launch (the row-sum block count)

template <int DT, typename CFG, typename Epi>
int launch_tiled(hipStream_t s, const void *A, const void *B, int M, int N, int K, long lda, long ldb, const Epi &epi) {
    typedef typename GemmTraits<DT>::elem T;
    int tiles_m = (M + CFG::BM - 1) / CFG::BM, tiles_n = (N + CFG::BN - 1) / CFG::BN;
    typedef EpiLds<CFG, Epi> L;
    const size_t lds = L::total;
    if (EmitsRowSums<Epi>::value) {
        // the row sums are not taken at the price of a workgroup per CU (the plain form runs instead)
        const size_t without = L::plain + L::side_bytes + 16;
        const long cu = 160 * 1024;
        if (lds > (size_t)cu || cu / (long)(lds + 1024) < (cu / (long)(without + 1024) > 4 ? 4 : cu / (long)(without + 1024)))
            return kTileTooLargeForSums;
    }
    auto kern   = gemm_nk_tiled_kernel<DT, CFG, Epi>;
    if (lds > 64 * 1024) {
        // the attribute belongs to the (kernel, device) pair: one bit per device, per instantiation
        static std::atomic<unsigned long long> attr_set{0};
        int dev = 0;
        TR_CHECK_HIP(hipGetDevice(&dev));
        const unsigned long long bit = 1ull << (dev & 63);
        if (dev > 63 || !(attr_set.load(std::memory_order_acquire) & bit)) {
            TR_CHECK_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            attr_set.fetch_or(bit, std::memory_order_release);
        }
    }
    // tiles resident together on one XCD (32 CUs): a square-ish group keeps their panels in that L2
    const long lds_per_cu = 160 * 1024;
    long per_cu   = lds_per_cu / (long)(lds + 1024);
    per_cu        = per_cu < 1 ? 1 : (per_cu > 4 ? 4 : per_cu);
    long resident = 32 * per_cu, per_xcd = ((long)tiles_m * tiles_n + 7) / 8;
    resident      = resident < per_xcd ? resident : per_xcd;
    int forced_group = g_gemm_group_m;
    if (forced_group <= 0)
        tune_override(N, K, &forced_group);
    int group_m   = forced_group > 0 ? forced_group : 1;
    if (forced_group <= 0)
        while ((long)(group_m + 1) * (group_m + 1) <= resident)
            ++group_m;
    group_m = group_m > tiles_m ? tiles_m : group_m;
    unsigned grid = (unsigned)(((tiles_m * tiles_n + 7) / 8) * 8);
    t_last_tiles_n = tiles_n;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(CFG::NT), lds, s, (const T *)A, (const T *)B, M, N, K, lda, ldb, tiles_m, tiles_n,
                       group_m, epi);
    TR_CHECK_LAUNCH();
    return 0;
}

// Configuration codes: TM TN WGM WGN WGK S (one decimal digit each; slab bytes = 64 << S).
//   112210 / 112211   64 x  64, 4 waves                 222210  128 x 128, 4 waves
//   222221           128 x 128, 8 waves (two k-waves)   224211  256 x 128, 8 waves
//   332221           192 x 192, 8 waves (two k-waves)   331182   96 x  96, 8 k-waves, 256-byte slabs
//   111182            32 x  32, 8 k-waves, 256-byte slabs (fp32 only: small products)
// Eight-wave workgroups put two waves on every SIMD inside one tile: while one waits for its LDS fragments the
// other issues MFMAs, and a larger tile per CU moves fewer bytes through LDS and L2 per flop.  Four-wave tiles
// larger than 128 x 128 (one wave per SIMD) were measured and never won with compiler-scheduled code.
constexpr int kNumCU = 256;

// Shape heuristic, from measurements on MI355X (fp16; M in {1024, 3072, 4096, 16384}, N and K in
// {768, 1024, 2304, 3072, 4096}; times in us, best alternative in parentheses):
//   * default 128x128 with eight waves: M=4096 N=3072 K=1024 37 (4 waves 43), M=4096 N=1024 K=4096 45 (54),
//     M=16384 N=3072 K=768 122 (135), M=16384 N=768 K=3072 95 (106);
//   * small launches (at most ~0.6 tiles of 128x128 per CU): 64x64 tiles keep every CU busy
//     (M=3072 N=768 K=768 12.4 vs 12.9; M=1024 shapes 9.5-19 vs 13-35);
//   * a narrow N with a long K and about one 96x96 tile per CU: eight k-waves on one 96x96 tile
//     (M=3072 N=768 K=3072 25.6 vs 30.7);
//   * between one and two 128x128 tiles per CU: 256x128 when that is a single round (M=3072 N=2304 19.7 vs 20.6);
//   * slightly more than one round of 128x128 at two workgroups per CU, but a single round of 192x192
//     (M=3072 N=3072: 576 tiles for 512 slots): 192x192 (28.8 vs 31.9).
inline int pick_tile_config(long M, long N, size_t kbytes) {
    auto tiles = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    const long t128 = tiles(128, 128), slots = 2 * kNumCU;
    if (kbytes % 128 != 0)
        return t128 > kNumCU ? 222210 : 112210;
    if (kbytes >= 4096 && kbytes % 256 == 0) {
        const long t96 = tiles(96, 96);
        if (t96 <= kNumCU && t96 > kNumCU / 2 && t128 <= kNumCU)
            return 331182;
    }
    if (t128 * 10 <= kNumCU * 6)
        return 112211;
    if (t128 > kNumCU && t128 <= slots && tiles(256, 128) <= kNumCU)
        return 224211;
    if (t128 > slots && t128 < slots + slots / 4 && tiles(192, 192) <= kNumCU)
        return 332221;
    return 222221;
}

// Experiment hook: "N:K:code,N:K:code,..." forces a configuration code for given (N, K); set from the environment
// variable TNN_ROCM_GEMM_TUNE at first use, or through tnn_rocm_debug_set_gemm_tune().
struct TuneEntry { int n, k, cfg, group_m; };
TuneEntry g_tune_table[16];
int g_tune_count = -1;
std::mutex g_tune_lock;
inline void parse_tune(const char *e) {  // caller holds g_tune_lock
    g_tune_count = 0;
    while (e && *e && g_tune_count < 16) {
        TuneEntry t;
        t.group_m = 0;
        if (sscanf(e, "%d:%d:%d:%d", &t.n, &t.k, &t.cfg, &t.group_m) >= 3)
            g_tune_table[g_tune_count++] = t;
        e = strchr(e, ',');
        if (e)
            ++e;
    }
}
inline int tune_override(int N, int K, int *group_m) {
    static std::once_flag env_read;  // instances on several threads may launch their first GEMM together
    std::call_once(env_read, [] {
        std::lock_guard<std::mutex> hold(g_tune_lock);
        if (g_tune_count < 0)
            parse_tune(getenv("TNN_ROCM_GEMM_TUNE"));
    });
    std::lock_guard<std::mutex> hold(g_tune_lock);
    for (int i = 0; i < g_tune_count; ++i)
        if (g_tune_table[i].n == N && g_tune_table[i].k == K) {
            if (group_m)
                *group_m = g_tune_table[i].group_m;
            return g_tune_table[i].cfg;
        }
    return 0;
}

template <int DT, typename Epi>
int launch_gemm_fast(hipStream_t s, const void *A, const void *B, int M, int N, int K, long lda, long ldb,
                     const Epi &epi) {
    typedef typename GemmTraits<DT>::elem T;
    const int forced = g_gemm_force_cfg;
    int cfg       = forced > 0 ? forced : tune_override(N, K, nullptr);
    size_t kbytes = (size_t)K * sizeof(T);
    if (cfg == 0) {
        // slabs that are whole 128-byte multiples go global -> LDS directly; average kernel durations inside a
        // 12-layer forward at M=3072 on MI355X (fp16, us, register-staged in parentheses): 192x192 three stages
        // N=3072 K=768 26.7 (28.7); 96x96 k-split three stages N=768 K=3072 25.9 (28.0); 64x64 two stages
        // N=768 K=768 11.4 (12.3); 128x128 two stages N=2304 K=768 19.1 (256x128 register-staged 20.5)
        int code = pick_tile_config(M, N, kbytes);
        if (DT == TNN_ROCM_I8 && kbytes % 128 == 0) {
            // int8 tiles finish their K loop in half the slabs, so the fixed cost per tile weighs more and small tiles
            // that fill every CU win earlier than for fp16.  Inside the 12-layer int8 encoder at M=4096 (forward
            // 1.258 ms): 64x64 for N=768 (192 tiles of 128x128, K=768 and K=3072) and for N=2304 (576 tiles of
            // 128x128 for 512 slots, a second round for an eighth of the work) -> 1.216 ms.
            const long t128 = (((long)M + 127) / 128) * (((long)N + 127) / 128), slots = 2 * kNumCU;
            if (t128 < kNumCU || (code == 222221 && t128 > slots && t128 * 4 <= slots * 5))
                code = 112211;
        }
        switch (code) {
            case 112211: cfg = 2112211; break;
            case 222221: cfg = 2222221; break;
            case 224211: cfg = 2222221; break;  // two 128x128 workgroups per CU beat one 256x128 (19.1 vs 20.3)
            case 332221: cfg = 3332221; break;
            case 331182: cfg = 3331182; break;
            default: cfg = code; break;
        }
    }
    if (DT == TNN_ROCM_F32 && (cfg % 1000000 == 224211 || cfg % 1000000 == 332221 || cfg % 1000000 == 331182))
        cfg = 222221;
    if (DT == TNN_ROCM_F32)
        cfg %= 1000000;  // the fp32 instantiations are register-staged only
    if (DT == TNN_ROCM_F32 && forced <= 0 && cfg == 112211 && kbytes % 256 == 0 && kbytes >= 2048 &&
        (((long)M + 63) / 64) * (((long)N + 63) / 64) * 2 <= kNumCU) {
        // A small fp32 product (one attention layer at 128 tokens: 24 tiles of 64x64) leaves nine CUs in ten idle,
        // and the fp32 matrix pipe is 16 times slower than the fp16 one: 32x32 tiles with the K range dealt to
        // eight waves put four times as many CUs to work on each a quarter of the MFMAs.
        cfg = 111182;
    }
    if (kbytes % (64u << (cfg % 10)) != 0) {
        set_error("gemm: K=%d is not a whole number of slabs for tuning configuration %d", K, cfg);
        return TNN_ROCM_ESHAPE;
    }
#define TR_FAST(TMv, TNv, WGMv, WGNv, WGKv, SLABv)                                                                    \
    return launch_tiled<DT, TileCfg<TMv, TNv, WGMv, WGNv, WGKv, SLABv>, Epi>(s, A, B, M, N, K, lda, ldb, epi)
#define TR_FAST_DL(TMv, TNv, WGMv, WGNv, WGKv, SLABv, NSv)                                                            \
    return launch_tiled<DT, TileCfg<TMv, TNv, WGMv, WGNv, WGKv, SLABv, NSv>, Epi>(s, A, B, M, N, K, lda, ldb, epi)
    if constexpr (Epi::kRowStats) {
        // the LayerNorm-folding epilogues exist for the direct-to-LDS pipeline only (half types, 128-byte slabs)
        switch (cfg % 1000000) {
            case 112211: TR_FAST_DL(1, 1, 2, 2, 1, 128, 2);
            case 222221:
            case 224211: TR_FAST_DL(2, 2, 2, 2, 2, 128, 2);
            case 332221: TR_FAST_DL(3, 3, 2, 2, 2, 128, 3);
            case 331182: TR_FAST_DL(3, 3, 1, 1, 8, 256, 3);
            default: break;
        }
        set_error("gemm: tuning configuration %d has no LayerNorm-folding form", cfg);
        return TNN_ROCM_EINVAL;
    } else {
    switch (cfg) {
        case 112210: TR_FAST(1, 1, 2, 2, 1, 64);
        case 112211: TR_FAST(1, 1, 2, 2, 1, 128);
        case 222210: TR_FAST(2, 2, 2, 2, 1, 64);
        case 222221: TR_FAST(2, 2, 2, 2, 2, 128);
        default: break;
    }
    if constexpr (DT == TNN_ROCM_F32) {
        if (cfg == 111182)
            TR_FAST(1, 1, 1, 1, 8, 256);
    }
    if constexpr (DT != TNN_ROCM_F32) {
        switch (cfg) {
            case 2112211: TR_FAST_DL(1, 1, 2, 2, 1, 128, 2);
            case 2222221: TR_FAST_DL(2, 2, 2, 2, 2, 128, 2);
            case 3332221: TR_FAST_DL(3, 3, 2, 2, 2, 128, 3);
            case 3331182: TR_FAST_DL(3, 3, 1, 1, 8, 256, 3);
            default: break;
        }
        switch (cfg) {
            case 224211: TR_FAST(2, 2, 4, 2, 1, 128);
            case 332221: TR_FAST(3, 3, 2, 2, 2, 128);
            case 331182: TR_FAST(3, 3, 1, 1, 8, 256);
            default: break;
        }
    }
    }
#undef TR_FAST
#undef TR_FAST_DL
    set_error("gemm: unknown tuning configuration %d", cfg);
    return TNN_ROCM_EINVAL;
}

template <int DT, int BM, int BN, int WM, int WN, typename Epi>
int launch_gemm_cfg(hipStream_t s, bool b_nk, bool aligned, const void *A, const void *B, int M, int N, int K, long lda,
                    long ldb, int batch, int batch_a, int batch_b, long stride_a, long stride_b, const Epi &epi) {
    typedef typename GemmTraits<DT>::elem T;
    int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch), block(WM * WN * 64);
#define TR_GEMM_LAUNCH(NK, AL)                                                                                        \
    hipLaunchKernelGGL((gemm_kernel<DT, BM, BN, WM, WN, NK, AL, Epi>), grid, block, 0, s, (const T *)A, (const T *)B, \
                       M, N, K, lda, ldb, batch_a, batch_b, stride_a, stride_b, tiles_m, tiles_n, epi)
    if (b_nk) {
        if (aligned)
            TR_GEMM_LAUNCH(true, true);
        else
            TR_GEMM_LAUNCH(true, false);
    } else {
        if (aligned)
            TR_GEMM_LAUNCH(false, true);
        else
            TR_GEMM_LAUNCH(false, false);
    }
#undef TR_GEMM_LAUNCH
    TR_CHECK_LAUNCH();
    return 0;
}

// Tile choice: 128x128 when that still yields at least ~1.5 waves of workgroups over the 256 CUs,
// otherwise 128x64 / 64x64 so small-N projections keep the chip busy.
template <int DT, typename Epi>
int launch_gemm(hipStream_t s, bool b_nk, bool aligned, const void *A, const void *B, int M, int N, int K, long lda,
                long ldb, int batch, int batch_a, int batch_b, long stride_a, long stride_b, const Epi &epi) {
    auto tiles = [&](int bm, int bn) { return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn) * batch; };
    if (tiles(128, 128) >= 384)
        return launch_gemm_cfg<DT, 128, 128, 2, 2, Epi>(s, b_nk, aligned, A, B, M, N, K, lda, ldb, batch, batch_a,
                                                        batch_b, stride_a, stride_b, epi);
    if (tiles(128, 64) >= 256)
        return launch_gemm_cfg<DT, 128, 64, 2, 2, Epi>(s, b_nk, aligned, A, B, M, N, K, lda, ldb, batch, batch_a,
                                                       batch_b, stride_a, stride_b, epi);
    return launch_gemm_cfg<DT, 64, 64, 2, 2, Epi>(s, b_nk, aligned, A, B, M, N, K, lda, ldb, batch, batch_a, batch_b,
                                                  stride_a, stride_b, epi);
}

inline bool al16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }

}  // namespace

extern "C" {

int tnn_rocm_gemm(void *stream, int dtype, int b_is_nk, const void *A, const void *B, void *C, int M, int N, int K,
                  int lda, int ldb, int ldc, int batch, int batch_a, int batch_b, int epilogue, const float *bias,
                  const void *residual, int ldr) {
    TR_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 0, TNN_ROCM_ESHAPE, "gemm: negative size");
    if (M == 0 || N == 0 || batch == 0)
        return 0;
    TR_REQUIRE(A && B && C, TNN_ROCM_EINVAL, "gemm: null matrix pointer");
    TR_REQUIRE(K > 0, TNN_ROCM_ESHAPE, "gemm: K must be positive");
    TR_REQUIRE(batch_a >= 1 && batch_b >= 1 && batch_a <= batch && batch_b <= batch, TNN_ROCM_ESHAPE,
               "gemm: batch_a=%d batch_b=%d must lie in [1, batch=%d]", batch_a, batch_b, batch);
    TR_REQUIRE(lda >= K && ldc >= N && ldb >= (b_is_nk ? K : N), TNN_ROCM_ESHAPE,
               "gemm: leading dimension smaller than the row length");
    TR_REQUIRE((epilogue & ~7) == 0, TNN_ROCM_EINVAL, "gemm: unknown epilogue bits 0x%x", epilogue);
    TR_REQUIRE(!(epilogue & TNN_ROCM_EPI_BIAS) || bias, TNN_ROCM_EINVAL, "gemm: bias epilogue without bias");
    TR_REQUIRE(!(epilogue & TNN_ROCM_EPI_RESIDUAL) || (residual && ldr >= N), TNN_ROCM_EINVAL,
               "gemm: residual epilogue without residual / ldr");
    TR_REQUIRE(batch <= 65535, TNN_ROCM_ESHAPE, "gemm: batch %d exceeds 65535", batch);
    hipStream_t s = (hipStream_t)stream;
    long sa = (long)M * lda, sb = (long)(b_is_nk ? N : K) * ldb, sc = (long)M * ldc, sr = (long)M * ldr;

#define TR_GEMM_DT(DT)                                                                                                \
    {                                                                                                                 \
        typedef Elem<DT>::type T;                                                                                     \
        constexpr int VEC = 16 / sizeof(T);                                                                           \
        bool aligned = al16(A) && al16(B) && lda % VEC == 0 && ldb % VEC == 0 && K % VEC == 0 &&                      \
                       (b_is_nk || N % VEC == 0) && (batch == 1 || (sa % VEC == 0 && sb % VEC == 0));                 \
        FloatEpilogue<DT> epi;                                                                                        \
        epi.flags          = epilogue;                                                                                \
        epi.bias           = bias;                                                                                    \
        epi.residual       = (const T *)residual;                                                                     \
        epi.ldr            = ldr;                                                                                     \
        epi.C              = (T *)C;                                                                                  \
        epi.ldc            = ldc;                                                                                     \
        epi.batch_stride_c = sc;                                                                                      \
        epi.batch_stride_r = sr;                                                                                      \
        bool vec_out = N % 4 == 0 && ldc % VEC == 0 && (((uintptr_t)C) & 15u) == 0 &&                                 \
                       (!(epilogue & TNN_ROCM_EPI_RESIDUAL) || (ldr % VEC == 0 && (((uintptr_t)residual) & 15u) == 0)) &&\
                       (!(epilogue & TNN_ROCM_EPI_BIAS) || (((uintptr_t)bias) & 15u) == 0);                            \
        if (b_is_nk && aligned && batch == 1 && vec_out && g_gemm_force_cfg >= 0 && (K * sizeof(T)) % 64 == 0)        \
            return launch_gemm_fast<DT, FloatEpilogue<DT>>(s, A, B, M, N, K, lda, ldb, epi);                          \
        return launch_gemm<DT, FloatEpilogue<DT>>(s, b_is_nk != 0, aligned, A, B, M, N, K, lda, ldb, batch, batch_a,  \
                                                  batch_b, sa, sb, epi);                                              \
    }
    switch (dtype) {
        case TNN_ROCM_F32: TR_GEMM_DT(TNN_ROCM_F32)
        case TNN_ROCM_F16: TR_GEMM_DT(TNN_ROCM_F16)
        case TNN_ROCM_BF16: TR_GEMM_DT(TNN_ROCM_BF16)
        default: set_error("gemm: unsupported dtype %d", dtype); return TNN_ROCM_EDTYPE;
    }
#undef TR_GEMM_DT
}

static int gemm_i8_impl(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias, const float *scale,
                        int8_t *out_i8, int32_t *acc_i32, int M, int N, int K, int lda, int ldw, int ldo, void *out_f,
                        int out_f_dtype, float dequant_scale, const void *residual, const int8_t *lut = nullptr) {
    TR_REQUIRE(M >= 0 && N >= 0 && K >= 0, TNN_ROCM_ESHAPE, "gemm_i8: negative size");
    if (M == 0 || N == 0)
        return 0;
    TR_REQUIRE(A && W, TNN_ROCM_EINVAL, "gemm_i8: null matrix pointer");
    TR_REQUIRE(K > 0, TNN_ROCM_ESHAPE, "gemm_i8: K must be positive");
    TR_REQUIRE(out_i8 || acc_i32 || out_f, TNN_ROCM_EINVAL, "gemm_i8: no output requested");
    TR_REQUIRE(!(out_i8 || out_f) || scale, TNN_ROCM_EINVAL, "gemm_i8: requantised output needs scale[N]");
    TR_REQUIRE(lda >= K && ldw >= K && ldo >= N, TNN_ROCM_ESHAPE, "gemm_i8: leading dimension too small");
    TR_REQUIRE(!out_f || out_f_dtype == TNN_ROCM_F32 || out_f_dtype == TNN_ROCM_F16, TNN_ROCM_EDTYPE,
               "gemm_i8: dequantised output must be F32 or F16");
    TR_REQUIRE(!residual || out_f, TNN_ROCM_EINVAL, "gemm_i8: a residual needs the dequantised output");
    bool aligned = al16(A) && al16(W) && lda % 16 == 0 && ldw % 16 == 0 && K % 16 == 0;
    TR_REQUIRE(!lut || (out_i8 && !out_f && (((uintptr_t)lut) & 3u) == 0), TNN_ROCM_EINVAL,
               "gemm_i8: a lookup table applies to the int8 output only and must be 4-byte aligned");
    Int8Epilogue epi;
    epi.lut         = lut;
    epi.bias        = bias;
    epi.scale       = scale;
    epi.out         = out_i8;
    epi.acc_out     = acc_i32;
    epi.ldo         = ldo;
    epi.out_f       = out_f;
    epi.out_f_dtype = out_f_dtype;
    epi.dq          = dequant_scale;
    epi.residual    = residual;
    bool vec_out = ldo % 8 == 0 && (!bias || al16(bias)) && (!scale || al16(scale)) &&
                   (!out_i8 || (((uintptr_t)out_i8) & 7u) == 0) && (!acc_i32 || al16(acc_i32)) && (!out_f || al16(out_f)) &&
                   (!residual || al16(residual));
    if (aligned && vec_out && g_gemm_force_cfg >= 0 && K % 64 == 0)
        return launch_gemm_fast<TNN_ROCM_I8, Int8Epilogue>((hipStream_t)stream, A, W, M, N, K, lda, ldw, epi);
    return launch_gemm<TNN_ROCM_I8, Int8Epilogue>((hipStream_t)stream, true, aligned, A, W, M, N, K, lda, ldw, 1, 1, 1,
                                                  0, 0, epi);
}

int tnn_rocm_gemm_i8(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias, const float *scale,
                     int8_t *out_i8, int32_t *acc_i32, int M, int N, int K, int lda, int ldw, int ldo, void *out_f,
                     int out_f_dtype, float dequant_scale) {
    return gemm_i8_impl(stream, A, W, bias, scale, out_i8, acc_i32, M, N, K, lda, ldw, ldo, out_f, out_f_dtype,
                        dequant_scale, nullptr);
}

int tnn_rocm_gemm_i8_lut(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias, const float *scale,
                         int8_t *out_i8, int M, int N, int K, int lda, int ldw, int ldo, const int8_t *lut) {
    TR_REQUIRE(out_i8 && lut, TNN_ROCM_EINVAL, "gemm_i8_lut: null pointer");
    return gemm_i8_impl(stream, A, W, bias, scale, out_i8, nullptr, M, N, K, lda, ldw, ldo, nullptr, 0, 0.f, nullptr, lut);
}

int tnn_rocm_gemm_i8_dequant_residual(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias,
                                      const float *scale, int M, int N, int K, int lda, int ldw, void *out_f,
                                      int out_f_dtype, int ldo, float dequant_scale, const void *residual) {
    TR_REQUIRE(out_f, TNN_ROCM_EINVAL, "gemm_i8_dequant_residual: null output");
    return gemm_i8_impl(stream, A, W, bias, scale, nullptr, nullptr, M, N, K, lda, ldw, ldo, out_f, out_f_dtype,
                        dequant_scale, residual);
}

int tnn_rocm_gemm_i8_qkv_split(void *stream, int out_dtype, const int8_t *x, const int8_t *wqkv, const int32_t *bias,
                               const float *scale, const float *dequant, void *qk, void *vt, int B, int S, int heads,
                               int K, int vt_key_order) {
    TR_REQUIRE(vt_key_order == 0 || (vt_key_order == 1 && S % 16 == 0), TNN_ROCM_EINVAL,
               "gemm_i8_qkv_split: V^T key order %d (0 or 1; 1 needs S %% 16 == 0, S=%d)", vt_key_order, S);
    TR_REQUIRE(B >= 0 && S >= 0 && heads >= 0 && K >= 0, TNN_ROCM_ESHAPE, "gemm_i8_qkv_split: negative size");
    if (B == 0 || S == 0 || heads == 0)
        return 0;
    TR_REQUIRE(x && wqkv && scale && dequant && qk && vt, TNN_ROCM_EINVAL, "gemm_i8_qkv_split: null pointer");
    TR_REQUIRE(out_dtype == TNN_ROCM_F16 || out_dtype == TNN_ROCM_BF16, TNN_ROCM_EDTYPE,
               "gemm_i8_qkv_split: F16 or BF16 outputs only");
    TR_REQUIRE(K > 0 && K % 64 == 0, TNN_ROCM_ESHAPE, "gemm_i8_qkv_split: K=%d must be a positive multiple of 64", K);
    TR_REQUIRE((long)B * S < (1l << 24) && (long)B * S * 3 * heads * 64 < (1l << 31), TNN_ROCM_ESHAPE,
               "gemm_i8_qkv_split: problem too large for 32-bit panel offsets");
    TR_REQUIRE(al16(x) && al16(wqkv) && al16(qk) && al16(vt) && (!bias || al16(bias)) && al16(scale) && al16(dequant),
               TNN_ROCM_EALIGN, "gemm_i8_qkv_split: pointers must be 16-byte aligned");
    const int H = heads * 64, T = B * S;
#define TR_QKV8(DT)                                                                                                   \
    {                                                                                                                 \
        Int8QkvSplitEpilogue<DT> epi;                                                                                 \
        epi.bias    = bias;                                                                                           \
        epi.scale   = scale;                                                                                          \
        epi.dequant = dequant;                                                                                        \
        epi.qk      = (Elem<DT>::type *)qk;                                                                           \
        epi.vt      = (Elem<DT>::type *)vt;                                                                           \
        epi.H       = H;                                                                                              \
        epi.S       = S;                                                                                              \
        epi.heads   = heads;                                                                                          \
        epi.vt_sh   = vt_key_order;                                                                                   \
        return launch_gemm_fast<TNN_ROCM_I8, Int8QkvSplitEpilogue<DT>>((hipStream_t)stream, x, wqkv, T, 3 * H, K, K, K, \
                                                                       epi);                                          \
    }
    if (out_dtype == TNN_ROCM_F16)
        TR_QKV8(TNN_ROCM_F16)
    else
        TR_QKV8(TNN_ROCM_BF16)
#undef TR_QKV8
}

int tnn_rocm_gemm_qkv_split(void *stream, int dtype, const void *x, const void *wqkv, const float *bqkv, void *qk,
                            void *vt, int B, int S, int heads, int K, int vt_key_order) {
    TR_REQUIRE(vt_key_order == 0 || (vt_key_order == 1 && S % 16 == 0), TNN_ROCM_EINVAL,
               "gemm_qkv_split: V^T key order %d (0 or 1; 1 needs S %% 16 == 0, S=%d)", vt_key_order, S);
    TR_REQUIRE(B >= 0 && S >= 0 && heads >= 0 && K >= 0, TNN_ROCM_ESHAPE, "gemm_qkv_split: negative size");
    if (B == 0 || S == 0 || heads == 0)
        return 0;
    TR_REQUIRE(x && wqkv && qk && vt, TNN_ROCM_EINVAL, "gemm_qkv_split: null pointer");
    TR_REQUIRE(dtype == TNN_ROCM_F16 || dtype == TNN_ROCM_BF16, TNN_ROCM_EDTYPE, "gemm_qkv_split: F16 or BF16 only");
    TR_REQUIRE(K > 0 && K % 64 == 0, TNN_ROCM_ESHAPE, "gemm_qkv_split: K=%d must be a positive multiple of 64", K);
    TR_REQUIRE((long)B * S < (1l << 24) && (long)B * S * 3 * heads * 64 < (1l << 31), TNN_ROCM_ESHAPE,
               "gemm_qkv_split: problem too large for 32-bit panel offsets");
    TR_REQUIRE(al16(x) && al16(wqkv) && al16(qk) && al16(vt) && (!bqkv || al16(bqkv)), TNN_ROCM_EALIGN,
               "gemm_qkv_split: pointers must be 16-byte aligned");
    const int H = heads * 64, T = B * S;
#define TR_QKV(DT)                                                                                                    \
    {                                                                                                                 \
        QkvSplitEpilogue<DT> epi;                                                                                     \
        epi.bias  = bqkv;                                                                                             \
        epi.qk    = (Elem<DT>::type *)qk;                                                                             \
        epi.vt    = (Elem<DT>::type *)vt;                                                                             \
        epi.H     = H;                                                                                                \
        epi.S     = S;                                                                                                \
        epi.heads = heads;                                                                                            \
        epi.vt_sh = vt_key_order;                                                                                     \
        return launch_gemm_fast<DT, QkvSplitEpilogue<DT>>((hipStream_t)stream, x, wqkv, T, 3 * H, K, K, K, epi);      \
    }
    if (dtype == TNN_ROCM_F16)
        TR_QKV(TNN_ROCM_F16)
    else
        TR_QKV(TNN_ROCM_BF16)
#undef TR_QKV
}

int tnn_rocm_gemm_ln(void *stream, int dtype, const void *t, const void *w_folded, const float *bias_folded,
                     const float *colsum, const float *gamma, const float *beta, float eps, void *C, void *y,
                     float *row_stats, const float *row_sums, int row_sum_blocks, int M, int N, int K, int flags,
                     const void *residual) {
    TR_REQUIRE(M >= 0 && N >= 0 && K >= 0, TNN_ROCM_ESHAPE, "gemm_ln: negative size");
    if (M == 0 || N == 0)
        return 0;
    TR_REQUIRE(t && w_folded && bias_folded && colsum && C, TNN_ROCM_EINVAL, "gemm_ln: null pointer");
    TR_REQUIRE(!y || (gamma && beta), TNN_ROCM_EINVAL, "gemm_ln: the LayerNorm output needs gamma and beta");
    TR_REQUIRE(dtype == TNN_ROCM_F16 || dtype == TNN_ROCM_BF16, TNN_ROCM_EDTYPE, "gemm_ln: F16 or BF16 only");
    TR_REQUIRE(K > 0 && K % 128 == 0 && N % 8 == 0, TNN_ROCM_ESHAPE,
               "gemm_ln: K=%d must be a positive multiple of 128 and N=%d a multiple of 8", K, N);
    TR_REQUIRE((long)M < (1l << 24) && (long)N < (1l << 24) && (long)M * K < (1l << 31) && (long)N * K < (1l << 31) &&
                   (long)M * N < (1l << 31),
               TNN_ROCM_ESHAPE, "gemm_ln: problem too large for 32-bit panel offsets");
    TR_REQUIRE(!(flags & TNN_ROCM_EPI_RESIDUAL) || residual, TNN_ROCM_EINVAL, "gemm_ln: residual flag without a residual");
    TR_REQUIRE(!row_sums || (row_sum_blocks >= 1 && row_sum_blocks <= kMaxRowSumBlocks && (((uintptr_t)row_sums) & 7u) == 0),
               TNN_ROCM_EINVAL, "gemm_ln: row sums come in 1..%d blocks, 8-byte aligned", kMaxRowSumBlocks);
    TR_REQUIRE(al16(t) && al16(w_folded) && al16(C) && al16(bias_folded) && al16(colsum) && (!residual || al16(residual)) &&
                   (!y || (al16(y) && al16(gamma) && al16(beta))) && (((uintptr_t)row_stats) & 7u) == 0,
               TNN_ROCM_EALIGN, "gemm_ln: pointers must be 16-byte aligned (row_stats: 8-byte)");
#define TR_LN(DT, SUMS)                                                                                               \
    {                                                                                                                 \
        LnFloatEpilogue<DT, SUMS> epi;                                                                                      \
        epi.flags    = flags;                                                                                         \
        epi.bias     = bias_folded;                                                                                   \
        epi.residual = (const Elem<DT>::type *)residual;                                                              \
        epi.C        = (Elem<DT>::type *)C;                                                                           \
        epi.ldc      = N;                                                                                             \
        epi.ln = LnFold{1.0f / (float)K, eps, colsum, gamma, beta, y, g_ln_y_ahead.load(), (float2 *)row_stats,       \
                        (const float2 *)row_sums, row_sum_blocks};                                                   \
        return launch_gemm_fast<DT, LnFloatEpilogue<DT, SUMS>>((hipStream_t)stream, t, w_folded, M, N, K, K, K, epi); \
    }
    if (dtype == TNN_ROCM_F16) {
        if (row_sums && row_sum_blocks <= 12)
            TR_LN(TNN_ROCM_F16, 12)
        else if (row_sums)
            TR_LN(TNN_ROCM_F16, kMaxRowSumBlocks)
        else
            TR_LN(TNN_ROCM_F16, 0)
    } else {
        if (row_sums && row_sum_blocks <= 12)
            TR_LN(TNN_ROCM_BF16, 12)
        else if (row_sums)
            TR_LN(TNN_ROCM_BF16, kMaxRowSumBlocks)
        else
            TR_LN(TNN_ROCM_BF16, 0)
    }
#undef TR_LN
}

int tnn_rocm_gemm_qkv_split_ln(void *stream, int dtype, const void *t, const void *wqkv_folded, const float *bqkv_folded,
                               const float *colsum, const float *gamma, const float *beta, float eps, void *qk, void *vt,
                               void *y, float *row_stats, const float *row_sums, int row_sum_blocks, int B, int S, int heads,
                               int K, int vt_key_order) {
    TR_REQUIRE(vt_key_order == 0 || (vt_key_order == 1 && S % 16 == 0), TNN_ROCM_EINVAL,
               "gemm_qkv_split_ln: V^T key order %d (0 or 1; 1 needs S %% 16 == 0, S=%d)", vt_key_order, S);
    TR_REQUIRE(B >= 0 && S >= 0 && heads >= 0 && K >= 0, TNN_ROCM_ESHAPE, "gemm_qkv_split_ln: negative size");
    if (B == 0 || S == 0 || heads == 0)
        return 0;
    TR_REQUIRE(t && wqkv_folded && bqkv_folded && colsum && qk && vt, TNN_ROCM_EINVAL, "gemm_qkv_split_ln: null pointer");
    TR_REQUIRE(!y || (gamma && beta), TNN_ROCM_EINVAL, "gemm_qkv_split_ln: the LayerNorm output needs gamma and beta");
    TR_REQUIRE(dtype == TNN_ROCM_F16 || dtype == TNN_ROCM_BF16, TNN_ROCM_EDTYPE, "gemm_qkv_split_ln: F16 or BF16 only");
    TR_REQUIRE(K > 0 && K % 128 == 0 && S % 8 == 0, TNN_ROCM_ESHAPE,
               "gemm_qkv_split_ln: K=%d must be a positive multiple of 128 and S=%d a multiple of 8", K, S);
    TR_REQUIRE((long)B * S < (1l << 24) && (long)heads * 192 < (1l << 24) && (long)B * S * 3 * heads * 64 < (1l << 31),
               TNN_ROCM_ESHAPE, "gemm_qkv_split_ln: problem too large for 32-bit panel offsets");
    TR_REQUIRE(al16(t) && al16(wqkv_folded) && al16(qk) && al16(vt) && al16(bqkv_folded) && al16(colsum) &&
                   (!y || (al16(y) && al16(gamma) && al16(beta))) && (((uintptr_t)row_stats) & 7u) == 0,
               TNN_ROCM_EALIGN, "gemm_qkv_split_ln: pointers must be 16-byte aligned (row_stats: 8-byte)");
    TR_REQUIRE(!row_sums || (row_sum_blocks >= 1 && row_sum_blocks <= kMaxRowSumBlocks && (((uintptr_t)row_sums) & 7u) == 0),
               TNN_ROCM_EINVAL, "gemm_qkv_split_ln: row sums come in 1..%d blocks, 8-byte aligned", kMaxRowSumBlocks);
    const int H = heads * 64, T = B * S;
#define TR_QKVLN(DT, SUMS)                                                                                            \
    {                                                                                                                 \
        LnQkvSplitEpilogue<DT, SUMS> epi;                                                                                   \
        epi.bias  = bqkv_folded;                                                                                      \
        epi.qk    = (Elem<DT>::type *)qk;                                                                             \
        epi.vt    = (Elem<DT>::type *)vt;                                                                             \
        epi.H     = H;                                                                                                \
        epi.S     = S;                                                                                                \
        epi.heads = heads;                                                                                            \
        epi.vt_sh = vt_key_order;                                                                                     \
        epi.ln = LnFold{1.0f / (float)K, eps, colsum, gamma, beta, y, g_ln_y_ahead.load(), (float2 *)row_stats,       \
                        (const float2 *)row_sums, row_sum_blocks};                                                   \
        return launch_gemm_fast<DT, LnQkvSplitEpilogue<DT, SUMS>>((hipStream_t)stream, t, wqkv_folded, T, 3 * H, K, K, K, \
                                                                  epi);                                              \
    }
    if (dtype == TNN_ROCM_F16) {
        if (row_sums && row_sum_blocks <= 12)
            TR_QKVLN(TNN_ROCM_F16, 12)
        else if (row_sums)
            TR_QKVLN(TNN_ROCM_F16, kMaxRowSumBlocks)
        else
            TR_QKVLN(TNN_ROCM_F16, 0)
    } else {
        if (row_sums && row_sum_blocks <= 12)
            TR_QKVLN(TNN_ROCM_BF16, 12)
        else if (row_sums)
            TR_QKVLN(TNN_ROCM_BF16, kMaxRowSumBlocks)
        else
            TR_QKVLN(TNN_ROCM_BF16, 0)
    }
#undef TR_QKVLN
}

int tnn_rocm_gemm_residual_ln(void *stream, int dtype, const void *x, const void *w, const float *bias, void *C,
                              const void *t, const float *row_stats, const float *gamma, const float *beta, int M, int N,
                              int K, int flags, float *row_sums, int *row_sum_blocks) {
    TR_REQUIRE(M >= 0 && N >= 0 && K >= 0, TNN_ROCM_ESHAPE, "gemm_residual_ln: negative size");
    if (M == 0 || N == 0)
        return 0;
    TR_REQUIRE(x && w && C && t && row_stats && gamma && beta, TNN_ROCM_EINVAL, "gemm_residual_ln: null pointer");
    TR_REQUIRE(!(flags & TNN_ROCM_EPI_BIAS) || bias, TNN_ROCM_EINVAL, "gemm_residual_ln: bias flag without a bias");
    TR_REQUIRE(!(flags & ~(TNN_ROCM_EPI_BIAS | TNN_ROCM_EPI_GELU)), TNN_ROCM_EINVAL,
               "gemm_residual_ln: flags may name bias and GELU only (the residual is the rebuilt LayerNorm)");
    TR_REQUIRE(dtype == TNN_ROCM_F16 || dtype == TNN_ROCM_BF16, TNN_ROCM_EDTYPE, "gemm_residual_ln: F16 or BF16 only");
    TR_REQUIRE(K > 0 && K % 64 == 0 && N % 8 == 0, TNN_ROCM_ESHAPE,
               "gemm_residual_ln: K=%d must be a positive multiple of 64 and N=%d a multiple of 8", K, N);
    TR_REQUIRE((long)M < (1l << 24) && (long)N < (1l << 24) && (long)M * K < (1l << 31) && (long)N * K < (1l << 31) &&
                   (long)M * N < (1l << 31),
               TNN_ROCM_ESHAPE, "gemm_residual_ln: problem too large for 32-bit panel offsets");
    TR_REQUIRE(al16(x) && al16(w) && al16(C) && al16(t) && al16(gamma) && al16(beta) && (!bias || al16(bias)) &&
                   (((uintptr_t)row_stats) & 7u) == 0,
               TNN_ROCM_EALIGN, "gemm_residual_ln: pointers must be 16-byte aligned (row_stats: 8-byte)");
    TR_REQUIRE(!row_sums || (row_sum_blocks && (((uintptr_t)row_sums) & 7u) == 0), TNN_ROCM_EINVAL,
               "gemm_residual_ln: the row sums need an 8-byte aligned buffer and a place for their block count");
    if (row_sum_blocks)
        *row_sum_blocks = 0;
#define TR_LNRES(DT, SUMS)                                                                                            \
    {                                                                                                                 \
        LnResidualEpilogue<DT, SUMS> epi;                                                                             \
        epi.row_sums = (float2 *)row_sums;                                                                            \
        epi.flags = flags;                                                                                            \
        epi.bias  = bias;                                                                                             \
        epi.t     = (const Elem<DT>::type *)t;                                                                        \
        epi.st    = (const float2 *)row_stats;                                                                        \
        epi.gamma = gamma;                                                                                            \
        epi.beta  = beta;                                                                                             \
        epi.C     = (Elem<DT>::type *)C;                                                                              \
        epi.ldc   = N;                                                                                                \
        rc = launch_gemm_fast<DT, LnResidualEpilogue<DT, SUMS>>((hipStream_t)stream, x, w, M, N, K, K, K, epi);       \
    }
    // With the row sums first.  Half-precision tiles are at least 64 columns wide, so N <= 64 * kMaxRowSumBlocks keeps
    // the tile columns within what a reader adds up (and within the caller's buffer of kMaxRowSumBlocks * M pairs); a
    // tile shape that leaves no LDS for the sums runs the plain form and reports zero blocks.
    int rc = kTileTooLargeForSums;
    if (row_sums && N <= 64 * kMaxRowSumBlocks) {
        if (dtype == TNN_ROCM_F16)
            TR_LNRES(TNN_ROCM_F16, true)
        else
            TR_LNRES(TNN_ROCM_BF16, true)
        if (rc == 0)
            *row_sum_blocks = t_last_tiles_n;
        if (rc != kTileTooLargeForSums)
            return rc;
    }
    if (dtype == TNN_ROCM_F16)
        TR_LNRES(TNN_ROCM_F16, false)
    else
        TR_LNRES(TNN_ROCM_BF16, false)
    return rc;
#undef TR_LNRES
}

// Experiment hook (not part of the documented ABI): 0 restores the shape heuristic, -1 forces the baseline
// kernel, other values select a configuration code of the tiled kernel.
__attribute__((visibility("default"))) int tnn_rocm_debug_set_gemm_config(int cfg) {
    g_gemm_force_cfg = cfg;
    return 0;
}
__attribute__((visibility("default"))) int tnn_rocm_debug_set_gemm_tune(const char *spec) {
    std::lock_guard<std::mutex> hold(g_tune_lock);
    parse_tune(spec);
    return 0;
}
TR_DEFINE_STORE_THROUGH_SETTER(gemm_set_store_through)
__attribute__((visibility("default"))) int tnn_rocm_debug_set_ln_y_ahead(int on) {
    g_ln_y_ahead = on ? 1 : 0;
    return 0;
}
__attribute__((visibility("default"))) int tnn_rocm_debug_set_gemm_group_m(int group_m) {
    g_gemm_group_m = group_m;
    return 0;
}

}  // extern "C"
