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
#include "common.h"

using namespace tnn_rocm;

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

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
template <int DT> struct FloatEpilogue {
    typedef typename Elem<DT>::type T;
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
};

struct Int8Epilogue {
    const int32_t *bias;
    const float *scale;
    int8_t *out;
    int32_t *acc_out;
    long ldo;
    void *out_f;
    int out_f_dtype;
    float dq;
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
            if (out)
                out[(size_t)m * ldo + n] = q;
            if (out_f) {
                float d = __fmul_rn((float)q, dq);
                if (out_f_dtype == TNN_ROCM_F32)
                    ((float *)out_f)[(size_t)m * ldo + n] = d;
                else
                    ((half_t *)out_f)[(size_t)m * ldo + n] = (half_t)d;
            }
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

int tnn_rocm_gemm_i8(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias, const float *scale,
                     int8_t *out_i8, int32_t *acc_i32, int M, int N, int K, int lda, int ldw, int ldo, void *out_f,
                     int out_f_dtype, float dequant_scale) {
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
    bool aligned = al16(A) && al16(W) && lda % 16 == 0 && ldw % 16 == 0 && K % 16 == 0;
    Int8Epilogue epi;
    epi.bias        = bias;
    epi.scale       = scale;
    epi.out         = out_i8;
    epi.acc_out     = acc_i32;
    epi.ldo         = ldo;
    epi.out_f       = out_f;
    epi.out_f_dtype = out_f_dtype;
    epi.dq          = dequant_scale;
    return launch_gemm<TNN_ROCM_I8, Int8Epilogue>((hipStream_t)stream, true, aligned, A, W, M, N, K, lda, ldw, 1, 1, 1,
                                                  0, 0, epi);
}

}  // extern "C"
