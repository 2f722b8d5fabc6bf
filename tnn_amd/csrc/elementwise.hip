// HBM-bound element-wise kernels: GELU, broadcast binary ops, permute, gather, casts and the
// int8 boundary ops (quantize / dequantize / int8 add / int8 GELU).
//
// All kernels move 16 bytes per lane per access where the pointers allow it, with a grid-stride
// loop over enough workgroups to cover the 256 CUs several times.
#include "common.h"

using namespace tnn_rocm;

namespace {
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBlock     = 256;
constexpr int kMaxBlocks = 256 * 16;

inline int grid_for(size_t work_items) {
    size_t b = (work_items + kBlock - 1) / kBlock;
    if (b < 1)
        b = 1;
    if (b > (size_t)kMaxBlocks)
        b = kMaxBlocks;
    return (int)b;
}

inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }

// ---- generic unary map over a float dtype, VEC elements (16 bytes) per lane -------------------
template <int DT, typename F>
__global__ void __launch_bounds__(kBlock) unary_vec_kernel(const typename Elem<DT>::type *__restrict__ x,
                                                           typename Elem<DT>::type *__restrict__ y, size_t n, F f) {
    typedef typename Elem<DT>::type T;
    constexpr int VEC = 16 / sizeof(T);
    size_t nvec       = n / VEC;
    size_t stride     = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        uint4 raw = reinterpret_cast<const uint4 *>(x)[i];
        T *e      = reinterpret_cast<T *>(&raw);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            Elem<DT>::st(&e[j], f(Elem<DT>::ld(&e[j])));
        reinterpret_cast<uint4 *>(y)[i] = raw;
    }
    // tail
    size_t t = nvec * VEC + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n)
        Elem<DT>::st(&y[t], f(Elem<DT>::ld(&x[t])));
}

template <int DT, typename F>
__global__ void __launch_bounds__(kBlock) unary_scalar_kernel(const typename Elem<DT>::type *__restrict__ x,
                                                              typename Elem<DT>::type *__restrict__ y, size_t n, F f) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        Elem<DT>::st(&y[i], f(Elem<DT>::ld(&x[i])));
}

struct GeluOp {
    __device__ __forceinline__ float operator()(float v) const { return gelu_erf(v); }
};
// fp16 / bf16 blobs: the result is rounded to 11 / 8 bits, so the short rational form (at most one ulp of the
// rounded result away, the same one the GEMM epilogue uses) keeps the launch on the memory side of the roofline:
// with the ~40 instructions of erff it is bound by the vector ALU at about half the HBM rate.
struct GeluHalfOp {
    __device__ __forceinline__ float operator()(float v) const { return gelu_erf_fast(v); }
};
struct TanhOp {  // cpu_tanh_layer_acc.cc:23-27
    __device__ __forceinline__ float operator()(float v) const { return tanhf(v); }
};

template <int DT, typename F>
int launch_unary(hipStream_t s, const void *x, void *y, size_t n, F f) {
    typedef typename Elem<DT>::type T;
    constexpr int VEC = 16 / sizeof(T);
    if (aligned16(x) && aligned16(y)) {
        // the tail is handled by the first (n % VEC) lanes of the grid, so the grid must hold them
        hipLaunchKernelGGL((unary_vec_kernel<DT, F>), dim3(grid_for(n / VEC + VEC)), dim3(kBlock), 0, s, (const T *)x,
                           (T *)y, n, f);
    } else {
        hipLaunchKernelGGL((unary_scalar_kernel<DT, F>), dim3(grid_for(n)), dim3(kBlock), 0, s, (const T *)x, (T *)y,
                           n, f);
    }
    TR_CHECK_LAUNCH();
    return 0;
}

// ---- broadcast binary -----------------------------------------------------------------------
struct BcastDesc {
    int rank;
    int out_dim[6];
    long a_stride[6];  // 0 where the operand broadcasts along the axis
    long b_stride[6];
};

template <int DT, int OP>
__global__ void __launch_bounds__(kBlock) binary_bcast_kernel(const typename Elem<DT>::type *__restrict__ a,
                                                              const typename Elem<DT>::type *__restrict__ b,
                                                              typename Elem<DT>::type *__restrict__ out, size_t n,
                                                              BcastDesc d) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        size_t rem = i;
        long oa = 0, ob = 0;
#pragma unroll
        for (int ax = 5; ax >= 0; --ax) {
            if (ax < d.rank) {
                int idx = (int)(rem % (size_t)d.out_dim[ax]);
                rem /= (size_t)d.out_dim[ax];
                oa += idx * d.a_stride[ax];
                ob += idx * d.b_stride[ax];
            }
        }
        float va = Elem<DT>::ld(&a[oa]);
        float vb = Elem<DT>::ld(&b[ob]);
        float r;
        if (OP == 0)
            r = __fadd_rn(va, vb);
        else if (OP == 1)
            r = __fsub_rn(va, vb);
        else if (OP == 2)
            r = __fmul_rn(va, vb);
        else
            r = __fdiv_rn(va, vb);
        Elem<DT>::st(&out[i], r);
    }
}

// Fast path: b is a vector over the last axis (bias add, gamma scale) or a scalar, a and out
// have the same shape.  16 bytes per lane.
template <int DT, int OP>
__global__ void __launch_bounds__(kBlock) binary_lastaxis_kernel(const typename Elem<DT>::type *__restrict__ a,
                                                                 const typename Elem<DT>::type *__restrict__ b,
                                                                 typename Elem<DT>::type *__restrict__ out,
                                                                 size_t nvec, int cols_vec, int b_is_scalar,
                                                                 int b_is_full) {
    typedef typename Elem<DT>::type T;
    constexpr int VEC = 16 / sizeof(T);
    size_t stride     = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        uint4 ra = reinterpret_cast<const uint4 *>(a)[i];
        T *ea    = reinterpret_cast<T *>(&ra);
        uint4 rb;
        T *eb = reinterpret_cast<T *>(&rb);
        if (b_is_full) {
            rb = reinterpret_cast<const uint4 *>(b)[i];
        } else if (!b_is_scalar) {
            rb = reinterpret_cast<const uint4 *>(b)[i % (size_t)cols_vec];
        }
        float sb = b_is_scalar ? Elem<DT>::ld(&b[0]) : 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            float va = Elem<DT>::ld(&ea[j]);
            float vb = b_is_scalar ? sb : Elem<DT>::ld(&eb[j]);
            float r;
            if (OP == 0)
                r = __fadd_rn(va, vb);
            else if (OP == 1)
                r = __fsub_rn(va, vb);
            else if (OP == 2)
                r = __fmul_rn(va, vb);
            else
                r = __fdiv_rn(va, vb);
            Elem<DT>::st(&ea[j], r);
        }
        reinterpret_cast<uint4 *>(out)[i] = ra;
    }
}

template <int DT>
int launch_binary(hipStream_t s, int op, const void *a, const void *b, void *out, size_t n, const BcastDesc &d,
                  int fast_kind, int cols) {
    typedef typename Elem<DT>::type T;
    constexpr int VEC = 16 / sizeof(T);
    bool fast = fast_kind != 0 && aligned16(a) && aligned16(out) && (n % VEC) == 0 &&
                (fast_kind == 2 || (aligned16(b) && (fast_kind == 3 || cols % VEC == 0)));
#define TR_BIN_CASE(OPV)                                                                                              \
    case OPV:                                                                                                         \
        if (fast)                                                                                                     \
            hipLaunchKernelGGL((binary_lastaxis_kernel<DT, OPV>), dim3(grid_for(n / VEC)), dim3(kBlock), 0, s,        \
                               (const T *)a, (const T *)b, (T *)out, n / VEC, cols / VEC > 0 ? cols / VEC : 1,        \
                               fast_kind == 2 ? 1 : 0, fast_kind == 3 ? 1 : 0);                                       \
        else                                                                                                          \
            hipLaunchKernelGGL((binary_bcast_kernel<DT, OPV>), dim3(grid_for(n)), dim3(kBlock), 0, s, (const T *)a,   \
                               (const T *)b, (T *)out, n, d);                                                         \
        break;
    switch (op) {
        TR_BIN_CASE(0)
        TR_BIN_CASE(1)
        TR_BIN_CASE(2)
        TR_BIN_CASE(3)
        default:
            set_error("binary: unknown op %d", op);
            return TNN_ROCM_EINVAL;
    }
#undef TR_BIN_CASE
    TR_CHECK_LAUNCH();
    return 0;
}

// ---- permute -----------------------------------------------------------------------------------
struct PermDesc {
    int rank;
    int out_dim[6];
    long in_stride_of_out_axis[6];
};

template <typename T>
__global__ void __launch_bounds__(kBlock) permute_kernel(const T *__restrict__ in, T *__restrict__ out, size_t n,
                                                         PermDesc d) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        size_t rem = i;
        long src   = 0;
#pragma unroll
        for (int ax = 5; ax >= 0; --ax) {
            if (ax < d.rank) {
                int idx = (int)(rem % (size_t)d.out_dim[ax]);
                rem /= (size_t)d.out_dim[ax];
                src += idx * d.in_stride_of_out_axis[ax];
            }
        }
        out[i] = in[src];
    }
}

// Transposing permutes (the output's fastest axis is not the input's): 64 x 64 element tiles over the pair
// (input-fastest axis F, the input axis A that becomes output-fastest) go through LDS, so both the reads (lanes along
// F) and the writes (lanes along A) touch whole cache lines.  Every other axis is a batch axis; a workgroup finds its
// tile and batch offsets from its index.
struct TransDesc {
    int n_batch_axes;
    int batch_dim[4];
    long batch_in_stride[4], batch_out_stride[4];
    int len_f, len_a;          // extents of the two tiled axes
    long in_stride_a;          // input stride of axis A (axis F has input stride 1)
    long out_stride_f;         // output stride of axis F (axis A has output stride 1)
    int tiles_f, tiles_a;
};

template <typename T>
__global__ void __launch_bounds__(kBlock) permute_transpose_kernel(const T *__restrict__ in, T *__restrict__ out,
                                                                   TransDesc d) {
    constexpr int TILE = 64;
    __shared__ T tile[TILE][TILE + (sizeof(T) >= 4 ? 1 : (sizeof(T) == 2 ? 2 : 4))];
    size_t blk  = blockIdx.x;
    const int tf = (int)(blk % (size_t)d.tiles_f);
    blk /= (size_t)d.tiles_f;
    const int ta = (int)(blk % (size_t)d.tiles_a);
    blk /= (size_t)d.tiles_a;
    long in_off = 0, out_off = 0;
#pragma unroll
    for (int k = 3; k >= 0; --k) {
        if (k < d.n_batch_axes) {
            const int idx = (int)(blk % (size_t)d.batch_dim[k]);
            blk /= (size_t)d.batch_dim[k];
            in_off += idx * d.batch_in_stride[k];
            out_off += idx * d.batch_out_stride[k];
        }
    }
    const int f0 = tf * TILE, a0 = ta * TILE;
    const int col = threadIdx.x & (TILE - 1), row0 = threadIdx.x / TILE;  // 4 rows of 64 lanes per pass
    const T *src = in + in_off;
    T *dst       = out + out_off;
#pragma unroll 4
    for (int r = row0; r < TILE; r += kBlock / TILE) {
        const int a = a0 + r, f = f0 + col;
        if (a < d.len_a && f < d.len_f)
            tile[r][col] = src[(long)a * d.in_stride_a + f];
    }
    __syncthreads();
#pragma unroll 4
    for (int r = row0; r < TILE; r += kBlock / TILE) {
        const int f = f0 + r, a = a0 + col;
        if (a < d.len_a && f < d.len_f)
            dst[(long)f * d.out_stride_f + a] = tile[col][r];
    }
}

// ---- gather --------------------------------------------------------------------------------------
// one workgroup per output row; rows are copied in 16-byte or 4-byte words when the slice size allows it.
__global__ void __launch_bounds__(kBlock) gather_kernel(const char *__restrict__ data, const int32_t *__restrict__ idx,
                                                        char *__restrict__ out, int slices, size_t slice_bytes,
                                                        int n_indices, int32_t *error_flag) {
    int row   = blockIdx.x;  // b * n_indices + i
    int b     = row / n_indices;
    int i     = row - b * n_indices;
    int s     = idx[i];
    if (s < 0)
        s += slices;
    bool bad        = (s < 0 || s >= slices);
    const char *src = data + ((size_t)b * slices + (bad ? 0 : s)) * slice_bytes;
    char *dst       = out + (size_t)row * slice_bytes;
    if (bad && threadIdx.x == 0 && error_flag)
        *error_flag = 1;
    if ((slice_bytes & 15) == 0 && ((((uintptr_t)src) | ((uintptr_t)dst)) & 15) == 0) {
        size_t vecs = slice_bytes >> 4;
        for (size_t w = threadIdx.x; w < vecs; w += blockDim.x)
            reinterpret_cast<uint4 *>(dst)[w] = bad ? make_uint4(0, 0, 0, 0) : reinterpret_cast<const uint4 *>(src)[w];
    } else if ((slice_bytes & 3) == 0 && ((((uintptr_t)src) | ((uintptr_t)dst)) & 3) == 0) {
        size_t words = slice_bytes >> 2;
        for (size_t w = threadIdx.x; w < words; w += blockDim.x)
            reinterpret_cast<uint32_t *>(dst)[w] = bad ? 0u : reinterpret_cast<const uint32_t *>(src)[w];
    } else {
        for (size_t w = threadIdx.x; w < slice_bytes; w += blockDim.x)
            dst[w] = bad ? 0 : src[w];
    }
}

// ---- casts ---------------------------------------------------------------------------------------
template <int SDT, int DDT>
__global__ void __launch_bounds__(kBlock) cast_kernel(const typename Elem<SDT>::type *__restrict__ x,
                                                      typename Elem<DDT>::type *__restrict__ y, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t n4     = n / 4;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            Elem<DDT>::st(&y[i * 4 + j], Elem<SDT>::ld(&x[i * 4 + j]));
    }
    size_t t = n4 * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n)
        Elem<DDT>::st(&y[t], Elem<SDT>::ld(&x[t]));
}

// ---- int8 boundary ops -----------------------------------------------------------------------------
template <int DT>
__global__ void __launch_bounds__(kBlock) quantize_kernel(const typename Elem<DT>::type *__restrict__ x, float inv,
                                                          int8_t *__restrict__ q, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t n4     = n / 4;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        char4 o;
        o.x = float2int8_ref(__fmul_rn(Elem<DT>::ld(&x[i * 4 + 0]), inv));
        o.y = float2int8_ref(__fmul_rn(Elem<DT>::ld(&x[i * 4 + 1]), inv));
        o.z = float2int8_ref(__fmul_rn(Elem<DT>::ld(&x[i * 4 + 2]), inv));
        o.w = float2int8_ref(__fmul_rn(Elem<DT>::ld(&x[i * 4 + 3]), inv));
        if ((((uintptr_t)q) & 3) == 0) {
            reinterpret_cast<char4 *>(q)[i] = o;
        } else {
            q[i * 4 + 0] = o.x;
            q[i * 4 + 1] = o.y;
            q[i * 4 + 2] = o.z;
            q[i * 4 + 3] = o.w;
        }
    }
    size_t t = n4 * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n)
        q[t] = float2int8_ref(__fmul_rn(Elem<DT>::ld(&x[t]), inv));
}

template <int DT>
__global__ void __launch_bounds__(kBlock) dequantize_kernel(const int8_t *__restrict__ q, float scale,
                                                            typename Elem<DT>::type *__restrict__ x, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        Elem<DT>::st(&x[i], __fmul_rn((float)q[i], scale));
}

// one scale per channel (a device array of `channels` values; element i belongs to channel (i / inner) % channels): the
// blob scales the reference's int8 unit tests generate, and what its Reformat kernels take (x86_compute_int8.cc:1193-1318)
template <int DT>
__global__ void __launch_bounds__(kBlock) quantize_per_channel_kernel(const typename Elem<DT>::type *__restrict__ x,
                                                                      const float *__restrict__ inv, int8_t *__restrict__ q,
                                                                      size_t n, unsigned channels, size_t inner) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        q[i] = float2int8_ref(__fmul_rn(Elem<DT>::ld(&x[i]), inv[(i / inner) % channels]));
}

template <int DT>
__global__ void __launch_bounds__(kBlock) dequantize_per_channel_kernel(const int8_t *__restrict__ q,
                                                                        const float *__restrict__ scale,
                                                                        typename Elem<DT>::type *__restrict__ x, size_t n,
                                                                        unsigned channels, size_t inner) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        Elem<DT>::st(&x[i], __fmul_rn((float)q[i], scale[(i / inner) % channels]));
}

// sixteen values per lane and access; value for value the scalar kernel's arithmetic
template <int DT>
__global__ void __launch_bounds__(kBlock) dequantize_vec_kernel(const int8_t *__restrict__ q, float scale,
                                                                typename Elem<DT>::type *__restrict__ x, size_t n) {
    typedef typename Elem<DT>::type T;
    const size_t stride = (size_t)gridDim.x * blockDim.x, first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nvec   = n / 16;
    for (size_t i = first; i < nvec; i += stride) {
        const u32x4 v = reinterpret_cast<const u32x4 *>(q)[i];
        __attribute__((aligned(16))) T o[16];
#pragma unroll
        for (int w = 0; w < 4; ++w)
#pragma unroll
            for (int b = 0; b < 4; ++b)
                Elem<DT>::st(&o[w * 4 + b], __fmul_rn((float)(int8_t)((v[w] >> (8 * b)) & 0xffu), scale));
        uint4 *dst = reinterpret_cast<uint4 *>(x + i * 16);
#pragma unroll
        for (int k = 0; k < (int)sizeof(T); ++k)
            dst[k] = reinterpret_cast<const uint4 *>(o)[k];
    }
    for (size_t t = nvec * 16 + first; t < n; t += stride)
        Elem<DT>::st(&x[t], __fmul_rn((float)q[t], scale));
}

// int8 Add in the form the reference's x86 build computes (x86_compute_int8.cc:795-831 compiled with -mfma
// -ffast-math, device/x86/CMakeLists.txt:1-27: one product is contracted into the sum).  Its 8-channel vector body
// evaluates fma(b, sb, a*sa); the scalar tail - the last four channels when round_up(channels, 4) % 8 == 4 -
// evaluates fma(a, sa, b*sb).  `body` selects the form.
__device__ __forceinline__ int8_t add_i8_value(int8_t a, float sa, int8_t b, float sb, float inv_so, bool body) {
    const float fa = (float)a, fb = (float)b;
    const float s  = body ? fmaf(fb, sb, __fmul_rn(fa, sa)) : fmaf(fa, sa, __fmul_rn(fb, sb));
    return float2int8_ref(__fmul_rn(s, inv_so));
}

__global__ void __launch_bounds__(kBlock) add_i8_vec_kernel(const int8_t *__restrict__ a, float sa,
                                                            const int8_t *__restrict__ b, float sb, float inv_so,
                                                            int8_t *__restrict__ y, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x, first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nvec   = n / 16;
    for (size_t i = first; i < nvec; i += stride) {
        const u32x4 va = reinterpret_cast<const u32x4 *>(a)[i], vb = reinterpret_cast<const u32x4 *>(b)[i];
        u32x4 o;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            uint32_t packed = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int8_t qa = (int8_t)((va[w] >> (8 * k)) & 0xffu), qb = (int8_t)((vb[w] >> (8 * k)) & 0xffu);
                packed |= ((uint32_t)(uint8_t)add_i8_value(qa, sa, qb, sb, inv_so, true)) << (8 * k);
            }
            o[w] = packed;
        }
        reinterpret_cast<u32x4 *>(y)[i] = o;
    }
    for (size_t t = nvec * 16 + first; t < n; t += stride)
        y[t] = add_i8_value(a[t], sa, b[t], sb, inv_so, true);
}

// any alignment; channels from `tail_from` on (channel = (i / inner) % channels) take the scalar-tail form
__global__ void __launch_bounds__(kBlock) add_i8_kernel(const int8_t *__restrict__ a, float sa,
                                                        const int8_t *__restrict__ b, float sb, float inv_so,
                                                        int8_t *__restrict__ y, size_t n, unsigned channels,
                                                        size_t inner, unsigned tail_from) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const bool body = tail_from >= channels || (unsigned)((i / inner) % channels) < tail_from;
        y[i]            = add_i8_value(a[i], sa, b[i], sb, inv_so, body);
    }
}

// the same with one scale per channel for each of the three blobs (device arrays of `channels` values)
__global__ void __launch_bounds__(kBlock) add_i8_per_channel_kernel(const int8_t *__restrict__ a, const float *__restrict__ sa,
                                                                    const int8_t *__restrict__ b, const float *__restrict__ sb,
                                                                    const float *__restrict__ inv_so, int8_t *__restrict__ y,
                                                                    size_t n, unsigned channels, size_t inner,
                                                                    unsigned tail_from) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const unsigned c = (unsigned)((i / inner) % channels);
        y[i]             = add_i8_value(a[i], sa[c], b[i], sb[c], inv_so[c], tail_from >= channels || c < tail_from);
    }
}

// int8 -> GELU -> int8 has only 256 possible inputs, so the chain (dequantise, erf GELU, quantise) is a 256-entry
// table.  The launcher evaluates it on the host with the C library's double erf - the very routine the reference's
// CPU path calls - and hands it over by value as a kernel argument (256 bytes: no device memory, no copy, safe under
// graph capture); every workgroup copies it to LDS and maps bytes through it, sixteen per thread and access.
struct GeluTable {
    int8_t q[256];
};
__global__ void __launch_bounds__(256) gelu_i8_kernel(const int8_t *__restrict__ qi, GeluTable tab,
                                                      int8_t *__restrict__ qo, size_t n, int vector_ok) {
    __shared__ int8_t table[256];
    table[threadIdx.x] = tab.q[threadIdx.x];
    __syncthreads();
    const size_t stride = (size_t)gridDim.x * blockDim.x, first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nvec   = vector_ok ? n / 16 : 0;
    for (size_t i = first; i < nvec; i += stride) {
        u32x4 v = reinterpret_cast<const u32x4 *>(qi)[i];
        u32x4 o;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            uint32_t in = v[w], out = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                uint32_t idx = (((in >> (8 * b)) & 0xffu) ^ 0x80u);  // int8 value + 128
                out |= (uint32_t)(uint8_t)table[idx] << (8 * b);
            }
            o[w] = out;
        }
        reinterpret_cast<u32x4 *>(qo)[i] = o;
    }
    for (size_t i = nvec * 16 + first; i < n; i += stride)
        qo[i] = table[(int)qi[i] + 128];
}

}  // namespace

namespace {
// int32 <-> float types: static_cast both ways as the CPU path (cpu_cast_layer_acc.cc:41-53); a float outside the int
// range saturates here (the C++ conversion is undefined there)
template <int DDT>
__global__ void __launch_bounds__(kBlock) cast_from_i32_kernel(const int32_t *__restrict__ x,
                                                               typename Elem<DDT>::type *__restrict__ y, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        Elem<DDT>::st(&y[i], (float)x[i]);
}
template <int SDT>
__global__ void __launch_bounds__(kBlock) cast_to_i32_kernel(const typename Elem<SDT>::type *__restrict__ x,
                                                             int32_t *__restrict__ y, size_t n) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        y[i] = (int32_t)Elem<SDT>::ld(&x[i]);
}

}  // namespace

extern "C" {

int tnn_rocm_gelu(void *stream, int dtype, const void *x, void *y, size_t count) {
    if (count == 0)
        return 0;
    TR_REQUIRE(x && y, TNN_ROCM_EINVAL, "gelu: null pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case TNN_ROCM_F32: return launch_unary<TNN_ROCM_F32>(s, x, y, count, GeluOp());
        case TNN_ROCM_F16: return launch_unary<TNN_ROCM_F16>(s, x, y, count, GeluHalfOp());
        case TNN_ROCM_BF16: return launch_unary<TNN_ROCM_BF16>(s, x, y, count, GeluHalfOp());
        default: set_error("gelu: unsupported dtype %d", dtype); return TNN_ROCM_EDTYPE;
    }
}

int tnn_rocm_tanh(void *stream, int dtype, const void *x, void *y, size_t count) {
    if (count == 0)
        return 0;
    TR_REQUIRE(x && y, TNN_ROCM_EINVAL, "tanh: null pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case TNN_ROCM_F32: return launch_unary<TNN_ROCM_F32>(s, x, y, count, TanhOp());
        case TNN_ROCM_F16: return launch_unary<TNN_ROCM_F16>(s, x, y, count, TanhOp());
        case TNN_ROCM_BF16: return launch_unary<TNN_ROCM_BF16>(s, x, y, count, TanhOp());
        default: set_error("tanh: unsupported dtype %d", dtype); return TNN_ROCM_EDTYPE;
    }
}

int tnn_rocm_binary(void *stream, int dtype, int op, const void *a, const int *sa, int ra, const void *b,
                    const int *sb, int rb, void *out, const int *so, int ro) {
    TR_REQUIRE(a && b && out && sa && sb && so, TNN_ROCM_EINVAL, "binary: null pointer");
    TR_REQUIRE(ro >= 1 && ro <= 6 && ra >= 0 && ra <= ro && rb >= 0 && rb <= ro, TNN_ROCM_ESHAPE,
               "binary: ranks a=%d b=%d out=%d unsupported (max 6, operands may not exceed the output rank)", ra, rb,
               ro);
    BcastDesc d;
    d.rank   = ro;
    size_t n = 1;
    for (int i = 0; i < 6; ++i) {
        d.out_dim[i]  = 1;
        d.a_stride[i] = 0;
        d.b_stride[i] = 0;
    }
    for (int i = 0; i < ro; ++i) {
        TR_REQUIRE(so[i] >= 0, TNN_ROCM_ESHAPE, "binary: negative dim");
        d.out_dim[i] = so[i];
        n *= (size_t)so[i];
    }
    if (n == 0)
        return 0;
    // right-aligned strides; an operand dim of 1 (or smaller than the output) broadcasts.
    auto fill = [&](const int *shape, int rank, long *stride) -> bool {
        long acc = 1;
        for (int i = rank - 1; i >= 0; --i) {
            int oi = i + (ro - rank);
            if (shape[i] == so[oi])
                stride[oi] = acc;
            else if (shape[i] == 1)
                stride[oi] = 0;
            else
                return false;
            acc *= shape[i];
        }
        return true;
    };
    TR_REQUIRE(fill(sa, ra, d.a_stride) && fill(sb, rb, d.b_stride), TNN_ROCM_ESHAPE,
               "binary: operand shape does not broadcast to the output shape");
    // classify the fast cases: a has the full output shape and b is scalar / last-axis vector / full.
    size_t na = 1, nb = 1;
    for (int i = 0; i < ra; ++i)
        na *= (size_t)sa[i];
    for (int i = 0; i < rb; ++i)
        nb *= (size_t)sb[i];
    int fast_kind = 0, cols = so[ro - 1];
    if (na == n) {
        if (nb == 1)
            fast_kind = 2;
        else if (nb == n)
            fast_kind = 3;
        else if (nb == (size_t)cols && rb >= 1 && sb[rb - 1] == cols)
            fast_kind = 1;
    }
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case TNN_ROCM_F32: return launch_binary<TNN_ROCM_F32>(s, op, a, b, out, n, d, fast_kind, cols);
        case TNN_ROCM_F16: return launch_binary<TNN_ROCM_F16>(s, op, a, b, out, n, d, fast_kind, cols);
        case TNN_ROCM_BF16: return launch_binary<TNN_ROCM_BF16>(s, op, a, b, out, n, d, fast_kind, cols);
        default: set_error("binary: unsupported dtype %d", dtype); return TNN_ROCM_EDTYPE;
    }
}

int tnn_rocm_permute(void *stream, int elem_bytes, const void *in, void *out, const int *in_dims, const int *order,
                     int rank) {
    TR_REQUIRE(in && out && in_dims && order, TNN_ROCM_EINVAL, "permute: null pointer");
    TR_REQUIRE(rank >= 1 && rank <= 6, TNN_ROCM_ESHAPE, "permute: rank %d unsupported (1..6)", rank);
    size_t n = 1;
    bool seen[6] = {false, false, false, false, false, false};
    for (int i = rank - 1; i >= 0; --i) {
        TR_REQUIRE(in_dims[i] >= 0, TNN_ROCM_ESHAPE, "permute: negative dim");
        n *= (size_t)in_dims[i];
    }
    for (int j = 0; j < rank; ++j) {
        TR_REQUIRE(order[j] >= 0 && order[j] < rank && !seen[order[j]], TNN_ROCM_EINVAL,
                   "permute: order is not a permutation");
        seen[order[j]] = true;
    }
    if (n == 0)
        return 0;
    hipStream_t s = (hipStream_t)stream;
    // Normal form: axes of extent 1 dropped, input axes that stay neighbours in the output merged.  nd / nord
    // describe the same copy with as few axes as possible (output position -> input axis).
    int nd[6], nord[6], nrank = 0;
    {
        int keep_pos[6], kept = 0;  // output positions with extent > 1
        for (int j = 0; j < rank; ++j)
            if (in_dims[order[j]] != 1)
                keep_pos[kept++] = j;
        // runs of output positions whose input axes are consecutive (ignoring extent-1 axes in between)
        int run_first_axis[6], run_len_elems[6], runs = 0;
        for (int k = 0; k < kept; ++k) {
            const int ax = order[keep_pos[k]];
            bool joins = false;
            if (runs > 0) {
                const int prev = order[keep_pos[k - 1]];
                joins = ax > prev;
                for (int t = prev + 1; joins && t < ax; ++t)
                    joins = in_dims[t] == 1;
            }
            if (joins && (long)run_len_elems[runs - 1] * in_dims[ax] < (1l << 31)) {
                run_len_elems[runs - 1] *= in_dims[ax];
            } else {
                run_first_axis[runs] = ax;
                run_len_elems[runs]  = in_dims[ax];
                ++runs;
            }
        }
        // input order of the runs = order of their first axes
        int rank_of_run[6];
        for (int a = 0; a < runs; ++a) {
            int pos = 0;
            for (int b = 0; b < runs; ++b)
                pos += run_first_axis[b] < run_first_axis[a];
            rank_of_run[a] = pos;
        }
        nrank = runs;
        for (int a = 0; a < runs; ++a) {
            nord[a]              = rank_of_run[a];
            nd[rank_of_run[a]]   = run_len_elems[a];
        }
        if (nrank == 0) {  // a single element
            nrank = 1, nd[0] = 1, nord[0] = 0;
        }
    }
    long nin_stride[6], nout_stride_of_in_axis[6];
    {
        long acc = 1;
        for (int i = nrank - 1; i >= 0; --i) {
            nin_stride[i] = acc;
            acc *= nd[i];
        }
        acc = 1;
        for (int j = nrank - 1; j >= 0; --j) {
            nout_stride_of_in_axis[nord[j]] = acc;
            acc *= nd[nord[j]];
        }
    }
    auto generic = [&](int unit_bytes, const int *dims_u) -> int {
        // element-wise gather over units of unit_bytes (the innermost input axis re-expressed in those units)
        PermDesc d;
        d.rank = nrank;
        for (int j = 0; j < 6; ++j) {
            d.out_dim[j]               = 1;
            d.in_stride_of_out_axis[j] = 0;
        }
        long stride_u[6], acc = 1;
        size_t total = 1;
        for (int i = nrank - 1; i >= 0; --i) {
            stride_u[i] = acc;
            acc *= dims_u[i];
            total *= (size_t)dims_u[i];
        }
        for (int j = 0; j < nrank; ++j) {
            d.out_dim[j]               = dims_u[nord[j]];
            d.in_stride_of_out_axis[j] = stride_u[nord[j]];
        }
        switch (unit_bytes) {
            case 1:
                hipLaunchKernelGGL(permute_kernel<uint8_t>, dim3(grid_for(total)), dim3(kBlock), 0, s,
                                   (const uint8_t *)in, (uint8_t *)out, total, d);
                break;
            case 2:
                hipLaunchKernelGGL(permute_kernel<uint16_t>, dim3(grid_for(total)), dim3(kBlock), 0, s,
                                   (const uint16_t *)in, (uint16_t *)out, total, d);
                break;
            case 4:
                hipLaunchKernelGGL(permute_kernel<uint32_t>, dim3(grid_for(total)), dim3(kBlock), 0, s,
                                   (const uint32_t *)in, (uint32_t *)out, total, d);
                break;
            case 16:
                hipLaunchKernelGGL(permute_kernel<uint4>, dim3(grid_for(total)), dim3(kBlock), 0, s, (const uint4 *)in,
                                   (uint4 *)out, total, d);
                break;
            default: set_error("permute: element size %d unsupported", unit_bytes); return TNN_ROCM_EDTYPE;
        }
        TR_CHECK_LAUNCH();
        return 0;
    };
    TR_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, TNN_ROCM_EDTYPE,
               "permute: element size %d unsupported", elem_bytes);
    if (nord[nrank - 1] == nrank - 1) {
        // the innermost run is copied as it is: move it in 16-byte (else 4-byte) units when it divides and is aligned
        const long inner_bytes = (long)nd[nrank - 1] * elem_bytes;
        int dims_u[6];
        for (int i = 0; i < nrank; ++i)
            dims_u[i] = nd[i];
        if (inner_bytes % 16 == 0 && aligned16(in) && aligned16(out)) {
            dims_u[nrank - 1] = (int)(inner_bytes / 16);
            return generic(16, dims_u);
        }
        if (inner_bytes % 4 == 0 && (((uintptr_t)in | (uintptr_t)out) & 3) == 0) {
            dims_u[nrank - 1] = (int)(inner_bytes / 4);
            return generic(4, dims_u);
        }
        return generic(elem_bytes, nd);
    }
    // the output's fastest axis differs from the input's: tiled transpose over that pair of axes
    {
        TransDesc t;
        const int F = nrank - 1, A = nord[nrank - 1];
        t.n_batch_axes = 0;
        size_t batch   = 1;
        for (int i = 0; i < nrank; ++i)
            if (i != F && i != A) {
                t.batch_dim[t.n_batch_axes]        = nd[i];
                t.batch_in_stride[t.n_batch_axes]  = nin_stride[i];
                t.batch_out_stride[t.n_batch_axes] = nout_stride_of_in_axis[i];
                ++t.n_batch_axes;
                batch *= (size_t)nd[i];
            }
        for (int k = t.n_batch_axes; k < 4; ++k)
            t.batch_dim[k] = 1, t.batch_in_stride[k] = 0, t.batch_out_stride[k] = 0;
        t.len_f        = nd[F];
        t.len_a        = nd[A];
        t.in_stride_a  = nin_stride[A];
        t.out_stride_f = nout_stride_of_in_axis[F];
        t.tiles_f      = (t.len_f + 63) / 64;
        t.tiles_a      = (t.len_a + 63) / 64;
        const size_t blocks = (size_t)t.tiles_f * t.tiles_a * batch;
        if (blocks >= (1ull << 31))
            return generic(elem_bytes, nd);
        switch (elem_bytes) {
            case 1:
                hipLaunchKernelGGL(permute_transpose_kernel<uint8_t>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                                   (const uint8_t *)in, (uint8_t *)out, t);
                break;
            case 2:
                hipLaunchKernelGGL(permute_transpose_kernel<uint16_t>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                                   (const uint16_t *)in, (uint16_t *)out, t);
                break;
            default:
                hipLaunchKernelGGL(permute_transpose_kernel<uint32_t>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                                   (const uint32_t *)in, (uint32_t *)out, t);
                break;
        }
    }
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_gather(void *stream, const void *data, const int32_t *indices, void *out, int batch, int slices,
                    size_t slice_bytes, int n_indices, int32_t *error_flag) {
    TR_REQUIRE(batch >= 0 && slices >= 0 && n_indices >= 0, TNN_ROCM_ESHAPE, "gather: negative size");
    if (batch == 0 || n_indices == 0 || slice_bytes == 0)
        return 0;
    TR_REQUIRE(data && indices && out, TNN_ROCM_EINVAL, "gather: null pointer");
    TR_REQUIRE(slices > 0, TNN_ROCM_ESHAPE, "gather: empty table");
    TR_REQUIRE((long)batch * n_indices < (1l << 31), TNN_ROCM_ESHAPE, "gather: too many rows");
    // a row is copied by as many waves as it has 16-byte vectors to hand out (1536-byte rows: two waves, not four)
    size_t lanes = (slice_bytes / 16 + 63) / 64 * 64;
    lanes        = lanes < 64 ? 64 : (lanes > (size_t)kBlock ? (size_t)kBlock : lanes);
    hipLaunchKernelGGL(gather_kernel, dim3(batch * n_indices), dim3((unsigned)lanes), 0, (hipStream_t)stream,
                       (const char *)data, indices, (char *)out, slices, slice_bytes, n_indices, error_flag);
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_cast(void *stream, int sdt, const void *src, int ddt, void *dst, size_t n) {
    if (n == 0)
        return 0;
    TR_REQUIRE(src && dst, TNN_ROCM_EINVAL, "cast: null pointer");
    hipStream_t s = (hipStream_t)stream;
    int g         = grid_for(n / 4 + 4);
#define TR_CAST(S, D)                                                                                                 \
    if (sdt == S && ddt == D) {                                                                                       \
        hipLaunchKernelGGL((cast_kernel<S, D>), dim3(g), dim3(kBlock), 0, s, (const Elem<S>::type *)src,              \
                           (Elem<D>::type *)dst, n);                                                                  \
        TR_CHECK_LAUNCH();                                                                                            \
        return 0;                                                                                                     \
    }
    TR_CAST(TNN_ROCM_F32, TNN_ROCM_F16)
    TR_CAST(TNN_ROCM_F16, TNN_ROCM_F32)
    TR_CAST(TNN_ROCM_F32, TNN_ROCM_BF16)
    TR_CAST(TNN_ROCM_BF16, TNN_ROCM_F32)
    TR_CAST(TNN_ROCM_F16, TNN_ROCM_BF16)
    TR_CAST(TNN_ROCM_BF16, TNN_ROCM_F16)
    TR_CAST(TNN_ROCM_F32, TNN_ROCM_F32)
    TR_CAST(TNN_ROCM_F16, TNN_ROCM_F16)
    TR_CAST(TNN_ROCM_BF16, TNN_ROCM_BF16)
#undef TR_CAST
#define TR_CAST_I32(F)                                                                                                \
    if (sdt == TNN_ROCM_I32 && ddt == F) {                                                                            \
        hipLaunchKernelGGL((cast_from_i32_kernel<F>), dim3(grid_for(n)), dim3(kBlock), 0, s, (const int32_t *)src,    \
                           (Elem<F>::type *)dst, n);                                                                  \
        TR_CHECK_LAUNCH();                                                                                            \
        return 0;                                                                                                     \
    }                                                                                                                 \
    if (sdt == F && ddt == TNN_ROCM_I32) {                                                                            \
        hipLaunchKernelGGL((cast_to_i32_kernel<F>), dim3(grid_for(n)), dim3(kBlock), 0, s, (const Elem<F>::type *)src, \
                           (int32_t *)dst, n);                                                                        \
        TR_CHECK_LAUNCH();                                                                                            \
        return 0;                                                                                                     \
    }
    TR_CAST_I32(TNN_ROCM_F32)
    TR_CAST_I32(TNN_ROCM_F16)
    TR_CAST_I32(TNN_ROCM_BF16)
#undef TR_CAST_I32
    if (sdt == TNN_ROCM_I32 && ddt == TNN_ROCM_I32) {
        TR_CHECK_HIP(hipMemcpyAsync(dst, src, n * sizeof(int32_t), hipMemcpyDeviceToDevice, s));
        return 0;
    }
    set_error("cast: unsupported dtype pair %d -> %d", sdt, ddt);
    return TNN_ROCM_EDTYPE;
}

int tnn_rocm_quantize(void *stream, int sdt, const void *x, float inv_scale, int8_t *q, size_t n) {
    if (n == 0)
        return 0;
    TR_REQUIRE(x && q, TNN_ROCM_EINVAL, "quantize: null pointer");
    hipStream_t s = (hipStream_t)stream;
    int g         = grid_for(n / 4 + 4);
    switch (sdt) {
        case TNN_ROCM_F32:
            hipLaunchKernelGGL(quantize_kernel<TNN_ROCM_F32>, dim3(g), dim3(kBlock), 0, s, (const float *)x, inv_scale,
                               q, n);
            break;
        case TNN_ROCM_F16:
            hipLaunchKernelGGL(quantize_kernel<TNN_ROCM_F16>, dim3(g), dim3(kBlock), 0, s, (const half_t *)x,
                               inv_scale, q, n);
            break;
        case TNN_ROCM_BF16:
            hipLaunchKernelGGL(quantize_kernel<TNN_ROCM_BF16>, dim3(g), dim3(kBlock), 0, s, (const bf16_bits *)x,
                               inv_scale, q, n);
            break;
        default: set_error("quantize: unsupported source dtype %d", sdt); return TNN_ROCM_EDTYPE;
    }
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_dequantize(void *stream, const int8_t *q, float scale, int ddt, void *x, size_t n) {
    if (n == 0)
        return 0;
    TR_REQUIRE(x && q, TNN_ROCM_EINVAL, "dequantize: null pointer");
    hipStream_t s = (hipStream_t)stream;
    int g         = grid_for(n);
    if (aligned16(q) && aligned16(x) && n >= 16) {
        g = grid_for(n / 16);
        switch (ddt) {
            case TNN_ROCM_F32:
                hipLaunchKernelGGL(dequantize_vec_kernel<TNN_ROCM_F32>, dim3(g), dim3(kBlock), 0, s, q, scale, (float *)x,
                                   n);
                break;
            case TNN_ROCM_F16:
                hipLaunchKernelGGL(dequantize_vec_kernel<TNN_ROCM_F16>, dim3(g), dim3(kBlock), 0, s, q, scale, (half_t *)x,
                                   n);
                break;
            case TNN_ROCM_BF16:
                hipLaunchKernelGGL(dequantize_vec_kernel<TNN_ROCM_BF16>, dim3(g), dim3(kBlock), 0, s, q, scale,
                                   (bf16_bits *)x, n);
                break;
            default: set_error("dequantize: unsupported destination dtype %d", ddt); return TNN_ROCM_EDTYPE;
        }
        TR_CHECK_LAUNCH();
        return 0;
    }
    switch (ddt) {
        case TNN_ROCM_F32:
            hipLaunchKernelGGL(dequantize_kernel<TNN_ROCM_F32>, dim3(g), dim3(kBlock), 0, s, q, scale, (float *)x, n);
            break;
        case TNN_ROCM_F16:
            hipLaunchKernelGGL(dequantize_kernel<TNN_ROCM_F16>, dim3(g), dim3(kBlock), 0, s, q, scale, (half_t *)x, n);
            break;
        case TNN_ROCM_BF16:
            hipLaunchKernelGGL(dequantize_kernel<TNN_ROCM_BF16>, dim3(g), dim3(kBlock), 0, s, q, scale, (bf16_bits *)x,
                               n);
            break;
        default: set_error("dequantize: unsupported destination dtype %d", ddt); return TNN_ROCM_EDTYPE;
    }
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_quantize_per_channel(void *stream, int sdt, const void *x, const float *inv_scale, int8_t *q, size_t n,
                                  int channels, size_t inner) {
    if (n == 0)
        return 0;
    TR_REQUIRE(x && q && inv_scale, TNN_ROCM_EINVAL, "quantize_per_channel: null pointer");
    TR_REQUIRE(channels >= 1 && inner >= 1, TNN_ROCM_EINVAL, "quantize_per_channel: channels %d, inner %zu", channels, inner);
    hipStream_t s = (hipStream_t)stream;
    const int g   = grid_for(n);
    switch (sdt) {
        case TNN_ROCM_F32:
            hipLaunchKernelGGL(quantize_per_channel_kernel<TNN_ROCM_F32>, dim3(g), dim3(kBlock), 0, s, (const float *)x,
                               inv_scale, q, n, (unsigned)channels, inner);
            break;
        case TNN_ROCM_F16:
            hipLaunchKernelGGL(quantize_per_channel_kernel<TNN_ROCM_F16>, dim3(g), dim3(kBlock), 0, s, (const half_t *)x,
                               inv_scale, q, n, (unsigned)channels, inner);
            break;
        case TNN_ROCM_BF16:
            hipLaunchKernelGGL(quantize_per_channel_kernel<TNN_ROCM_BF16>, dim3(g), dim3(kBlock), 0, s,
                               (const bf16_bits *)x, inv_scale, q, n, (unsigned)channels, inner);
            break;
        default: set_error("quantize_per_channel: unsupported source dtype %d", sdt); return TNN_ROCM_EDTYPE;
    }
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_dequantize_per_channel(void *stream, const int8_t *q, const float *scale, int ddt, void *x, size_t n,
                                    int channels, size_t inner) {
    if (n == 0)
        return 0;
    TR_REQUIRE(x && q && scale, TNN_ROCM_EINVAL, "dequantize_per_channel: null pointer");
    TR_REQUIRE(channels >= 1 && inner >= 1, TNN_ROCM_EINVAL, "dequantize_per_channel: channels %d, inner %zu", channels, inner);
    hipStream_t s = (hipStream_t)stream;
    const int g   = grid_for(n);
    switch (ddt) {
        case TNN_ROCM_F32:
            hipLaunchKernelGGL(dequantize_per_channel_kernel<TNN_ROCM_F32>, dim3(g), dim3(kBlock), 0, s, q, scale, (float *)x,
                               n, (unsigned)channels, inner);
            break;
        case TNN_ROCM_F16:
            hipLaunchKernelGGL(dequantize_per_channel_kernel<TNN_ROCM_F16>, dim3(g), dim3(kBlock), 0, s, q, scale,
                               (half_t *)x, n, (unsigned)channels, inner);
            break;
        case TNN_ROCM_BF16:
            hipLaunchKernelGGL(dequantize_per_channel_kernel<TNN_ROCM_BF16>, dim3(g), dim3(kBlock), 0, s, q, scale,
                               (bf16_bits *)x, n, (unsigned)channels, inner);
            break;
        default: set_error("dequantize_per_channel: unsupported destination dtype %d", ddt); return TNN_ROCM_EDTYPE;
    }
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_add_i8(void *stream, const int8_t *a, float sa, const int8_t *b, float sb, float inv_so, int8_t *y,
                    size_t n, int channels, size_t inner) {
    if (n == 0)
        return 0;
    TR_REQUIRE(a && b && y, TNN_ROCM_EINVAL, "add_i8: null pointer");
    TR_REQUIRE(channels >= 1 && inner >= 1, TNN_ROCM_EINVAL, "add_i8: channels %d, inner %zu", channels, inner);
    const int c4        = (channels + 3) / 4 * 4;
    const int tail_from = c4 % 8 == 4 ? c4 - 4 : c4;  // first channel of the reference loop's scalar tail
    if (tail_from >= channels && aligned16(a) && aligned16(b) && aligned16(y) && n >= 16)
        hipLaunchKernelGGL(add_i8_vec_kernel, dim3(grid_for(n / 16)), dim3(kBlock), 0, (hipStream_t)stream, a, sa, b, sb,
                           inv_so, y, n);
    else
        hipLaunchKernelGGL(add_i8_kernel, dim3(grid_for(n)), dim3(kBlock), 0, (hipStream_t)stream, a, sa, b, sb, inv_so,
                           y, n, (unsigned)channels, inner, (unsigned)tail_from);
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_add_i8_per_channel(void *stream, const int8_t *a, const float *sa, const int8_t *b, const float *sb,
                                const float *inv_so, int8_t *y, size_t n, int channels, size_t inner) {
    if (n == 0)
        return 0;
    TR_REQUIRE(a && b && y && sa && sb && inv_so, TNN_ROCM_EINVAL, "add_i8_per_channel: null pointer");
    TR_REQUIRE(channels >= 1 && inner >= 1, TNN_ROCM_EINVAL, "add_i8_per_channel: channels %d, inner %zu", channels, inner);
    const int c4        = (channels + 3) / 4 * 4;
    const int tail_from = c4 % 8 == 4 ? c4 - 4 : c4;
    hipLaunchKernelGGL(add_i8_per_channel_kernel, dim3(grid_for(n)), dim3(kBlock), 0, (hipStream_t)stream, a, sa, b, sb,
                       inv_so, y, n, (unsigned)channels, inner, (unsigned)tail_from);
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_gelu_i8(void *stream, const int8_t *qi, float in_scale, float out_inv_scale, int8_t *qo, size_t n) {
    if (n == 0)
        return 0;
    TR_REQUIRE(qi && qo, TNN_ROCM_EINVAL, "gelu_i8: null pointer");
    // x86_compute_int8.cc:1193-1252 (q*scale), cpu_gelu_layer_acc.cc:42-45 (fp32 products, double erf, one rounding
    // to fp32), x86_compute_int8.cc:26-39 + 1254-1318 (x*(1/scale), +-0.5f, clamp, truncate)
    GeluTable tab;
    for (int q = -128; q < 128; ++q) {
        const float x  = (float)q * in_scale;
        const float hv = 0.5f * x;
        const double e = erf((double)(x * 0.707106793288165f)) + 1.0;
        const float g  = (float)((double)hv * e);
        float t        = g * out_inv_scale;
        t              = t + (t >= 0.f ? 0.5f : -0.5f);
        t              = t > 127.0f ? 127.0f : t;
        t              = t < -128.0f ? -128.0f : t;
        tab.q[q + 128] = (t != t) ? (int8_t)0 : (int8_t)(int)t;
    }
    const int vector_ok = ((uintptr_t)qi % 16 == 0 && (uintptr_t)qo % 16 == 0) ? 1 : 0;
    size_t blocks       = (n / 16 + 255) / 256;
    blocks              = blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks);
    hipLaunchKernelGGL(gelu_i8_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, qi, tab, qo, n,
                       vector_ok);
    TR_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
