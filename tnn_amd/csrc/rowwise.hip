// Row-wise HBM-bound kernels: LayerNorm (+residual, +int8 quantised copy) and Softmax.
//
// One 64-lane wavefront owns one row (LayerNorm rows of at most 128 vectors: half a wavefront): the row is read
// once with 16-byte accesses, kept in registers, reduced with cross-lane shuffles (no LDS), and written once.
// Four waves per workgroup, so a launch over T rows issues T/4 or T/8 workgroups (>> 256 CUs for encoder shapes).
#include "common.h"

using namespace tnn_rocm;

namespace {

constexpr int kBlock       = 256;
constexpr int kRowsPerBlk  = kBlock / kWave;
constexpr int kMaxVecPerLn = 8;  // row cached in registers when cols <= 64 * VEC * 8

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

// sum over each aligned group of LPR lanes (32: the two halves of a wave hold different rows)
template <int LPR>
__device__ __forceinline__ double lanes_sum_f64(double v) {
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

// ---- LayerNorm ----------------------------------------------------------------------------------
// Statistics follow the reference's one-pass form var = E[x^2] - E[x]^2 with its types: the square
// is an fp32 product, both sums, the mean, the variance and rstd are double.  An all-fp32
// E[x^2]-E[x]^2 loses the variance to cancellation when |mean| >> std.
// Optional row sources of the embedding front end: row r of the input is word_table[ids[r]] (x is the table),
// the residual is pos_table[r % period] (res is the table) and a second addend type_table[type_ids[r]]; the sum is
// ((word + pos) + type), the order of the Add layers it replaces.
struct EmbedRows {
    const int32_t *ids      = nullptr;  // null: plain LayerNorm
    const int32_t *type_ids = nullptr;
    const void *type_table  = nullptr;
    int vocab = 0, n_types = 0, period = 0;
    // optional third lookup: row r takes position row pos_ids[r % n_pos_ids] of a table of pos_rows rows
    const int32_t *pos_ids = nullptr;
    int n_pos_ids = 0, pos_rows = 0;
    int32_t *error_flag = nullptr;
};

// LPR lanes own one row (64: a wave per row; 32: a wave holds two rows, which keeps every lane busy and twice the
// bytes in flight for rows of at most 128 vectors); NV = 16-byte vectors a lane can hold.
template <int DT, bool VECTOR, int LPR, int NV>
__global__ void __launch_bounds__(kBlock) layernorm_kernel(const typename Elem<DT>::type *__restrict__ x,
                                                           const typename Elem<DT>::type *__restrict__ res,
                                                           const float *__restrict__ gamma,
                                                           const float *__restrict__ beta,
                                                           typename Elem<DT>::type *__restrict__ y, int rows, int cols,
                                                           float eps, int8_t *__restrict__ out_q, float q_inv,
                                                           EmbedRows emb) {
    typedef typename Elem<DT>::type T;
    constexpr int VEC = VECTOR ? (int)(16 / sizeof(T)) : 1;
    const int lane    = threadIdx.x & (LPR - 1);
    const int row     = (blockIdx.x * kRowsPerBlk + (threadIdx.x >> 6)) * (kWave / LPR) + ((threadIdx.x & (kWave - 1)) / LPR);
    if (row >= rows)
        return;  // the lanes of a row exit together; no workgroup barrier is used below and shuffles stay inside a row
    const T *px  = x + (size_t)row * cols;
    const T *pr  = res ? res + (size_t)row * cols : nullptr;
    const T *pr2 = nullptr;
    if (VECTOR && emb.ids) {
        // negative indices wrap, an index outside the table raises the flag and reads row 0
        // (cpu_gather_layer_acc.cc:27-86)
        int wi = emb.ids[row], ti = emb.type_ids[row];
        int pi = emb.pos_ids ? emb.pos_ids[row % emb.n_pos_ids] : row % emb.period;
        wi += wi < 0 ? emb.vocab : 0;
        ti += ti < 0 ? emb.n_types : 0;
        bool bad = wi < 0 || wi >= emb.vocab || ti < 0 || ti >= emb.n_types;
        if (emb.pos_ids) {
            pi += pi < 0 ? emb.pos_rows : 0;
            bad |= pi < 0 || pi >= emb.pos_rows;
        }
        if (bad) {
            if (lane == 0 && emb.error_flag)
                *emb.error_flag = 1;
            wi = 0, ti = 0, pi = 0;
        }
        px  = x + (size_t)wi * cols;
        pr  = res + (size_t)pi * cols;
        pr2 = reinterpret_cast<const T *>(emb.type_table) + (size_t)ti * cols;
    }
    T *py        = y + (size_t)row * cols;
    int8_t *pq   = out_q ? out_q + (size_t)row * cols : nullptr;
    const int nv = cols / VEC;  // VECTOR launches guarantee cols % VEC == 0

    float v[NV][VEC];
    double s1 = 0.0, s2 = 0.0;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        int vi = lane + j * LPR;
        if (vi < nv) {
            if (VECTOR) {
                uint4 raw = reinterpret_cast<const uint4 *>(px)[vi];
                const T *e = reinterpret_cast<const T *>(&raw);
                uint4 rraw, rraw2;
                const T *re = reinterpret_cast<const T *>(&rraw), *re2 = reinterpret_cast<const T *>(&rraw2);
                if (pr)
                    rraw = reinterpret_cast<const uint4 *>(pr)[vi];
                if (pr2)
                    rraw2 = reinterpret_cast<const uint4 *>(pr2)[vi];
#pragma unroll
                for (int t = 0; t < VEC; ++t) {
                    float f = Elem<DT>::ld(&e[t]);
                    if (pr)
                        f = __fadd_rn(f, Elem<DT>::ld(&re[t]));
                    if (pr2)
                        f = __fadd_rn(f, Elem<DT>::ld(&re2[t]));
                    v[j][t] = f;
                }
            } else {
                float f = Elem<DT>::ld(&px[vi]);
                if (pr)
                    f = __fadd_rn(f, Elem<DT>::ld(&pr[vi]));
                v[j][0] = f;
            }
#pragma unroll
            for (int t = 0; t < VEC; ++t) {
                s1 += (double)v[j][t];
                s2 += (double)__fmul_rn(v[j][t], v[j][t]);  // fp32 square, double sum (as the reference)
            }
        }
    }
    double d1    = lanes_sum_f64<LPR>(s1);
    double d2    = lanes_sum_f64<LPR>(s2);
    double mean  = d1 / cols;
    double var   = d2 / cols - mean * mean;
    double rstdd;
    if (DT == TNN_ROCM_F32) {
        rstdd = 1.0 / sqrt(var + (double)eps);  // the reference's expression, correctly rounded
    } else {
        // only the fp32 roundings of rstd and mean*rstd are used below: the hardware estimate (about 2^-26 relative)
        // refined by one Newton step is within a few double ulps, far inside what those roundings can see
        const double a = var + (double)eps;
        double r       = __builtin_amdgcn_rsq(a);
        rstdd          = r + r * (0.5 - 0.5 * a * r * r);
    }
    float rstd   = (float)rstdd;
    float mrs    = (float)(mean * rstdd);

#pragma unroll
    for (int j = 0; j < NV; ++j) {
        int vi = lane + j * LPR;
        if (vi < nv) {
            float o[VEC];
#pragma unroll
            for (int t = 0; t < VEC; ++t) {
                int c   = vi * VEC + t;
                float k = gamma[c];
                if (DT == TNN_ROCM_F32) {
                    // the reference's operand order and widths (cpu_layer_norm_layer_acc.cc:126-131): the shifted
                    // bias is formed in double and rounded to float, the affine combination is evaluated in double
                    float b = (float)((double)beta[c] - mean * rstdd * (double)k);
                    o[t]    = (float)((double)v[j][t] * rstdd * (double)k + (double)b);
                } else {
                    float b = beta[c] - mrs * k;
                    o[t]    = v[j][t] * rstd * k + b;
                }
            }
            if (VECTOR) {
                uint4 raw;
                T *e = reinterpret_cast<T *>(&raw);
#pragma unroll
                for (int t = 0; t < VEC; ++t)
                    Elem<DT>::st(&e[t], o[t]);
                store_out16(reinterpret_cast<uint4 *>(py) + vi, store_u32x4{raw.x, raw.y, raw.z, raw.w});
                if (pq) {  // the VEC (4 or 8) quantised values of this lane leave as one 4- or 8-byte store
                    uint32_t w[2] = {0u, 0u};
#pragma unroll
                    for (int t = 0; t < VEC; ++t) {
                        const int8_t q = float2int8_ref(__fmul_rn(Elem<DT>::ld(&e[t]), q_inv));
                        w[t >> 2] |= (uint32_t)(uint8_t)q << (8 * (t & 3));
                    }
                    if (VEC == 8)
                        store_out8(pq + (size_t)vi * VEC, store_u32x2{w[0], w[1]});
                    else
                        store_out4(pq + (size_t)vi * VEC, w[0]);
                }
            } else {
                T tmp;
                Elem<DT>::st(&tmp, o[0]);
                py[vi] = tmp;
                if (pq)
                    pq[vi] = float2int8_ref(__fmul_rn(Elem<DT>::ld(&tmp), q_inv));
            }
        }
    }
}

// Rows too long for the register cache: three passes over the row (statistics, then output).
template <int DT>
__global__ void __launch_bounds__(kBlock) layernorm_long_kernel(const typename Elem<DT>::type *__restrict__ x,
                                                                const typename Elem<DT>::type *__restrict__ res,
                                                                const float *__restrict__ gamma,
                                                                const float *__restrict__ beta,
                                                                typename Elem<DT>::type *__restrict__ y, int rows,
                                                                int cols, float eps, int8_t *__restrict__ out_q,
                                                                float q_inv) {
    typedef typename Elem<DT>::type T;
    const int lane = threadIdx.x & (kWave - 1);
    const int row  = blockIdx.x * kRowsPerBlk + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const T *px = x + (size_t)row * cols;
    const T *pr = res ? res + (size_t)row * cols : nullptr;
    T *py       = y + (size_t)row * cols;
    int8_t *pq  = out_q ? out_q + (size_t)row * cols : nullptr;
    double s1 = 0, s2 = 0;
    for (int c = lane; c < cols; c += kWave) {
        float f = Elem<DT>::ld(&px[c]);
        if (pr)
            f = __fadd_rn(f, Elem<DT>::ld(&pr[c]));
        s1 += (double)f;
        s2 += (double)__fmul_rn(f, f);
    }
    s1           = wave_sum_f64(s1);
    s2           = wave_sum_f64(s2);
    double mean  = s1 / cols;
    double var   = s2 / cols - mean * mean;
    double rstdd = 1.0 / sqrt(var + (double)eps);
    float rstd   = (float)rstdd;
    float mrs    = (float)(mean * rstdd);
    for (int c = lane; c < cols; c += kWave) {
        float f = Elem<DT>::ld(&px[c]);
        if (pr)
            f = __fadd_rn(f, Elem<DT>::ld(&pr[c]));
        float k = gamma[c];
        float o;
        if (DT == TNN_ROCM_F32) {
            float b = (float)((double)beta[c] - mean * rstdd * (double)k);
            o       = (float)((double)f * rstdd * (double)k + (double)b);
        } else {
            o = f * rstd * k + (beta[c] - mrs * k);
        }
        T tmp;
        Elem<DT>::st(&tmp, o);
        py[c] = tmp;
        if (pq)
            pq[c] = float2int8_ref(__fmul_rn(Elem<DT>::ld(&tmp), q_inv));
    }
}

template <int DT>
int launch_layernorm(hipStream_t s, const void *x, const void *res, const float *gamma, const float *beta, void *y,
                     int rows, int cols, float eps, int8_t *out_q, float q_inv, const EmbedRows &emb = EmbedRows()) {
    typedef typename Elem<DT>::type T;
    constexpr int VEC = 16 / sizeof(T);
    dim3 grid((rows + kRowsPerBlk - 1) / kRowsPerBlk), block(kBlock);
    const int nv = cols / VEC;
    bool al = ((((uintptr_t)x) | ((uintptr_t)y) | ((uintptr_t)res) | ((uintptr_t)emb.type_table) | ((uintptr_t)out_q)) & 15u) == 0 &&
              cols % VEC == 0;
    if (emb.ids && !(al && cols <= kWave * VEC * kMaxVecPerLn)) {
        set_error("embed_layernorm: hidden size %d needs 16-byte aligned rows of at most %d elements", cols,
                  kWave * VEC * kMaxVecPerLn);
        return TNN_ROCM_ESHAPE;
    }
    if (al && cols <= kWave * VEC * kMaxVecPerLn) {
#define TR_LN(LPR, NV)                                                                                                \
    hipLaunchKernelGGL((layernorm_kernel<DT, true, LPR, NV>),                                                         \
                       dim3((rows + kRowsPerBlk * (kWave / LPR) - 1) / (kRowsPerBlk * (kWave / LPR))), block, 0, s,   \
                       (const T *)x, (const T *)res, gamma, beta, (T *)y, rows, cols, eps, out_q, q_inv, emb)
        if (nv <= 64)
            TR_LN(32, 2);
        else if (nv <= 128)
            TR_LN(32, 4);
        else if (nv <= 256)
            TR_LN(64, 4);
        else
            TR_LN(64, 8);
#undef TR_LN
    } else if (cols <= kWave * kMaxVecPerLn) {
        hipLaunchKernelGGL((layernorm_kernel<DT, false, kWave, kMaxVecPerLn>), grid, block, 0, s, (const T *)x,
                           (const T *)res, gamma, beta, (T *)y, rows, cols, eps, out_q, q_inv, emb);
    } else {
        hipLaunchKernelGGL((layernorm_long_kernel<DT>), grid, block, 0, s, (const T *)x, (const T *)res, gamma, beta,
                           (T *)y, rows, cols, eps, out_q, q_inv);
    }
    TR_CHECK_LAUNCH();
    return 0;
}

// ---- Softmax ------------------------------------------------------------------------------------
constexpr int kSmMaxPerLane = 16;  // last-axis rows up to 1024 values stay in registers

// inner == 1: one wave per row.
template <int DT>
__global__ void __launch_bounds__(kBlock) softmax_lastaxis_kernel(const typename Elem<DT>::type *__restrict__ x,
                                                                  typename Elem<DT>::type *__restrict__ y, int rows,
                                                                  int channel) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row  = blockIdx.x * kRowsPerBlk + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const typename Elem<DT>::type *px = x + (size_t)row * channel;
    typename Elem<DT>::type *py       = y + (size_t)row * channel;
    if (channel <= kWave * kSmMaxPerLane) {
        float v[kSmMaxPerLane];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < kSmMaxPerLane; ++j) {
            int c = lane + j * kWave;
            v[j]  = c < channel ? Elem<DT>::ld(&px[c]) : -INFINITY;
            mx    = fmaxf(mx, v[j]);
        }
        mx        = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < kSmMaxPerLane; ++j) {
            int c = lane + j * kWave;
            v[j]  = c < channel ? expf(v[j] - mx) : 0.f;
            sum += v[j];
        }
        sum       = wave_sum(sum);
        float inv = 1.0f / sum;
#pragma unroll
        for (int j = 0; j < kSmMaxPerLane; ++j) {
            int c = lane + j * kWave;
            if (c < channel)
                Elem<DT>::st(&py[c], v[j] * inv);
        }
    } else {
        float mx = -INFINITY;
        for (int c = lane; c < channel; c += kWave)
            mx = fmaxf(mx, Elem<DT>::ld(&px[c]));
        mx        = wave_max(mx);
        float sum = 0.f;
        for (int c = lane; c < channel; c += kWave)
            sum += expf(Elem<DT>::ld(&px[c]) - mx);
        sum       = wave_sum(sum);
        float inv = 1.0f / sum;
        for (int c = lane; c < channel; c += kWave)
            Elem<DT>::st(&py[c], expf(Elem<DT>::ld(&px[c]) - mx) * inv);
    }
}

// inner > 1: one lane per (outer, inner) column; consecutive lanes touch consecutive addresses.
template <int DT>
__global__ void __launch_bounds__(kBlock) softmax_strided_kernel(const typename Elem<DT>::type *__restrict__ x,
                                                                 typename Elem<DT>::type *__restrict__ y, int outer,
                                                                 int channel, int inner) {
    size_t total  = (size_t)outer * inner;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        size_t n = i / inner, e = i % inner;
        const typename Elem<DT>::type *px = x + n * channel * inner + e;
        typename Elem<DT>::type *py       = y + n * channel * inner + e;
        float mx                          = -INFINITY;
        for (int c = 0; c < channel; ++c)
            mx = fmaxf(mx, Elem<DT>::ld(&px[(size_t)c * inner]));
        float sum = 0.f;
        for (int c = 0; c < channel; ++c)
            sum += expf(Elem<DT>::ld(&px[(size_t)c * inner]) - mx);
        float inv = 1.0f / sum;
        for (int c = 0; c < channel; ++c)
            Elem<DT>::st(&py[(size_t)c * inner], expf(Elem<DT>::ld(&px[(size_t)c * inner]) - mx) * inv);
    }
}

template <int DT>
int launch_softmax(hipStream_t s, const void *x, void *y, int outer, int channel, int inner) {
    typedef typename Elem<DT>::type T;
    if (inner == 1) {
        dim3 grid((outer + kRowsPerBlk - 1) / kRowsPerBlk);
        hipLaunchKernelGGL((softmax_lastaxis_kernel<DT>), grid, dim3(kBlock), 0, s, (const T *)x, (T *)y, outer,
                           channel);
    } else {
        size_t total = (size_t)outer * inner;
        size_t g     = (total + kBlock - 1) / kBlock;
        if (g > 4096)
            g = 4096;
        hipLaunchKernelGGL((softmax_strided_kernel<DT>), dim3((unsigned)g), dim3(kBlock), 0, s, (const T *)x, (T *)y,
                           outer, channel, inner);
    }
    TR_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" {
TR_DEFINE_STORE_THROUGH_SETTER(rowwise_set_store_through)

int tnn_rocm_layernorm(void *stream, int dtype, const void *x, const void *residual, const float *gamma,
                       const float *beta, void *y, int rows, int cols, float eps, int8_t *out_q, float q_inv_scale) {
    TR_REQUIRE(rows >= 0 && cols >= 0, TNN_ROCM_ESHAPE, "layernorm: negative size");
    // the reference rejects an empty reduction (cpu_layer_norm_layer_acc.cc:87-90)
    TR_REQUIRE(rows > 0 && cols > 0, TNN_ROCM_ESHAPE, "layernorm: blob count is zero");
    TR_REQUIRE(x && y && gamma && beta, TNN_ROCM_EINVAL, "layernorm: null pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case TNN_ROCM_F32:
            return launch_layernorm<TNN_ROCM_F32>(s, x, residual, gamma, beta, y, rows, cols, eps, out_q, q_inv_scale);
        case TNN_ROCM_F16:
            return launch_layernorm<TNN_ROCM_F16>(s, x, residual, gamma, beta, y, rows, cols, eps, out_q, q_inv_scale);
        case TNN_ROCM_BF16:
            return launch_layernorm<TNN_ROCM_BF16>(s, x, residual, gamma, beta, y, rows, cols, eps, out_q,
                                                   q_inv_scale);
        default: set_error("layernorm: unsupported dtype %d", dtype); return TNN_ROCM_EDTYPE;
    }
}

static int embed_layernorm_impl(void *stream, int dtype, const int32_t *ids, const int32_t *type_ids, const void *word_table,
                                int vocab, const void *type_table, int n_types, const void *pos_table, int period,
                                const int32_t *pos_ids, int n_pos_ids, int pos_rows, const float *gamma, const float *beta,
                                float eps, void *y, int rows, int cols, int32_t *error_flag);

int tnn_rocm_embed_layernorm(void *stream, int dtype, const int32_t *ids, const int32_t *type_ids, const void *word_table,
                             int vocab, const void *type_table, int n_types, const void *pos_table, int period,
                             const float *gamma, const float *beta, float eps, void *y, int rows, int cols,
                             int32_t *error_flag) {
    return embed_layernorm_impl(stream, dtype, ids, type_ids, word_table, vocab, type_table, n_types, pos_table, period,
                                nullptr, 0, 0, gamma, beta, eps, y, rows, cols, error_flag);
}

int tnn_rocm_embed_layernorm_pos(void *stream, int dtype, const int32_t *ids, const int32_t *type_ids,
                                 const int32_t *pos_ids, int n_pos_ids, const void *word_table, int vocab,
                                 const void *type_table, int n_types, const void *pos_table, int pos_rows,
                                 const float *gamma, const float *beta, float eps, void *y, int rows, int cols,
                                 int32_t *error_flag) {
    TR_REQUIRE(pos_ids && n_pos_ids > 0 && pos_rows > 0, TNN_ROCM_EINVAL, "embed_layernorm_pos: position ids and table rows required");
    return embed_layernorm_impl(stream, dtype, ids, type_ids, word_table, vocab, type_table, n_types, pos_table, 1, pos_ids,
                                n_pos_ids, pos_rows, gamma, beta, eps, y, rows, cols, error_flag);
}

static int embed_layernorm_impl(void *stream, int dtype, const int32_t *ids, const int32_t *type_ids, const void *word_table,
                                int vocab, const void *type_table, int n_types, const void *pos_table, int period,
                                const int32_t *pos_ids, int n_pos_ids, int pos_rows, const float *gamma, const float *beta,
                                float eps, void *y, int rows, int cols, int32_t *error_flag) {
    TR_REQUIRE(rows >= 0 && cols > 0 && vocab > 0 && n_types > 0 && period > 0, TNN_ROCM_ESHAPE,
               "embed_layernorm: sizes must be positive");
    if (rows == 0)
        return 0;
    TR_REQUIRE(ids && type_ids && word_table && type_table && pos_table && gamma && beta && y, TNN_ROCM_EINVAL,
               "embed_layernorm: null pointer");
    EmbedRows emb;
    emb.pos_ids   = pos_ids;
    emb.n_pos_ids = n_pos_ids;
    emb.pos_rows  = pos_rows;
    emb.ids        = ids;
    emb.type_ids   = type_ids;
    emb.type_table = type_table;
    emb.vocab      = vocab;
    emb.n_types    = n_types;
    emb.period     = period;
    emb.error_flag = error_flag;
    hipStream_t s  = (hipStream_t)stream;
    switch (dtype) {
        case TNN_ROCM_F32:
            return launch_layernorm<TNN_ROCM_F32>(s, word_table, pos_table, gamma, beta, y, rows, cols, eps, nullptr, 0.f, emb);
        case TNN_ROCM_F16:
            return launch_layernorm<TNN_ROCM_F16>(s, word_table, pos_table, gamma, beta, y, rows, cols, eps, nullptr, 0.f, emb);
        case TNN_ROCM_BF16:
            return launch_layernorm<TNN_ROCM_BF16>(s, word_table, pos_table, gamma, beta, y, rows, cols, eps, nullptr, 0.f, emb);
        default: set_error("embed_layernorm: unsupported dtype %d", dtype); return TNN_ROCM_EDTYPE;
    }
}

int tnn_rocm_softmax(void *stream, int dtype, const void *x, void *y, int outer, int channel, int inner) {
    TR_REQUIRE(outer >= 0 && channel >= 0 && inner >= 0, TNN_ROCM_ESHAPE, "softmax: negative size");
    if (outer == 0 || channel == 0 || inner == 0)
        return 0;
    TR_REQUIRE(x && y, TNN_ROCM_EINVAL, "softmax: null pointer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case TNN_ROCM_F32: return launch_softmax<TNN_ROCM_F32>(s, x, y, outer, channel, inner);
        case TNN_ROCM_F16: return launch_softmax<TNN_ROCM_F16>(s, x, y, outer, channel, inner);
        case TNN_ROCM_BF16: return launch_softmax<TNN_ROCM_BF16>(s, x, y, outer, channel, inner);
        default: set_error("softmax: unsupported dtype %d", dtype); return TNN_ROCM_EDTYPE;
    }
}

}  // extern "C"
