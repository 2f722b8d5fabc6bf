/*
 * CPU restatement of the reference engine's transformer-encoder ops (plain C).
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP kernels are compared
 * against; nothing in the shipped library may call, link or fall back to it.
 *
 * Every function follows the arithmetic (operand order, accumulator type, rounding) of the
 * reference function cited above it.  Paths are relative to the reference tree's source/tnn/.
 * Floating point is compiled with -ffp-contract=off and without fast-math, matching how the
 * reference builds its DEVICE_NAIVE objects (no -mfma, no -ffast-math).
 *
 * OpenMP is only used across independent output rows, so per-element results do not depend
 * on the thread count.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------------------------------------
 * MatMul   device/cpu/acc/cpu_mat_mul_layer_acc.cc:87-113
 * c[bc][m][k] = float( sum_n double(a[ba][m][n]) * double(b[bb][n][k]) ),  ba = bc % batch_a,
 * bb = bc % batch_b.  The sum runs n = 0..N-1 in order, in double.
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_matmul_f32(const float *a, const float *b, float *c, int M, int N, int K, int batch_a, int batch_b,
                            int batch_c) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int bc = 0; bc < batch_c; ++bc) {
        for (int m = 0; m < M; ++m) {
            const float *pa = a + (size_t)(bc % batch_a) * M * N + (size_t)m * N;
            const float *pb = b + (size_t)(bc % batch_b) * N * K;
            float *pc       = c + (size_t)bc * M * K + (size_t)m * K;
            for (int k = 0; k < K; ++k) {
                double sum = 0;
                for (int n = 0; n < N; ++n) {
                    sum += (double)pa[n] * (double)pb[(size_t)n * K + k];
                }
                pc[k] = (float)sum;
            }
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * InnerProduct fp32   utils/naive_compute.cc:271-288 (NaiveFC<float>)
 * y[r][oc] = (float acc: sum_ic w[oc][ic]*x[r][ic], ic ascending) + bias[oc]
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_inner_product_f32(const float *x, const float *w, const float *bias, float *y, int rows, int K,
                                   int N) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int r = 0; r < rows; ++r) {
        for (int oc = 0; oc < N; ++oc) {
            const float *px = x + (size_t)r * K;
            const float *pw = w + (size_t)oc * K;
            float acc       = 0;
            for (int ic = 0; ic < K; ++ic) {
                acc += pw[ic] * px[ic];
            }
            if (bias)
                acc += bias[oc];
            y[(size_t)r * N + oc] = acc;
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * Softmax   device/cpu/acc/cpu_softmax_layer_acc.cc:46-93
 * x viewed as [outer][channel][inner]; per (outer, inner): max over channel, expf(x-max),
 * float sum in channel order, then multiply by (1.0f / sum).
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_softmax_f32(const float *x, float *y, int outer, int channel, int inner) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < outer; ++n) {
        const float *xb = x + (size_t)n * channel * inner;
        float *yb       = y + (size_t)n * channel * inner;
        for (int e = 0; e < inner; ++e) {
            float mx = xb[e];
            for (int c = 1; c < channel; ++c) {
                float v = xb[(size_t)c * inner + e];
                mx      = mx > v ? mx : v; /* std::max(temp, v) */
            }
            for (int c = 0; c < channel; ++c) {
                yb[(size_t)c * inner + e] = expf(xb[(size_t)c * inner + e] - mx);
            }
            float sum = yb[e];
            for (int c = 1; c < channel; ++c) {
                sum += yb[(size_t)c * inner + e];
            }
            float inv = 1.0f / sum;
            for (int c = 0; c < channel; ++c) {
                yb[(size_t)c * inner + e] *= inv;
            }
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * LayerNorm   device/cpu/acc/cpu_layer_norm_layer_acc.cc:105-133
 * double sum_x, sum_x2 (the square itself is a float product), var = E[x^2]-E[x]^2,
 * rstd = 1.0f / sqrt(var + eps) evaluated in double, bias' = float(beta - mean*rstd*k),
 * y = float(x * rstd * k + bias').
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_layernorm_f32(const float *x, const float *gamma, const float *beta, float *y, int rows, int cols,
                               float eps) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        const float *px = x + (size_t)r * cols;
        float *py       = y + (size_t)r * cols;
        double sum_x = 0, sum_x2 = 0;
        for (int i = 0; i < cols; ++i) {
            float t = px[i];
            sum_x += t;
            sum_x2 += t * t;
        }
        double mean_x   = sum_x / cols;
        double mean_x2  = sum_x2 / cols;
        double variance = mean_x2 - mean_x * mean_x;
        variance        = 1.0f / sqrt(variance + eps);
        for (int i = 0; i < cols; ++i) {
            float k    = gamma[i];
            float bias = beta[i];
            bias -= mean_x * variance * k; /* float -= double: computed in double, rounded to float */
            py[i] = (float)(px[i] * variance * k + bias);
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * GELU   device/cpu/acc/cpu_gelu_layer_acc.cc:42-45 ;  erf-based, never the tanh form.
 * The source reads 0.5f * x * (erf(x*0.707106793288165f) + 1.0f) with only <cmath> included, so the
 * unqualified erf resolves to the C library's double erf(double): the argument product and 0.5f*x
 * are fp32, erf and the final product are double, and the store rounds to fp32.  (Checked against
 * the compiled reference: this form is bit-identical, the erff form differs in the last ulp.)
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_gelu_f32(const float *x, float *y, size_t count) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; ++i) {
        float v  = x[i];
        float hv = 0.5f * v;
        double e = erf((double)(v * 0.707106793288165f)) + 1.0f;
        y[i]     = (float)(hv * e);
    }
}

/* ---------------------------------------------------------------------------------------------
 * Add / Sub / Mul / Div with numpy-style broadcast
 *   device/cpu/acc/compute/compute_elewise.cc:37-65 (CPU_ELEWISE)
 * shapes are right-aligned to the output rank; an input index is min(out_index, dim-1).
 * op: 0 add, 1 sub, 2 mul, 3 div.
 * ------------------------------------------------------------------------------------------- */
static size_t orc_bcast_offset(const int *out_index, int out_rank, const int *shape, int rank) {
    int diff   = out_rank - rank;
    size_t off = 0;
    for (int i = 0; i < rank; ++i) {
        int idx = out_index[i + diff];
        if (idx > shape[i] - 1)
            idx = shape[i] - 1;
        off = off * (size_t)shape[i] + (size_t)idx;
    }
    return off;
}

ORC_API void orc_binary_f32(int op, const float *a, const int *shape_a, int rank_a, const float *b, const int *shape_b,
                            int rank_b, float *out, const int *shape_out, int rank_out) {
    size_t count = 1;
    for (int i = 0; i < rank_out; ++i)
        count *= (size_t)shape_out[i];
#pragma omp parallel for schedule(static)
    for (size_t offset = 0; offset < count; ++offset) {
        int index[8];
        size_t rem = offset;
        for (int i = rank_out - 1; i >= 0; --i) {
            index[i] = (int)(rem % (size_t)shape_out[i]);
            rem /= (size_t)shape_out[i];
        }
        float va = a[orc_bcast_offset(index, rank_out, shape_a, rank_a)];
        float vb = b[orc_bcast_offset(index, rank_out, shape_b, rank_b)];
        float r;
        switch (op) {
            case 0: r = va + vb; break;
            case 1: r = va - vb; break;
            case 2: r = va * vb; break;
            default: r = va / vb; break;
        }
        out[offset] = r;
    }
}

/* ---------------------------------------------------------------------------------------------
 * Permute   utils/naive_compute.cc:943-956 (NaivePermute): out dims[j] = in dims[order[j]].
 * elem_size in bytes (1, 2 or 4).
 * ------------------------------------------------------------------------------------------- */
ORC_API void orc_permute(const void *in, void *out, const int *in_dims, const int *order, int rank, int elem_size) {
    size_t old_steps[8], count = 1;
    int out_dims[8];
    for (int i = rank - 1; i >= 0; --i) {
        old_steps[i] = count;
        count *= (size_t)in_dims[i];
    }
    for (int j = 0; j < rank; ++j)
        out_dims[j] = in_dims[order[j]];
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; ++i) {
        size_t old_idx = 0, idx = i;
        for (int j = rank - 1; j >= 0; --j) {
            old_idx += (idx % (size_t)out_dims[j]) * old_steps[order[j]];
            idx /= (size_t)out_dims[j];
        }
        memcpy((char *)out + i * elem_size, (const char *)in + old_idx * elem_size, (size_t)elem_size);
    }
}

/* ---------------------------------------------------------------------------------------------
 * Gather   device/cpu/acc/cpu_gather_layer_acc.cc:56-85
 * data viewed as [batch][slices][slice_bytes]; negative indices wrap once; returns -1 on an
 * out-of-range index (the reference returns TNNERR_MODEL_ERR).
 * ------------------------------------------------------------------------------------------- */
ORC_API int orc_gather(const void *data, const int *indices, void *out, int batch, int slices, size_t slice_bytes,
                       int n_indices) {
    for (int b = 0; b < batch; ++b) {
        for (int i = 0; i < n_indices; ++i) {
            int s = indices[i];
            if (s < 0)
                s += slices;
            if (s < 0 || s >= slices)
                return -1;
            memcpy((char *)out + ((size_t)b * n_indices + i) * slice_bytes,
                   (const char *)data + ((size_t)b * slices + s) * slice_bytes, slice_bytes);
        }
    }
    return 0;
}

/* =============================================================================================
 * int8 path
 * ===========================================================================================*/

/* utils/naive_compute.cc:32-34 : round half away from zero by adding +-0.5f in float, clamp in
 * float, truncate. */
ORC_API int8_t orc_float2int8(float val) {
    float t = val + (val >= 0.f ? 0.5f : -0.5f);
    t       = t < 127.0f ? t : 127.0f;   /* MIN(t, 127) */
    t       = t > -128.0f ? t : -128.0f; /* MAX(., -128) */
    return (int8_t)t;
}

ORC_API void orc_float2int8_array(const float *v, int8_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i)
        out[i] = orc_float2int8(v[i]);
}

/* Requantisation factor prepared on the host at Init:
 *   device/cpu/acc/cpu_inner_product_layer_acc.cc:66-73 and
 *   device/x86/acc/x86_inner_product_layer_acc.cc:212-220
 * scale[oc] = w_scale[oc or 0] / o_scale[oc or 0] as one fp32 division, 0 when o_scale < FLT_MIN. */
ORC_API void orc_fc_int8_scale(const float *w_scale, int n_w, const float *o_scale, int n_o, float *scale, int N) {
    for (int i = 0; i < N; ++i) {
        float ws = w_scale[n_w == 1 ? 0 : i];
        float os = o_scale[n_o == 1 ? 0 : i];
        scale[i] = (os >= FLT_MIN) ? ws / os : 0.0f;
    }
}

/* Quantized InnerProduct with zero zero-points
 *   utils/naive_compute.cc:316-347 (NaiveFCBias) == device/x86/acc/compute/x86_compute_int8.cc:833-914
 * acc = sum int32(x*w) (+ bias) exactly; y = float2int8( (float)acc * scale[oc] ).
 * acc_out (optional) receives the int32 accumulator including bias. */
ORC_API void orc_fc_int8(const int8_t *x, const int8_t *w, const int32_t *bias, const float *scale, int8_t *y,
                         int32_t *acc_out, int rows, int K, int N) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int r = 0; r < rows; ++r) {
        for (int oc = 0; oc < N; ++oc) {
            const int8_t *px = x + (size_t)r * K;
            const int8_t *pw = w + (size_t)oc * K;
            int32_t acc      = 0;
            for (int ic = 0; ic < K; ++ic) {
                acc += (int32_t)pw[ic] * (int32_t)px[ic];
            }
            if (bias)
                acc += bias[oc];
            if (acc_out)
                acc_out[(size_t)r * N + oc] = acc;
            float f               = (float)acc * scale[oc];
            y[(size_t)r * N + oc] = orc_float2int8(f);
        }
    }
}

/* Quantize, DEVICE_X86 form: multiply by the reciprocal prepared as float(1.0 / scale)
 *   device/x86/acc/x86_reformat_layer_acc.cc:66-75, compute/x86_compute_int8.cc:1254-1318 */
ORC_API void orc_quantize_x86(const float *x, float scale, int8_t *q, size_t n) {
    float inv = (float)(1.0 / scale);
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
        q[i] = orc_float2int8(x[i] * inv);
}

/* Quantize, DEVICE_NAIVE form: divide by the scale    utils/naive_compute.cc:1674-1690 */
ORC_API void orc_quantize_naive(const float *x, float scale, int8_t *q, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
        q[i] = (scale != 0) ? orc_float2int8(x[i] / scale + 0.0f) : 0;
}

/* Dequantize: x = (float)q * scale     compute/x86_compute_int8.cc:1193-1252 (naive: scale*(q-0)) */
ORC_API void orc_dequantize(const int8_t *q, float scale, float *x, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
        x[i] = (float)q[i] * scale;
}

/* int8 residual add, DEVICE_X86 form
 *   device/x86/acc/x86_add_layer_acc.cc:54-58 (dst scale = 1.0 / so), compute/x86_compute_int8.cc:795-831
 * The source reads float2int8( (a*sa + b*sb) * inv_so ).  Its translation unit is built with -mavx2 -mfma
 * -ffast-math (device/x86/CMakeLists.txt:1-27), and g++ contracts one product into the sum.  Which one was
 * established against the compiled reference over all 65536 (a, b) pairs on a tie-heavy scale triple
 * (tests/test_oracle_vs_reference.py): the 8-channel vector body computes fma(b, sb, a*sa), the scalar tail (the last
 * four channels when round_up(channels, 4) % 8 == 4) computes fma(a, sa, b*sb); the un-contracted form differs from
 * either in thousands of those pairs.  `channels` = dims[1], `inner` = count(dims[2:]), element i of the plain
 * row-major array sits in channel (i / inner) % channels.
 * The x86 acc walks only the first batch entry (dims[0] is never read, :86-87: round_up(dims[1], 4) channels times
 * count(dims, 2) positions) and leaves the rest of its output unwritten; this restatement computes every entry. */
ORC_API void orc_add_int8_x86(const int8_t *a, float sa, const int8_t *b, float sb, float so, int8_t *y, size_t n,
                              int channels, size_t inner) {
    float inv     = (float)(1.0 / so);
    int c4        = (channels + 3) / 4 * 4;
    int vec_end   = c4 - ((c4 % 8 == 4) ? 4 : 0);
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        int c = (int)((i / inner) % (size_t)channels);
        float s;
        if (c < vec_end) {
            float pa = (float)a[i] * sa;
            s        = fmaf((float)b[i], sb, pa);
        } else {
            float pb = (float)b[i] * sb;
            s        = fmaf((float)a[i], sa, pb);
        }
        y[i] = orc_float2int8(s * inv);
    }
}

/* int8 residual add, DEVICE_NAIVE form
 *   device/cpu/acc/cpu_add_layer_acc.cc:31-47, compute/compute_int8.cc:54-84 (zero points are 0 on this path)
 * y = float2int8( (sa*a + sb*b) / so + 0.0f ): a division where the x86 form multiplies by float(1.0/so). */
ORC_API void orc_add_int8_naive(const int8_t *a, float sa, const int8_t *b, float sb, float so, int8_t *y, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        float acc = sa * ((float)a[i] - 0.0f);
        acc       = acc + sb * ((float)b[i] - 0.0f);
        y[i]      = orc_float2int8(acc / so + 0.0f);
    }
}

/* =============================================================================================
 * Composite: the decomposed attention core as the reference graph computes it
 *   MatMul(Q, K^T) -> Mul(scale) -> Add(mask) -> Softmax(axis=-1) -> MatMul(P, V)
 * q,k,v,out: [B][h][S][d] fp32; mask: additive [B][S] (broadcast over heads and query rows) or
 * NULL.  Intermediates are fp32 blobs exactly as in the reference (scores rounded to float after
 * the double-accumulated MatMul).
 * ===========================================================================================*/
ORC_API int orc_attention_core_f32(const float *q, const float *k, const float *v, const float *mask, float *out,
                                   int B, int h, int S, int d, float scale) {
    int nb = B * h;
#pragma omp parallel for schedule(dynamic)
    for (int bh = 0; bh < nb; ++bh) {
        float *scores = (float *)malloc(sizeof(float) * (size_t)S * S);
        float *kt     = (float *)malloc(sizeof(float) * (size_t)S * d);
        const float *pq = q + (size_t)bh * S * d;
        const float *pk = k + (size_t)bh * S * d;
        const float *pv = v + (size_t)bh * S * d;
        float *po       = out + (size_t)bh * S * d;
        const float *pm = mask ? mask + (size_t)(bh / h) * S : NULL;
        /* Permute K -> K^T [d][S] (a separate Permute layer in the graph) */
        for (int j = 0; j < S; ++j)
            for (int e = 0; e < d; ++e)
                kt[(size_t)e * S + j] = pk[(size_t)j * d + e];
        for (int i = 0; i < S; ++i) {
            float *row = scores + (size_t)i * S;
            for (int j = 0; j < S; ++j) {
                double sum = 0;
                for (int e = 0; e < d; ++e)
                    sum += (double)pq[(size_t)i * d + e] * (double)kt[(size_t)e * S + j];
                float s = (float)sum;
                s       = s * scale;
                if (pm)
                    s = s + pm[j];
                row[j] = s;
            }
            float mx = row[0];
            for (int j = 1; j < S; ++j)
                mx = mx > row[j] ? mx : row[j];
            for (int j = 0; j < S; ++j)
                row[j] = expf(row[j] - mx);
            float sum = row[0];
            for (int j = 1; j < S; ++j)
                sum += row[j];
            float inv = 1.0f / sum;
            for (int j = 0; j < S; ++j)
                row[j] *= inv;
            for (int e = 0; e < d; ++e) {
                double acc = 0;
                for (int j = 0; j < S; ++j)
                    acc += (double)row[j] * (double)pv[(size_t)j * d + e];
                po[(size_t)i * d + e] = (float)acc;
            }
        }
        free(scores);
        free(kt);
    }
    return 0;
}
