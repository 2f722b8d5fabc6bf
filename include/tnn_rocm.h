/*
 * tnn_rocm.h — C ABI of the MI355X (gfx950) kernels behind the DEVICE_ROCM backend.
 *
 * This is the only interface between the g++-compiled host code (the layer accelerators that
 * implement the engine's AbstractDevice / Context / AbstractLayerAcc contract) and the
 * hipcc-compiled kernels.  Signatures use plain pointers and sizes only.
 *
 * Conventions
 *   - every function returns 0 on success, a positive hipError_t value when a HIP call failed,
 *     or a negative TNN_ROCM_E* code for a rejected argument; tnn_rocm_last_error() returns a
 *     message for the most recent failure on the calling thread.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Work is only
 *     enqueued; nothing synchronises unless the name says so.
 *   - all data pointers are device pointers unless the parameter name starts with `host_`.
 *   - `dtype` uses the engine's DataType numbering (include/tnn/core/common.h:51-66 of the
 *     reference): 0 float32, 1 float16, 2 int8, 3 int32, 4 bfloat16.
 *   - matrices are row-major; "rows" are tokens (T = batch * sequence).
 *
 * Each entry point names the reference function whose result it reproduces (paths relative to
 * the reference tree).
 */
#ifndef TNN_ROCM_H_
#define TNN_ROCM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TNN_ROCM_API __attribute__((visibility("default")))

enum {
    TNN_ROCM_F32  = 0,
    TNN_ROCM_F16  = 1,
    TNN_ROCM_I8   = 2,
    TNN_ROCM_I32  = 3,
    TNN_ROCM_BF16 = 4
};

enum {
    TNN_ROCM_EINVAL   = -1, /* bad argument (null pointer, negative size, unknown enum)            */
    TNN_ROCM_ESHAPE   = -2, /* shape the kernel family does not implement                          */
    TNN_ROCM_EDTYPE   = -3, /* dtype the entry point does not implement                            */
    TNN_ROCM_EALIGN   = -4, /* pointer or leading dimension not aligned as documented              */
    TNN_ROCM_ENODEV   = -5  /* no gfx950 device visible                                            */
};

/* ---- runtime: what AbstractDevice / Context need -------------------------------------------
 * replaces source/tnn/device/cuda/cuda_device.cc:53-137 (Allocate/Free/CopyTo/FromDevice) and
 * source/tnn/device/cuda/cuda_context.cc:47-154 (stream create / synchronize) in role. */
TNN_ROCM_API const char *tnn_rocm_last_error(void);
TNN_ROCM_API int tnn_rocm_device_count(int *count);
TNN_ROCM_API int tnn_rocm_set_device(int device_id);
TNN_ROCM_API int tnn_rocm_device_name(int device_id, char *buf, size_t buf_len);
TNN_ROCM_API int tnn_rocm_malloc(void **ptr, size_t bytes);
TNN_ROCM_API int tnn_rocm_free(void *ptr);
/* page-locked host memory that kernels can also write (used for the context's error word, which the
 * host reads after a stream synchronise instead of issuing a device-to-host copy per forward) */
TNN_ROCM_API int tnn_rocm_malloc_host(void **host_ptr, size_t bytes);
TNN_ROCM_API int tnn_rocm_free_host(void *host_ptr);
TNN_ROCM_API int tnn_rocm_memset(void *ptr, int value, size_t bytes, void *stream);
TNN_ROCM_API int tnn_rocm_memcpy_h2d(void *dst, const void *host_src, size_t bytes, void *stream);
TNN_ROCM_API int tnn_rocm_memcpy_d2h(void *host_dst, const void *src, size_t bytes, void *stream);
TNN_ROCM_API int tnn_rocm_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
TNN_ROCM_API int tnn_rocm_stream_create(void **stream);
TNN_ROCM_API int tnn_rocm_stream_destroy(void *stream);
TNN_ROCM_API int tnn_rocm_stream_sync(void *stream);
/* hipEvent timing on a stream, for the profiler hook of Context (source/tnn/core/context.cc:84-100) */
TNN_ROCM_API int tnn_rocm_event_create(void **event);
TNN_ROCM_API int tnn_rocm_event_destroy(void *event);
TNN_ROCM_API int tnn_rocm_event_record(void *event, void *stream);
TNN_ROCM_API int tnn_rocm_event_elapsed_ms(void *start, void *stop, float *ms); /* synchronises on `stop` */

/* Stream capture into an executable graph, used by the network to replay a whole forward pass (about ninety
 * launches for a 12-layer encoder) with one submission.  Only kernel launches may be issued on the stream between
 * begin and end (no allocation, synchronisation or memset). */
TNN_ROCM_API int tnn_rocm_graph_begin_capture(void *stream);
TNN_ROCM_API int tnn_rocm_graph_end_capture(void *stream, void **graph_exec);
TNN_ROCM_API int tnn_rocm_graph_launch(void *graph_exec, void *stream);
TNN_ROCM_API int tnn_rocm_graph_destroy(void *graph_exec);

/* ---- dense contractions --------------------------------------------------------------------
 * GEMM epilogue selectors (combinable): y = act(acc + bias) + residual                       */
enum {
    TNN_ROCM_EPI_NONE     = 0,
    TNN_ROCM_EPI_BIAS     = 1, /* + bias[N] (fp32 vector)                                     */
    TNN_ROCM_EPI_GELU     = 2, /* erf GELU: 0.5*x*(erf(x*0.70710679)+1)  (cpu_gelu_layer_acc.cc:42-45) */
    TNN_ROCM_EPI_RESIDUAL = 4  /* + residual[M,N] (same dtype as C)                            */
};

/* C[batch][M,N] = A[batch][M,K] * op(B) with fp32 accumulation.
 *   b_is_nk = 1: B is [N,K] row-major (InnerProduct weight layout; y = x * W^T):
 *       NaiveFC                      source/tnn/utils/naive_compute.cc:271-288
 *       X86InnerProductLayerAcc      source/tnn/device/x86/acc/x86_inner_product_layer_acc.cc:226-273
 *   b_is_nk = 0: B is [K,N] row-major (MatMul layout):
 *       CpuMatMulLayerAcc::Forward   source/tnn/device/cpu/acc/cpu_mat_mul_layer_acc.cc:64-117
 *       X86MatMulLayerAcc::DoForward source/tnn/device/x86/acc/x86_mat_mul_layer_acc.cc:49-114
 * Batches: `batch` output matrices; A uses matrix (i % batch_a), B uses (i % batch_b) — the
 * reference's broadcast rule (cpu_mat_mul_layer_acc.cc:99-100).
 * dtype: F32, F16 or BF16 for A, B, C and residual; bias is always fp32.
 * lda/ldb/ldc are row strides in elements. */
TNN_ROCM_API int tnn_rocm_gemm(void *stream, int dtype, int b_is_nk, const void *A, const void *B, void *C, int M,
                               int N, int K, int lda, int ldb, int ldc, int batch, int batch_a, int batch_b,
                               int epilogue, const float *bias, const void *residual, int ldr);

/* int8 x int8 -> int32 GEMM with the reference requantisation fused:
 *   acc[m][n] = sum_k A[m][k]*W[n][k] (+ bias_i32[n]);  out = float2int8((float)acc * scale[n])
 *       NaiveFCBias   source/tnn/utils/naive_compute.cc:316-347   (zero zero-points)
 *       X86GemvInt8   source/tnn/device/x86/acc/compute/x86_compute_int8.cc:833-914
 *       float2int8    source/tnn/utils/naive_compute.cc:32-34
 * scale[n] is the host-prepared w_scale[n]/o_scale (x86_inner_product_layer_acc.cc:212-220).
 * out_i8 and/or acc_i32 may be NULL (acc_i32 exposes the exact accumulators for parity tests).
 * Optional fused dequantisation for a float consumer: if out_f (dtype out_f_dtype F32/F16) is
 * non-NULL it receives (float)q * dequant_scale, the value a following Reformat layer would
 * produce (x86_compute_int8.cc:1193-1252). */
TNN_ROCM_API int tnn_rocm_gemm_i8(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias,
                                  const float *scale, int8_t *out_i8, int32_t *acc_i32, int M, int N, int K, int lda,
                                  int ldw, int ldo, void *out_f, int out_f_dtype, float dequant_scale);

/* ---- fused attention core -------------------------------------------------------------------
 * out = softmax(Q K^T * scale + mask) V per (batch, head): the sub-graph
 *   MatMul -> Mul/Div -> Add(mask) -> Softmax(axis=-1) -> MatMul
 * of cpu_mat_mul_layer_acc.cc:64-117, compute_elewise.cc:37-65, cpu_softmax_layer_acc.cc:30-97,
 * without materialising the [B*h,S,S] scores.  fp32 accumulation, online softmax.
 * Element (b, head, s, e) of Q is at q[b*q_sb + head*q_sh + s*q_ss + e] (e contiguous); same for
 * K, V (kv strides) and out.  head_dim must be 64.  dtype F16 or BF16.
 *   mask   : optional additive fp32 [B, S] (broadcast over heads and query rows), e.g. 0 / -10000
 *   kv_len : optional int32 [B]; keys j >= kv_len[b] are excluded exactly (−inf) and their tiles
 *            skipped.  kv_len[b] = 0 (the mask routines below never produce it: a row that masks every key keeps all
 *            of them, as the reference's softmax does) writes the sequence's output rows as zeros.
 *            (bit 30 of an entry may be set by tnn_rocm_mask_to_kv_len_flagged: mask row b is then not read). */
TNN_ROCM_API int tnn_rocm_attention(void *stream, int dtype, const void *q, const void *k, const void *v, void *out,
                                    int B, int heads, int S, int head_dim, long q_sb, long q_sh, long q_ss, long kv_sb,
                                    long kv_sh, long kv_ss, long o_sb, long o_sh, long o_ss, float scale,
                                    const float *mask, const int32_t *kv_len);

/* Same computation with V supplied transposed per head, V^T[b][head][d][s] (element at
 * vt[b*vt_sb + head*vt_sh + d*vt_sd + s], s contiguous, S a multiple of 8): the layout tnn_rocm_gemm_qkv_split
 * writes, which lets the kernel stage V tiles with 16-byte copies instead of transposing them.
 * Precision: this form multiplies Q by scale * log2(e) in the half type before the score product (so that the scores
 * leave the matrix pipe ready for exp2).  That second rounding of Q moves a score s by about |s| * 2^-11 / sqrt(head_dim) in
 * the exponent: nothing next to the blob type's own rounding while |s * scale| stays below ~20, as encoder
 * activations do, and up to 1e-2 of the output range once |s * scale| reaches ~70 (a softmax that is one-hot anyway). */
TNN_ROCM_API int tnn_rocm_attention_vt(void *stream, int dtype, const void *q, const void *k, const void *vt, void *out,
                                       int B, int heads, int S, int head_dim, long q_sb, long q_sh, long q_ss,
                                       long k_sb, long k_sh, long k_ss, long vt_sb, long vt_sh, long vt_sd, long o_sb,
                                       long o_sh, long o_ss, float scale, const float *mask, const int32_t *kv_len);

/* tnn_rocm_attention_vt that also writes the output quantised to int8 (out_q, same element strides as out; NULL = not
 * wanted): q = float2int8(out * out_q_inv_scale) on the values as stored in out, i.e. the Reformat(float -> int8) layer
 * that follows the attention block of a quantised net (x86_reformat_layer_acc / naive float2int8: multiply by
 * 1/scale, round half away from zero, saturate), in the same launch. */
TNN_ROCM_API int tnn_rocm_attention_vt_q8(void *stream, int dtype, const void *q, const void *k, const void *vt, void *out,
                                          int8_t *out_q, float out_q_inv_scale, int B, int heads, int S, int head_dim,
                                          long q_sb, long q_sh, long q_ss, long k_sb, long k_sh, long k_ss, long vt_sb,
                                          long vt_sh, long vt_sd, long o_sb, long o_sh, long o_ss, float scale,
                                          const float *mask, const int32_t *kv_len, int vt_key_order);

/* The int8 GEMM above with a float consumer folded in: out_f = (float)q * dequant_scale (+ residual), where q is
 * the requantised int8 value of tnn_rocm_gemm_i8 (never written).  This is QuantizedInnerProduct -> Reformat
 * (int8 -> float, x86_compute_int8.cc:1193-1252) -> Add(residual) (compute_elewise.cc:37-65) in one launch; the
 * product and the sum are rounded separately in fp32 as in that chain.  residual (NULL or dtype out_f_dtype, leading
 * dimension ldo) has the output's shape. */
TNN_ROCM_API int tnn_rocm_gemm_i8_dequant_residual(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias,
                                                   const float *scale, int M, int N, int K, int lda, int ldw,
                                                   void *out_f, int out_f_dtype, int ldo, float dequant_scale,
                                                   const void *residual);

/* tnn_rocm_gemm_i8 whose int8 result is passed through a 256-entry table on the way out: out = lut[q + 128].  Any
 * int8 -> int8 layer chain that followed the projection can be folded this way, value for value; the host uses it for
 * QuantizedInnerProduct -> Reformat -> GELU -> Reformat with the table produced by tnn_rocm_gelu_i8 on the 256 inputs
 * (cpu_gelu_layer_acc.cc:42-45 between the two x86 Reformat forms). */
TNN_ROCM_API int tnn_rocm_gemm_i8_lut(void *stream, const int8_t *A, const int8_t *W, const int32_t *bias,
                                      const float *scale, int8_t *out_i8, int M, int N, int K, int lda, int ldw, int ldo,
                                      const int8_t *lut);

/* Quantised Q, K, V projections of one attention layer as a single int8 GEMM over the concatenated weights
 * wqkv[3H,K] (three QuantizedInnerProduct layers reading the same int8 input): scale[n] = w_scale[n] / o_scale of the
 * column's projection, dequant[n] = that projection's output blob scale.  Each column is requantised to int8 as in
 * tnn_rocm_gemm_i8 and written dequantised (the three Reformat layers) in the layout of tnn_rocm_gemm_qkv_split:
 * Q | K row-major in qk[T,2H], V transposed per head in vt[B][heads][64][S].  out_dtype F16 or BF16. */
TNN_ROCM_API int tnn_rocm_gemm_i8_qkv_split(void *stream, int out_dtype, const int8_t *x, const int8_t *wqkv,
                                            const int32_t *bias, const float *scale, const float *dequant, void *qk,
                                            void *vt, int B, int S, int heads, int K, int vt_key_order);

/* Fused QKV projection for the attention layer: [T,K] x Wqkv[3H,K]^T + bqkv with the result split on the way out:
 * Q and K go to qk[T, 2H] (row-major, Q | K column blocks), V goes transposed per head to
 * vt[B][heads][64][S] (T = B*S tokens, H = heads*64).  Same arithmetic as three MatMul+Add pairs
 * (cpu_mat_mul_layer_acc.cc:64-117, compute_elewise.cc:37-65) followed by the head-split Permutes
 * (naive_compute.cc:943-956).  dtype F16 or BF16; K and H multiples of 64. */
/* V^T key order (vt_key_order of the three QKV-split projections and of tnn_rocm_attention_vt_q8; no counterpart in the
 * reference, whose Permute layers this layout replaces).  0: row d of a head holds its S keys in natural order.  1: inside
 * every group of 16 keys the blocks k4-7 and k8-11 have changed places ([k0-3 | k8-11 | k4-7 | k12-15]), the order in
 * which the attention kernel's lanes hold a score tile's probabilities, so that it needs no register exchange in front of
 * its second MFMA.  Needs S % 16 == 0; producer and consumer must agree.  tnn_rocm_attention_vt reads order 0. */
TNN_ROCM_API int tnn_rocm_gemm_qkv_split(void *stream, int dtype, const void *x, const void *wqkv, const float *bqkv,
                                         void *qk, void *vt, int B, int S, int heads, int K, int vt_key_order);

/* LayerNorm folded into the projection that reads it: y = LayerNorm(t) over the last axis of t[M,K]
 * (cpu_layer_norm_layer_acc.cc:86-135) followed by C = act(y W^T + b) (+ residual) (cpu_mat_mul_layer_acc.cc:64-117,
 * compute_elewise.cc:37-65, cpu_gelu_layer_acc.cc:42-45) as ONE GEMM on the raw t.  The caller prepares, once,
 *   w_folded[n,k] = gamma[k] * W[n,k] (in dtype),  colsum[n] = sum_k w_folded[n,k],  bias_folded[n] = b[n] + sum_k beta[k] W[n,k];
 * the kernel takes each row's mean and variance from the A tiles it streams anyway and forms
 *   y W^T + b = rstd * (t w_folded^T - mean * colsum) + bias_folded       on its fp32 accumulators.
 * y (optional, [M,K] in dtype) receives LayerNorm(t) itself for the other readers of that tensor (needs gamma, beta).
 * row_stats (optional, [M][2] fp32) receives {rstd, mean} of every row instead, for a reader that rebuilds
 * LayerNorm(t) from t on the fly (tnn_rocm_gemm_residual_ln).
 * row_sums (optional, [row_sum_blocks][M][2] fp32, as left by tnn_rocm_gemm_residual_ln when it wrote t): every row's
 * sum and sum of squares per block of columns of t; the kernel then adds those up instead of taking the statistics
 * from the A tiles.  At most TNN_ROCM_MAX_ROW_SUM_BLOCKS blocks.
 * flags: TNN_ROCM_EPI_GELU, TNN_ROCM_EPI_RESIDUAL (residual [M,N] in dtype).  dtype F16 or BF16; K a multiple of 128
 * (the whole normalised row is one GEMM row), N a multiple of 8; all tensors dense row-major.
 * Size limits of the three LayerNorm-folding entry points (TNN_ROCM_ESHAPE beyond them): rows and columns below 2^24,
 * M*K, N*K and M*N below 2^31 elements (their kernels address with 32-bit offsets). */
TNN_ROCM_API int tnn_rocm_gemm_ln(void *stream, int dtype, const void *t, const void *w_folded, const float *bias_folded,
                                  const float *colsum, const float *gamma, const float *beta, float eps, void *C, void *y,
                                  float *row_stats, const float *row_sums, int row_sum_blocks, int M, int N, int K,
                                  int flags, const void *residual);

/* tnn_rocm_gemm_qkv_split on LayerNorm(t), folded the same way (wqkv_folded, bqkv_folded, colsum over the 3H rows). */
TNN_ROCM_API int tnn_rocm_gemm_qkv_split_ln(void *stream, int dtype, const void *t, const void *wqkv_folded,
                                            const float *bqkv_folded, const float *colsum, const float *gamma,
                                            const float *beta, float eps, void *qk, void *vt, void *y,
                                            float *row_stats, const float *row_sums, int row_sum_blocks, int B,
                                            int S, int heads, int K, int vt_key_order);

/* C = act(x W^T + b) + LayerNorm(t), the residual Add of a transformer block whose residual operand is the output of
 * a LayerNorm layer (compute_elewise.cc:37-65 after cpu_layer_norm_layer_acc.cc:86-135), without that output ever
 * being stored: t[M,N] is the tensor the LayerNorm read, row_stats[M][2] = {rstd, mean} per row as left by
 * tnn_rocm_gemm_ln / tnn_rocm_gemm_qkv_split_ln on the same t, gamma / beta [N] the LayerNorm's scale and shift; each
 * value is formed as t * rstd * gamma + (beta - mean * rstd * gamma).  x[M,K], W[N,K], C[M,N] dense row-major in dtype
 * (F16 or BF16); K a multiple of 64, N a multiple of 8.  flags: TNN_ROCM_EPI_BIAS, TNN_ROCM_EPI_GELU.
 * row_sums (optional, room for TNN_ROCM_MAX_ROW_SUM_BLOCKS * M pairs of fp32) receives, per block of columns of C (one
 * block per tile column of the launch) and row, the sum and the sum of squares of the values stored, for a
 * LayerNorm-folding GEMM that reads C next; *row_sum_blocks receives the number of blocks written, 0 if none were
 * (N above 64 * TNN_ROCM_MAX_ROW_SUM_BLOCKS, or a tile shape with no room for them): the reader then takes the
 * statistics itself. */
#define TNN_ROCM_MAX_ROW_SUM_BLOCKS 24
TNN_ROCM_API int tnn_rocm_gemm_residual_ln(void *stream, int dtype, const void *x, const void *w, const float *bias,
                                           void *C, const void *t, const float *row_stats, const float *gamma,
                                           const float *beta, int M, int N, int K, int flags, float *row_sums,
                                           int *row_sum_blocks);

/* kv_len[b] = 1 + the last key index whose additive mask value is > (the row's largest value + threshold), threshold
 * being a large negative number (the host passes -1000): softmax(scores + mask) is unchanged by a constant added to a
 * whole row, so the cut is taken relative to the row's best key -- a key that far below it contributes
 * exp(threshold + score difference) = 0 in fp32.  A row that holds no value above the cut (only -inf / NaN) keeps all
 * S keys, as the reference's softmax over all S keys does; so does a row that masks every key with the same value. */
/* The _flagged form additionally sets bit 30 of kv_len[b] when mask[b][j] is exactly 0 for every j < kv_len[b] (a plain
 * padding mask): the attention kernels accept such entries and then do not read mask row b at all (the keys at and
 * beyond kv_len[b] are excluded by the length), which lets full key tiles take the path without a per-key bias. */
TNN_ROCM_API int tnn_rocm_mask_to_kv_len_flagged(void *stream, const float *mask, int32_t *kv_len, int B, int S,
                                                 float threshold);
TNN_ROCM_API int tnn_rocm_mask_to_kv_len(void *stream, const float *mask, int32_t *kv_len, int B, int S,
                                         float threshold);
/* The flagged form for a mask [B,S] of any float type, in one launch: a half-precision mask is also widened into
 * mask_f32 [B,S] (the form the attention kernels read; may be NULL for an fp32 mask, which is used where it lies). */
TNN_ROCM_API int tnn_rocm_mask_prepare(void *stream, int dtype, const void *mask, float *mask_f32, int32_t *kv_len,
                                       int B, int S, float threshold);
/* The same for a mask whose row b starts mask_batch_stride elements after row b-1; 0 = one row [S] that serves every
 * sequence (an additive mask of shape [1,1,1,S], broadcast over the batch as the reference's Add does,
 * source/tnn/layer/multidir_broadcast_layer.cc:59-111).  mask_f32, when given, receives the dense fp32 [B,S] copy
 * whatever the source type; it is required unless the source is dense fp32. */
TNN_ROCM_API int tnn_rocm_mask_prepare_strided(void *stream, int dtype, const void *mask, long mask_batch_stride,
                                               float *mask_f32, int32_t *kv_len, int B, int S, float threshold);

/* ---- row-wise ops ---------------------------------------------------------------------------
 * Softmax over `channel` of x viewed as [outer][channel][inner]
 *       cpu_softmax_layer_acc.cc:30-97 ; x86_softmax_layer_acc.cc:28-151 */
TNN_ROCM_API int tnn_rocm_softmax(void *stream, int dtype, const void *x, void *y, int outer, int channel, int inner);

/* y = LayerNorm(x (+ residual)) * gamma + beta over the last `cols` elements of each row;
 * one-pass E[x^2]-E[x]^2 variance as the reference (cpu_layer_norm_layer_acc.cc:63-140,
 * x86_layer_norm_layer_acc.cc:26-86); gamma/beta fp32.  residual may be NULL.
 * Optional fused quantisation: if out_q is non-NULL it also receives
 * float2int8(y * q_inv_scale) (X86FloatToInt8, x86_compute_int8.cc:1254-1318). */
TNN_ROCM_API int tnn_rocm_layernorm(void *stream, int dtype, const void *x, const void *residual, const float *gamma,
                                    const float *beta, void *y, int rows, int cols, float eps, int8_t *out_q,
                                    float q_inv_scale);

/* ---- element-wise ops -----------------------------------------------------------------------
 * erf GELU   cpu_gelu_layer_acc.cc:31-51 */
TNN_ROCM_API int tnn_rocm_gelu(void *stream, int dtype, const void *x, void *y, size_t count);
/* tanh (the pooler's activation)   cpu_tanh_layer_acc.cc:23-27 */
TNN_ROCM_API int tnn_rocm_tanh(void *stream, int dtype, const void *x, void *y, size_t count);

/* out = a op b with numpy-style broadcast (shapes right-aligned, rank <= 6)
 *       CPU_ELEWISE  source/tnn/device/cpu/acc/compute/compute_elewise.cc:37-65
 * op: 0 add, 1 sub, 2 mul, 3 div. */
TNN_ROCM_API int tnn_rocm_binary(void *stream, int dtype, int op, const void *a, const int *host_shape_a, int rank_a,
                                 const void *b, const int *host_shape_b, int rank_b, void *out,
                                 const int *host_shape_out, int rank_out);

/* out dims[j] = in dims[order[j]]   NaivePermute, source/tnn/utils/naive_compute.cc:943-956 */
TNN_ROCM_API int tnn_rocm_permute(void *stream, int elem_bytes, const void *in, void *out, const int *host_in_dims,
                                  const int *host_order, int rank);

/* out[b][i][:] = data[b][indices[i]][:]; negative indices wrap; an out-of-range index leaves the
 * row zero-filled and sets *error_flag (device int32) to 1.
 *       CpuGatherLayerAcc::Forward  source/tnn/device/cpu/acc/cpu_gather_layer_acc.cc:27-86 */
TNN_ROCM_API int tnn_rocm_gather(void *stream, const void *data, const int32_t *indices, void *out, int batch,
                                 int slices, size_t slice_bytes, int n_indices, int32_t *error_flag);

/* Embedding front end of a BERT-style encoder in one launch:
 *   y[r][:] = LayerNorm((word_table[ids[r]][:] + pos_table[r % period][:]) + type_table[type_ids[r]][:])
 * i.e. Gather, Gather, Add(position constant), Add, LayerNorm (cpu_gather_layer_acc.cc:27-86,
 * compute_elewise.cc:37-65, cpu_layer_norm_layer_acc.cc:63-140) with the sums formed in that order.  Tables, y: dtype;
 * gamma/beta fp32.  Index rules as tnn_rocm_gather (negative wraps; out of range sets *error_flag and reads row 0).
 * Rows must be 16-byte aligned and at most 64*8 vectors of 16 bytes long. */
TNN_ROCM_API int tnn_rocm_embed_layernorm(void *stream, int dtype, const int32_t *ids, const int32_t *type_ids,
                                          const void *word_table, int vocab, const void *type_table, int n_types,
                                          const void *pos_table, int period, const float *gamma, const float *beta,
                                          float eps, void *y, int rows, int cols, int32_t *error_flag);

/* The same with the positions looked up as well (a third Gather over a position-id input instead of the constant
 * position rows): row r adds pos_table[pos_ids[r % n_pos_ids]] (n_pos_ids = rows, or S for ids of shape [1,S] that
 * broadcast over the batch); pos_table has pos_rows rows, index rules as for the other two tables. */
TNN_ROCM_API int tnn_rocm_embed_layernorm_pos(void *stream, int dtype, const int32_t *ids, const int32_t *type_ids,
                                              const int32_t *pos_ids, int n_pos_ids, const void *word_table, int vocab,
                                              const void *type_table, int n_types, const void *pos_table, int pos_rows,
                                              const float *gamma, const float *beta, float eps, void *y, int rows,
                                              int cols, int32_t *error_flag);

/* dtype conversion between F32, F16 and BF16 (round to nearest even), and between I32 and those three
 * (static_cast both ways: reference source/tnn/device/cpu/acc/cpu_cast_layer_acc.cc:41-53) */
TNN_ROCM_API int tnn_rocm_cast(void *stream, int src_dtype, const void *src, int dst_dtype, void *dst, size_t count);

/* ---- int8 boundary ops ----------------------------------------------------------------------
 * q = float2int8(x * inv_scale), inv_scale = (float)(1.0/scale) prepared by the host
 *       X86FloatToInt8  x86_compute_int8.cc:1254-1318 ; x86_reformat_layer_acc.cc:66-75 */
TNN_ROCM_API int tnn_rocm_quantize(void *stream, int src_dtype, const void *x, float inv_scale, int8_t *q,
                                   size_t count);
/* x = (float)q * scale     X86Int8ToFloat  x86_compute_int8.cc:1193-1252 */
TNN_ROCM_API int tnn_rocm_dequantize(void *stream, const int8_t *q, float scale, int dst_dtype, void *x, size_t count);
/* The same two with one scale per channel: element i of a [batch, channels, inner] blob takes entry (i / inner) % channels
 * of a device array of `channels` fp32 values (inverse scales for the quantiser, prepared by the host as above).
 *       X86FloatToInt8 / X86Int8ToFloat take the scale array and the channel count  x86_compute_int8.cc:1193-1318 ;
 *       per-channel blob scales as the int8 unit tests generate them  layer_resource_generator.cc:348-371 */
TNN_ROCM_API int tnn_rocm_quantize_per_channel(void *stream, int src_dtype, const void *x, const float *inv_scale, int8_t *q,
                                               size_t count, int channels, size_t inner);
TNN_ROCM_API int tnn_rocm_dequantize_per_channel(void *stream, const int8_t *q, const float *scale, int dst_dtype, void *x,
                                                 size_t count, int channels, size_t inner);
/* int8 Add, X86MatrixAddInt8 (x86_compute_int8.cc:795-831; scales x86_add_layer_acc.cc:33-66) as the reference's x86
 * build evaluates it (-mfma -ffast-math contract one product into the sum): y = float2int8(fma(b, sb, a*sa) * inv_so)
 * in the 8-channel vector body, float2int8(fma(a, sa, b*sb) * inv_so) in the scalar tail, i.e. the last four
 * channels when round_up(channels, 4) % 8 == 4.  channels = dims[1], inner = count(dims[2:]) of the blobs (plain
 * row-major); every batch entry is computed (the reference's loop stops after the first). */
TNN_ROCM_API int tnn_rocm_add_i8(void *stream, const int8_t *a, float sa, const int8_t *b, float sb, float inv_so,
                                 int8_t *y, size_t count, int channels, size_t inner);
/* The same with one scale per channel for each blob, as the reference's acc prepares them (x86_add_layer_acc.cc:33-66:
 * a_scale[c], b_scale[c] and 1.0 / o_scale[c]); sa, sb, inv_so are device arrays of `channels` values. */
TNN_ROCM_API int tnn_rocm_add_i8_per_channel(void *stream, const int8_t *a, const float *sa, const int8_t *b,
                                             const float *sb, const float *inv_so, int8_t *y, size_t count,
                                             int channels, size_t inner);
/* q_out = float2int8(gelu((float)q_in * in_scale) * out_inv_scale): Reformat -> GELU -> Reformat
 * collapsed into one pass (same three roundings as the separate layers). */
TNN_ROCM_API int tnn_rocm_gelu_i8(void *stream, const int8_t *q_in, float in_scale, float out_inv_scale,
                                  int8_t *q_out, size_t count);

/* ---- tuning and test hooks --------------------------------------------------------------------
 * No counterpart in the reference.  Process-wide switches for experiments and for the tests that force each kernel
 * variant; plain words read by later launches, so set them while no other thread is launching.  All return 0.
 *   gemm_config   : 0 = shape heuristic, -1 = the baseline kernel, else a tile-configuration code of the tiled kernel
 *   gemm_tune     : "MxNxK:code,..." overrides of the heuristic for single shapes (also TNN_ROCM_GEMM_TUNE at first use)
 *   gemm_group_m  : tiles per group of the XCD-aware tile order (0 = default)
 *   ln_y_ahead    : 1 (default) = the LayerNorm-folding GEMMs request the source vectors of their y output early
 *   attention_dma : 1 (default) = V^T attention stages K / V^T tiles global -> LDS directly, 0 = through registers
 *   store_through : 1 (default) = GEMM and attention results are stored through the L2 at device scope, so that no
 *                   dirty lines wait for the write-back at the end of the kernel; 0 = ordinary write-back stores.
 *                   Read by the kernels when they run (recorded graphs follow it too); waits for the device first. */
TNN_ROCM_API int tnn_rocm_debug_set_gemm_config(int cfg);
TNN_ROCM_API int tnn_rocm_debug_set_gemm_tune(const char *spec);
TNN_ROCM_API int tnn_rocm_debug_set_gemm_group_m(int group_m);
TNN_ROCM_API int tnn_rocm_debug_set_ln_y_ahead(int on);
TNN_ROCM_API int tnn_rocm_debug_set_attention_dma(int on);
TNN_ROCM_API int tnn_rocm_debug_set_store_through(int on);

#ifdef __cplusplus
}
#endif
#endif /* TNN_ROCM_H_ */
