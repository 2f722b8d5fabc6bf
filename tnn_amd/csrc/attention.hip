// Fused attention core for gfx950: out = softmax(Q K^T * scale + mask) V, head_dim 64, fp16/bf16
// inputs with fp32 accumulation and an online (running max / running sum) softmax, so the
// [B*h, S, S] score tensor of the decomposed graph never exists in memory.
//
// Work split: one workgroup = one (batch, head, block of NW*32 query rows); each 64-lane wave owns
// 32 query rows.  Keys/values are walked in tiles of 64 keys staged in LDS (double buffered, the
// next tile's global loads are in flight during the current tile's MFMAs).
//
// The scores are computed TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16: in the 32x32
// accumulator layout a lane then holds ONE query column (lane % 32) and 16 of the 32 keys of the
// block, so the row max / row sum of the softmax are 16 in-register operations plus a single
// exchange with lane^32, and the rescale factor of the running output is a per-lane scalar.
// The probabilities are already in the register order the second MFMA wants for its B operand
// (O^T = V^T P^T): slot e of lane-half g of a 16-key step maps to key
//     16*step + 4*g + e        (e < 4)      and      16*step + 8 + 4*g + (e-4)   (e >= 4),
// so V is stored transposed in LDS ([d][key]) and each lane fetches its two 4-key groups with two
// 8-byte reads.  Padding keys (>= kv_len) are excluded exactly (−inf) in-register and whole tiles
// past kv_len are never loaded.
#include <atomic>
#include <type_traits>

#include "common.h"

using namespace tnn_rocm;

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kD        = 64;            // head dim
constexpr int kTileKV   = 64;            // keys per LDS tile
constexpr int kRowBytes = kD * 2 + 16;   // padded LDS row (K: one key's 64 halfs; V^T: one d's 64 keys)
constexpr float kLog2e  = 1.4426950408889634f;
constexpr int kKvLenMaskZero = 1 << 30;  // flag bit of a kv_len entry, see tnn_rocm_mask_to_kv_len_flagged

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int DT> struct AttnT;
template <> struct AttnT<TNN_ROCM_F16> {
    template <typename V> static __device__ __forceinline__ void mma(const V &a, const V &b, f32x16 &c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                   0);
    }
    // First product of an accumulation chain, d = a b + c0, with c0 read from registers of its own and left intact.
    // Written as an instruction because the compiler only emits the form whose destination is also the C operand and
    // copies c0 into d first (16 moves per chain).  The early-clobber output keeps d apart from the inputs.  The compiler
    // does not look inside the statement, so it inserts none of the wait states an instruction that reads d right
    // after a matrix instruction needs (none for an accumulating MFMA of the same opcode into d; passes + 3 = 11 for a
    // vector instruction and passes + 2 for an MFMA with another destination, this product taking 8 passes of 4
    // clocks): the statement carries them itself, so that whatever the compiler schedules next is safe.  They pass
    // while the matrix pipe works on this product.
    template <typename V> static __device__ __forceinline__ f32x16 mma_from(const V &a, const V &b, const f32x16 &c0) {
        f32x16 d;
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3\n\ts_nop 10" : "=&v"(d) : "v"(a), "v"(b), "v"(c0));
        return d;
    }
    static __device__ __forceinline__ float to_float(uint16_t bits) { return (float)__builtin_bit_cast(half_t, bits); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        half_t l = (half_t)lo, h = (half_t)hi;
        return (uint32_t)__builtin_bit_cast(uint16_t, l) | ((uint32_t)__builtin_bit_cast(uint16_t, h) << 16);
    }
    // the same in two steps, for callers that shuffle the packed pairs before summing them
    static __device__ __forceinline__ uint32_t pack_only(float lo, float hi) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
    }
    static __device__ __forceinline__ void add_packed(uint32_t pk, float &sum) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 one = {(_Float16)1.0f, (_Float16)1.0f};
        sum    = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, pk), one, sum, false);
    }
    // Probabilities (0..1) for the second MFMA: one v_cvt_pkrtz per pair.  The row sum is taken over the SAME
    // rounded values (v_dot2 with (1,1), fp32 accumulate), so numerator and denominator of the softmax stay
    // consistent and the truncation does not bias the normalised weights.
    static __device__ __forceinline__ uint32_t pack_prob(float lo, float hi, float &sum) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
        fp16x2 pk = __builtin_amdgcn_cvt_pkrtz(lo, hi);
        h2 one    = {(_Float16)1.0f, (_Float16)1.0f};
        sum       = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, pk), one, sum, false);
        return __builtin_bit_cast(uint32_t, pk);
    }
};
template <> struct AttnT<TNN_ROCM_BF16> {
    template <typename V> static __device__ __forceinline__ void mma(const V &a, const V &b, f32x16 &c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                    0, 0);
    }
    template <typename V> static __device__ __forceinline__ f32x16 mma_from(const V &a, const V &b, const f32x16 &c0) {
        f32x16 d;
        asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3\n\ts_nop 10" : "=&v"(d) : "v"(a), "v"(b), "v"(c0));
        return d;
    }
    static __device__ __forceinline__ float to_float(uint16_t bits) { return __uint_as_float((uint32_t)bits << 16); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        return (uint32_t)float_to_bf16(lo) | ((uint32_t)float_to_bf16(hi) << 16);
    }
    static __device__ __forceinline__ uint32_t pack_only(float lo, float hi) {
        return (uint32_t)float_to_bf16(lo) | ((uint32_t)float_to_bf16(hi) << 16);
    }
    static __device__ __forceinline__ void add_packed(uint32_t pk, float &sum) {
        sum += __uint_as_float(pk << 16) + __uint_as_float(pk & 0xffff0000u);
    }
    static __device__ __forceinline__ uint32_t pack_prob(float lo, float hi, float &sum) {
        uint32_t l = float_to_bf16(lo), h = float_to_bf16(hi);
        sum += __uint_as_float(l << 16) + __uint_as_float(h << 16);  // the rounded values, as in the fp16 path
        return l | (h << 16);
    }
};

struct AttnParams {
    const uint16_t *q, *k, *v;
    uint16_t *o;
    long q_sb, q_sh, q_ss, kv_sb, kv_sh, kv_ss, o_sb, o_sh, o_ss;
    long vt_sb, vt_sh, vt_sd;  // V^T layout (VT kernels): element (b, head, d, s) at v[b*vt_sb + head*vt_sh + d*vt_sd + s]
    int S, B, heads;
    float scale_log2e;  // scale * log2(e)
    const float *mask;  // [B,S] additive or null
    const int32_t *kv_len;
    int8_t *oq;   // optional second output: the stored values quantised, same element strides as o
    float q_inv;  // 1 / scale of that int8 tensor
    // V^T key order (VT kernels).  0: natural.  1: inside every group of 16 keys the two middle blocks of four have
    // changed places ([k0-3 | k8-11 | k4-7 | k12-15]), which is the order in which a lane half holds the probabilities
    // of a score tile (rows 8*(r/4) + 4*half + r%4 of the accumulator block): the packed probabilities then feed the
    // second MFMA as they are, with no exchange between the lane halves.  Needs S % 16 == 0.
    int vt_perm;
};

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Combine a value with the one held by lane ^ 32 (the other half of the same query column) with one
// v_permlane32_swap: after swapping the upper half of one copy with the lower half of the other, every lane
// holds its own value in one register and its partner's in the other.
__device__ __forceinline__ float half_swap_max(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The second launch bound (at least two waves per SIMD) caps the kernel at 256 registers, which keeps the MFMA accumulators in ordinary VGPRs: the softmax
// reads and rescales them with VALU instructions, and accumulators parked in AGPRs cost a move per access.
template <int DT, int NW, bool VT>
__global__ void __launch_bounds__(NW * 64, (NW == 4 && DT == TNN_ROCM_F16) ? 3 : 2) attention_kernel(AttnParams p) {
    constexpr int NT = NW * 64;
    constexpr int BQ = NW * 32;
    // per tile: 64 rows (keys, or d for V^T) x 8 sixteen-byte chunks
    constexpr int KV_VECS  = kTileKV * 8 / NT;
    constexpr int ROW_STEP = NT / 8;
    static_assert(kTileKV * 8 % NT == 0, "tile must divide over the workgroup");

    // one LDS block: [K tile 0 | V^T tile 0 | K tile 1 | V^T tile 1]; the second half doubles as the staging area of
    // the Q block before the first tile is stored there, the first half as the staging area of the output block
    constexpr int kTileBytes = kTileKV * kRowBytes;  // = kD * kRowBytes
    __shared__ __attribute__((aligned(16))) unsigned char lds_all[4 * kTileBytes];
    __shared__ __attribute__((aligned(16))) float lds_bias[2][kTileKV];
    unsigned char *const lds_k0 = lds_all, *const lds_vt0 = lds_all + kTileBytes;
    unsigned char *const lds_k1 = lds_all + 2 * kTileBytes, *const lds_vt1 = lds_all + 3 * kTileBytes;
    static_assert(BQ * kRowBytes <= 2 * kTileBytes, "Q / O staging must fit half of the tile buffers");

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int g    = lane >> 5;  // lane half
    const int lq   = lane & 31;  // query column owned by this lane
    const int S    = p.S;
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Every XCD takes a contiguous run of
    // (batch, head) pairs and all query tiles of a pair, so the K and V of a head are fetched into one L2 only
    // (with the plain 3-D grid the query tiles of one head land on different XCDs and each re-reads K and V).
    const int n_q   = (S + BQ - 1) / BQ;
    const int total = n_q * p.heads * p.B;
    const int per   = (total + 7) >> 3;
    const int vid   = (int)(blockIdx.x & 7) * per + (int)(blockIdx.x >> 3);
    if (vid >= total)
        return;  // the grid is padded to a multiple of 8; whole workgroups leave before any barrier
    const int bh   = vid / n_q;
    const int b    = bh / p.heads;
    const int head = bh - b * p.heads;
    const int q0   = (vid - bh * n_q) * BQ + wave * 32;

    int kv_end = S;
    bool mask_is_zero = false;  // kv_len[b] may carry kKvLenMaskZero: the mask row is 0 for every key below kv_len[b]
    if (p.kv_len) {
        int l        = p.kv_len[b];
        mask_is_zero = l >= 0 && (l & kKvLenMaskZero) != 0;
        l            = l >= 0 ? (l & ~kKvLenMaskZero) : l;
        kv_end       = l < 0 ? 0 : (l < S ? l : S);
    }
    const int n_tiles = (kv_end + kTileKV - 1) / kTileKV;

    const uint16_t *qb = p.q + (size_t)b * p.q_sb + (size_t)head * p.q_sh;
    const uint16_t *kb = p.k + (size_t)b * p.kv_sb + (size_t)head * p.kv_sh;
    const uint16_t *vb = VT ? p.v + (size_t)b * p.vt_sb + (size_t)head * p.vt_sh
                            : p.v + (size_t)b * p.kv_sb + (size_t)head * p.kv_sh;
    uint16_t *ob       = p.o + (size_t)b * p.o_sb + (size_t)head * p.o_sh;
    const float *mb    = p.mask && !mask_is_zero ? p.mask + (size_t)b * S : nullptr;

    // No load below is guarded by a branch: row indices past the end are clamped to the last valid row.  Keys at or
    // beyond kv_end then carry finite (wrong) data, and their score bias of -inf makes their probability exactly 0,
    // so neither the max, the sum nor P.V sees them; query rows past S are computed but never stored.
    // Q fragments (B operand of S^T = K Q^T): lane (lq, g) holds Q[q0+lq][16*kk + 8*g .. +7]
    // The block's BQ x 64 Q rows are copied through LDS with whole 128-byte rows per 8 lanes (a lane reading its own
    // row directly touches 32 rows per instruction with 32 bytes each).
    u32x4 qf[4];
    {
        unsigned char *const stage = lds_k1;  // free until the end of the first tile
        constexpr int Q_VECS = BQ * 8 / NT;
#pragma unroll
        for (int i = 0; i < Q_VECS; ++i) {
            const int v = tid + i * NT, r = v >> 3, c = v & 7;
            int qrow = (q0 - wave * 32) + r;
            qrow     = qrow < S ? qrow : S - 1;
            *reinterpret_cast<u32x4 *>(stage + r * kRowBytes + c * 16) =
                *reinterpret_cast<const u32x4 *>(qb + (size_t)qrow * p.q_ss + c * 8);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
            qf[kk] = *reinterpret_cast<const u32x4 *>(stage + (wave * 32 + lq) * kRowBytes + kk * 32 + g * 16);
        __syncthreads();  // the staging area becomes tile buffer 1
    }

    const int vrow = tid >> 3, vch = tid & 7;  // this thread's row / 16-byte chunk inside a tile (plus i*ROW_STEP)
    // one tile of look-ahead in registers (a second register set for two tiles ahead was measured slower: the
    // extra registers cost a resident wave per SIMD, and the memory latency is already covered)
    u32x4 rk[KV_VECS], rv[KV_VECS];
    float rbias = 0.f;
    // element offsets from the (batch, head) base fit 32 bits (checked by the launcher)
    const uint32_t kv_ss32 = (uint32_t)p.kv_ss, vt_sd32 = (uint32_t)p.vt_sd;
    uint32_t v_off[KV_VECS];  // V^T: row d = vrow + i*ROW_STEP, plus the key offset of the tile
#pragma unroll
    for (int i = 0; i < KV_VECS; ++i)
        v_off[i] = (uint32_t)(vrow + i * ROW_STEP) * vt_sd32;

#define TR_LOAD_TILE(T)                                                                                               \
    {                                                                                                                 \
        const int kv0 = (T) * kTileKV;                                                                                \
        int k8        = kv0 + vch * 8;                                                                                \
        k8            = k8 < S ? k8 : S - 8;                                                                          \
        _Pragma("unroll") for (int i = 0; i < KV_VECS; ++i) {                                                         \
            int key = kv0 + vrow + i * ROW_STEP;                                                                      \
            key     = key < S ? key : S - 1;                                                                          \
            const uint32_t ko = (uint32_t)key * kv_ss32 + (uint32_t)(vch * 8);                                        \
            rk[i]   = *reinterpret_cast<const u32x4 *>(kb + ko);                                                      \
            if (VT)                                                                                                   \
                rv[i] = *reinterpret_cast<const u32x4 *>(vb + (v_off[i] + (uint32_t)k8));                             \
            else                                                                                                      \
                rv[i] = *reinterpret_cast<const u32x4 *>(vb + ko);                                                    \
        }                                                                                                             \
        if (tid < kTileKV) {                                                                                          \
            int key  = kv0 + tid;                                                                                     \
            int keyc = key < S ? key : S - 1;                                                                         \
            float mv = mb ? mb[keyc] * kLog2e : 0.f;                                                                  \
            rbias    = key < kv_end ? mv : -INFINITY;                                                                 \
        }                                                                                                             \
    }
// V^T rows are stored with the two middle 8-byte chunks of every 16-key group swapped ([k0-3 | k8-11 | k4-7 | k12-15]):
// the eight keys a lane needs for one MFMA step (16*step + 4*g + 0..3 and 16*step + 8 + 4*g + 0..3) are then one
// aligned 16-byte read at step*32 + g*16.
#define TR_STORE_TILE(BUF)                                                                                            \
    {                                                                                                                 \
        _Pragma("unroll") for (int i = 0; i < KV_VECS; ++i) {                                                         \
            const int row = vrow + i * ROW_STEP;                                                                      \
            *reinterpret_cast<u32x4 *>(lds_k##BUF + row * kRowBytes + vch * 16) = rk[i];                              \
            if (VT && p.vt_perm) {                                                                                    \
                /* the rows already come in the order the fragments want */                                          \
                *reinterpret_cast<u32x4 *>(lds_vt##BUF + row * kRowBytes + vch * 16) = rv[i];                         \
            } else if (VT) {                                                                                          \
                /* this thread holds keys 8*vch .. 8*vch+7 of row d: chunk pair (2*(vch&1), 2*(vch&1)+1) of group */  \
                /* vch/2 goes to chunk positions (vch&1) and (vch&1)+2 */                                             \
                unsigned char *dst = lds_vt##BUF + row * kRowBytes + (vch >> 1) * 32 + (vch & 1) * 8;                 \
                *reinterpret_cast<u32x2 *>(dst)      = u32x2{rv[i][0], rv[i][1]};                                     \
                *reinterpret_cast<u32x2 *>(dst + 16) = u32x2{rv[i][2], rv[i][3]};                                     \
            } else {                                                                                                  \
                /* thread holds d = 8*vch .. +7 of key `row`: scatter into the transposed tile at the key's slot */  \
                const int kslot = (row & ~15) + ((row & 3) | ((row & 4) << 1) | ((row & 8) >> 1));                    \
                _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                                       \
                    *reinterpret_cast<uint16_t *>(lds_vt##BUF + (vch * 8 + 2 * e) * kRowBytes + kslot * 2) =          \
                        (uint16_t)(rv[i][e] & 0xffffu);                                                               \
                    *reinterpret_cast<uint16_t *>(lds_vt##BUF + (vch * 8 + 2 * e + 1) * kRowBytes + kslot * 2) =      \
                        (uint16_t)(rv[i][e] >> 16);                                                                   \
                }                                                                                                     \
            }                                                                                                         \
        }                                                                                                             \
        if (tid < kTileKV)                                                                                            \
            lds_bias[BUF][tid] = rbias;                                                                               \
    }

    f32x16 oacc[2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            oacc[dt][r] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;

    // one tile: scores, online softmax, P.V -- reads LDS buffer `buf`, which holds tile t
    auto tile_body = [&](const int buf, const int t) __attribute__((always_inline)) {
        const unsigned char *const kbuf  = buf ? lds_k1 : lds_k0;
        const unsigned char *const vtbuf = buf ? lds_vt1 : lds_vt0;
        // ---- S^T = K Q^T for the 64 keys of the tile: two 32-key blocks
        f32x16 sacc[2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                sacc[kt][r] = 0.f;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                u32x4 kf = *reinterpret_cast<const u32x4 *>(kbuf + (kt * 32 + lq) * kRowBytes + kk * 32 + g * 16);
                AttnT<DT>::mma(kf, qf[kk], sacc[kt]);
            }
        }

        // ---- online softmax in the exp2 domain; register r of block kt is key kt*32 + 8*(r/4) + 4*g + (r%4).
        // A tile needs the per-key bias only if it carries an additive mask or reaches past kv_end (the last tile):
        // all other tiles take the short path, p = exp2(s*c - m) with the row maximum taken on the raw scores.
        const bool biased = mb != nullptr || (t + 1) * kTileKV > kv_end || !(p.scale_log2e > 0.f);  // workgroup-uniform
        float mx = -INFINITY;
        if (biased) {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    float4 bias = *reinterpret_cast<const float4 *>(&lds_bias[buf][kt * 32 + r4 * 8 + g * 4]);
                    float bv[4] = {bias.x, bias.y, bias.z, bias.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float s2             = fmaf(sacc[kt][r4 * 4 + e], p.scale_log2e, bv[e]);
                        sacc[kt][r4 * 4 + e] = s2;
                        mx                   = fmaxf(mx, s2);
                    }
                }
            }
        } else {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    mx = fmaxf(mx, sacc[kt][r]);
            mx *= p.scale_log2e;  // scale > 0 on this path: the maximum commutes with it
        }
        mx          = half_swap_max(mx);
        float m_new = fmaxf(m_i, mx);
        float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        float alpha = __builtin_amdgcn_exp2f(m_i - m_use);
        if (biased) {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    sacc[kt][r] = __builtin_amdgcn_exp2f(sacc[kt][r] - m_use);
        } else {
            const float neg_m = -m_use;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    sacc[kt][r] = __builtin_amdgcn_exp2f(fmaf(sacc[kt][r], p.scale_log2e, neg_m));
        }
        // the running maximum rarely moves after the first tiles: skip the 32 rescale multiplies when no lane's did
        if (!__all(m_new == m_i)) {
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    oacc[dt][r] *= alpha;
        }
        m_i = m_new;

        // ---- O^T += V^T P^T : four 16-key steps; the row sum is accumulated while packing
        float rs = 0.f;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int kt = st >> 1, j = st & 1;
            u32x4 pf;
            pf[0] = AttnT<DT>::pack_prob(sacc[kt][8 * j + 0], sacc[kt][8 * j + 1], rs);
            pf[1] = AttnT<DT>::pack_prob(sacc[kt][8 * j + 2], sacc[kt][8 * j + 3], rs);
            pf[2] = AttnT<DT>::pack_prob(sacc[kt][8 * j + 4], sacc[kt][8 * j + 5], rs);
            pf[3] = AttnT<DT>::pack_prob(sacc[kt][8 * j + 6], sacc[kt][8 * j + 7], rs);
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const u32x4 vf = *reinterpret_cast<const u32x4 *>(vtbuf + (dt * 32 + lq) * kRowBytes + st * 32 + g * 16);
                AttnT<DT>::mma(vf, pf, oacc[dt]);
            }
        }
        rs  = half_swap_sum(rs);
        l_i = fmaf(l_i, alpha, rs);

    };

    if (n_tiles > 0) {
        TR_LOAD_TILE(0);
        TR_STORE_TILE(0);
    }
    __syncthreads();
    for (int t = 0; t < n_tiles; t += 2) {
        // look-ahead load of the next tile (clamped to the last one: the redundant copy is never consumed)
        TR_LOAD_TILE((t + 1 < n_tiles ? t + 1 : t));
        tile_body(0, t);
        TR_STORE_TILE(1);
        __syncthreads();
        if (t + 1 >= n_tiles)
            break;  // uniform over the workgroup
        TR_LOAD_TILE((t + 2 < n_tiles ? t + 2 : t + 1));
        tile_body(1, t + 1);
        TR_STORE_TILE(0);
        __syncthreads();
    }
#undef TR_LOAD_TILE
#undef TR_STORE_TILE

    // ---- normalise and store.  Lane owns query row q0+lq; register r of block dt is d = dt*32 + 8*(r/4) + 4*g + (r%4).
    // Written straight from this layout a store instruction would touch 32 rows with 16 bytes each; the wave's 32 x 64
    // block goes through LDS instead (the tile buffers are free now) and leaves with 8 lanes per 128-byte row.
    __syncthreads();  // every wave is done with the last tile
    {
        unsigned char *const stage = lds_all + wave * 32 * kRowBytes;  // private to this wave
        const float inv            = l_i > 0.f ? 1.0f / l_i : 0.f;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                u32x2 w;
                w[0] = AttnT<DT>::pack2(oacc[dt][r4 * 4 + 0] * inv, oacc[dt][r4 * 4 + 1] * inv);
                w[1] = AttnT<DT>::pack2(oacc[dt][r4 * 4 + 2] * inv, oacc[dt][r4 * 4 + 3] * inv);
                *reinterpret_cast<u32x2 *>(stage + lq * kRowBytes + (dt * 32 + r4 * 8 + g * 4) * 2) = w;
            }
        // LDS operations of one wave complete in order; the fences keep the compiler from reordering across them
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int r    = pass * 8 + (lane >> 3);
            const int qrow = q0 + r;
            if (qrow < S) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + r * kRowBytes + (lane & 7) * 16);
                store_out16(ob + (size_t)qrow * p.o_ss + (lane & 7) * 8, v);
                if (p.oq) {
                    // the Reformat layer that follows in a quantised net (x86 form: multiply by 1/scale, round half
                    // away from zero, saturate), applied to the values as stored
                    u32x2 q8;
#pragma unroll
                    for (int w = 0; w < 2; ++w) {
                        uint32_t packed = 0;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t word = v[w * 2 + (e >> 1)];
                            const float f       = AttnT<DT>::to_float((uint16_t)(e & 1 ? word >> 16 : word & 0xffffu));
                            packed |= (uint32_t)(uint8_t)float2int8_ref(__fmul_rn(f, p.q_inv)) << (8 * e);
                        }
                        q8[w] = packed;
                    }
                    int8_t *oqb = p.oq + (size_t)b * p.o_sb + (size_t)head * p.o_sh;
                    store_out8(oqb + (size_t)qrow * p.o_ss + (lane & 7) * 8, q8);
                }
            }
        }
    }
}

// ---- the same computation with the K and V^T tiles loaded global -> LDS directly -------------------------------------
// For the V^T layout.  Three 16 KB stages of un-padded 128-byte rows; global_load_lds_dwordx4 writes each lane's 16
// bytes at consecutive LDS addresses, so the XOR swizzle that keeps the fragment reads conflict-free (chunk p of row r
// holds logical chunk p ^ ((r >> 1) & 7)) is applied to the global addresses.  No staging registers, no LDS store
// instructions, no per-tile address arithmetic (the tile advances a scalar base); loads run two tiles ahead and the
// waits are placed by hand (the kernel issues no other vector-memory load inside the loop; the padding-mask values of
// a tile travel the same way).  V^T rows are plain here: the eight keys a lane half feeds into one P.V step are made
// contiguous by exchanging two packed probability registers between the lane halves (v_permlane32_swap) instead of
// permuting the keys inside the tile.
#define TR_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt((((n)&0xF) | ((((n) >> 4) & 3) << 14) | (0x7 << 4) | (0xF << 8)))

template <int DT, int NW, bool PERM>
__global__ void __launch_bounds__(NW * 64, (NW == 4 && DT == TNN_ROCM_F16) ? 3 : 2) attention_dma_kernel(AttnParams p) {
    constexpr int NT = NW * 64;
    constexpr int BQ = NW * 32;
    constexpr int kTile  = kTileKV * 128;  // one K or V^T tile, un-padded rows
    constexpr int kStage = 2 * kTile;
    constexpr int LD     = 8 / NW;         // 1 KB wave-loads per wave, tile and operand
    __shared__ __attribute__((aligned(16))) unsigned char lds_all[3 * kStage];
    __shared__ __attribute__((aligned(16))) float lds_bias[3][kTileKV];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int g    = lane >> 5;
    const int lq   = lane & 31;
    const int S    = p.S;
    const int n_q   = (S + BQ - 1) / BQ;
    const int total = n_q * p.heads * p.B;
    const int per   = (total + 7) >> 3;
    const int vid   = (int)(blockIdx.x & 7) * per + (int)(blockIdx.x >> 3);
    if (vid >= total)
        return;
    const int bh   = vid / n_q;
    const int b    = bh / p.heads;
    const int head = bh - b * p.heads;
    const int q0   = (vid - bh * n_q) * BQ + wave * 32;

    int kv_end = S;
    bool mask_is_zero = false;  // kv_len[b] may carry kKvLenMaskZero: the mask row is 0 for every key below kv_len[b]
    if (p.kv_len) {
        int l        = p.kv_len[b];
        mask_is_zero = l >= 0 && (l & kKvLenMaskZero) != 0;
        l            = l >= 0 ? (l & ~kKvLenMaskZero) : l;
        kv_end       = l < 0 ? 0 : (l < S ? l : S);
    }
    const int n_tiles = (kv_end + kTileKV - 1) / kTileKV;

    const uint16_t *qb = p.q + (size_t)b * p.q_sb + (size_t)head * p.q_sh;
    const uint16_t *kb = p.k + (size_t)b * p.kv_sb + (size_t)head * p.kv_sh;
    const uint16_t *vb = p.v + (size_t)b * p.vt_sb + (size_t)head * p.vt_sh;
    uint16_t *ob       = p.o + (size_t)b * p.o_sb + (size_t)head * p.o_sh;
    const float *mb    = p.mask && !mask_is_zero ? p.mask + (size_t)b * S : nullptr;

    // ---- tile loads.  Wave-load j = wave + i*NW covers LDS rows 8j .. 8j+7 of a tile
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds_all, bias_base = (uint32_t)(uintptr_t)&lds_bias[0][0];
    const int lrow = lane >> 3, lpos = lane & 7;
    const uint32_t kv_ss32 = (uint32_t)p.kv_ss, vt_sd32 = (uint32_t)p.vt_sd;
    uint32_t k_off[LD], v_off[LD];  // byte offsets of this lane's 16 bytes from the tile's first key
    int l_row[LD], l_chunk[LD];
#pragma unroll
    for (int i = 0; i < LD; ++i) {
        const int r = (wave + i * NW) * 8 + lrow;
        l_row[i]    = r;
        l_chunk[i]  = lpos ^ ((r >> 1) & 7);
        k_off[i]    = ((uint32_t)r * kv_ss32 + (uint32_t)l_chunk[i] * 8u) * 2u;
        v_off[i]    = ((uint32_t)r * vt_sd32 + (uint32_t)l_chunk[i] * 8u) * 2u;
    }
    auto load16 = [](const void *base, uint32_t byte_off, uint32_t lds_addr) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(byte_off), "s"(base), "s"(lds_addr) : "memory");
    };
    auto load4 = [](const void *base, uint32_t byte_off, uint32_t lds_addr) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(byte_off), "s"(base), "s"(lds_addr) : "memory");
    };
    const uint32_t wave_dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_base + (uint32_t)wave * 1024u));
    auto issue = [&](int t, int stage) {
        const int kv0      = t * kTileKV;
        const uint32_t dst = wave_dst + (uint32_t)(stage * kStage);
        if (kv0 + kTileKV <= S) {  // whole tile inside the sequence: the tile only moves the scalar base
            const uint16_t *kt_base = kb + (size_t)kv0 * p.kv_ss, *vt_base = vb + kv0;
#pragma unroll
            for (int i = 0; i < LD; ++i)
                load16(kt_base, k_off[i], dst + i * NW * 1024);
#pragma unroll
            for (int i = 0; i < LD; ++i)
                load16(vt_base, v_off[i], dst + kTile + i * NW * 1024);
        } else {  // last, partial tile: rows / key chunks past the end are clamped (their bias is -inf)
#pragma unroll
            for (int i = 0; i < LD; ++i) {
                int key = kv0 + l_row[i];
                key     = key < S ? key : S - 1;
                load16(kb, ((uint32_t)key * kv_ss32 + (uint32_t)l_chunk[i] * 8u) * 2u, dst + i * NW * 1024);
            }
#pragma unroll
            for (int i = 0; i < LD; ++i) {
                int k8 = kv0 + l_chunk[i] * 8;
                k8     = k8 < S ? k8 : S - 8;
                load16(vb, ((uint32_t)l_row[i] * vt_sd32 + (uint32_t)k8) * 2u, dst + kTile + i * NW * 1024);
            }
        }
        if (mb) {  // the tile's 64 additive mask values; every wave writes the same 256 bytes
            int key = kv0 + lane;
            key     = key < S ? key : S - 1;
            load4(mb, (uint32_t)key * 4u, bias_base + (uint32_t)(stage * kTileKV * 4));
        }
    };
    constexpr int LPW = 2 * LD;
    if (!mb)
        for (int i = tid; i < 3 * kTileKV; i += NT)
            (&lds_bias[0][0])[i] = 0.f;  // visible to everyone after the barrier that opens the first tile
    if (n_tiles > 0)
        issue(0, 0);

    // ---- Q fragments: lane (lq, g) holds elements 16 kk + 8 g .. + 7 of query row q0 + lq for the four k-steps.
    // Four waves take them straight from memory (sixteen bytes per row and lane half is a poor shape for one load, but
    // the four loads of a wave cover whole 128-byte rows between them: B32 S512 lengths U[16,512] 29.7 -> 29.2 us);
    // two waves go through LDS with whole-row loads (stages 1 and 2 are free until the second tile is requested), where
    // the direct form measured slower (B8 S384: 11.7 -> 12.3 us).
    u32x4 qf[4];
    if constexpr (NW == 4) {
        int qrow = q0 + lq;
        qrow     = qrow < S ? qrow : S - 1;
        const uint16_t *qp = qb + (size_t)qrow * p.q_ss + g * 8;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
            qf[kk] = *reinterpret_cast<const u32x4 *>(qp + kk * 16);
    } else {
        static_assert(BQ * kRowBytes <= 2 * kStage, "Q staging must fit stages 1 and 2");
        unsigned char *const stage = lds_all + kStage;
        constexpr int Q_VECS = BQ * 8 / NT;
#pragma unroll
        for (int i = 0; i < Q_VECS; ++i) {
            const int v = tid + i * NT, r = v >> 3, c = v & 7;
            int qrow = (q0 - wave * 32) + r;
            qrow     = qrow < S ? qrow : S - 1;
            *reinterpret_cast<u32x4 *>(stage + r * kRowBytes + c * 16) =
                *reinterpret_cast<const u32x4 *>(qb + (size_t)qrow * p.q_ss + c * 8);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
            qf[kk] = *reinterpret_cast<const u32x4 *>(stage + (wave * 32 + lq) * kRowBytes + kk * 32 + g * 16);
        __syncthreads();
    }
    if (n_tiles > 1)
        issue(1, 1);
    // Q is scaled by c = scale * log2(e) once (fp32 product, one rounding back to the input type), so the score
    // MFMAs deliver s*c and the key loop never multiplies a score again.
    {
        const float c = p.scale_log2e;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t word = qf[kk][w];
                qf[kk][w] = AttnT<DT>::pack2(AttnT<DT>::to_float((uint16_t)(word & 0xffffu)) * c,
                                             AttnT<DT>::to_float((uint16_t)(word >> 16)) * c);
            }
    }

    // fragment chunk x = 2*step + g of row lq (the same expression serves the K and the V^T tile)
    uint32_t frag_off[4];
#pragma unroll
    for (int x = 0; x < 4; ++x)
        frag_off[x] = (uint32_t)(lq * 128 + (((2 * x + g) ^ ((lq >> 1) & 7)) * 16));

    f32x16 oacc[2];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            oacc[dt][r] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;
    f32x16 negm;  // -m_i in every register: the start value of the score accumulators in the FAST tile form
#pragma unroll
    for (int r = 0; r < 16; ++r)
        negm[r] = INFINITY;
    asm volatile("" : "+v"(negm));

    // The tile body exists in three forms.  x = the scaled score as the MFMA delivers it (Q carries scale*log2 e):
    //   BIAS : x + bias (additive mask, -inf for keys past kv_end), exact running maximum m, p = exp2(x + bias - m)
    //   EXACT: the same without a bias (the first tile of a row block)
    //   FAST : no bias, m finite.  The first MFMA of each score chain starts from a register block holding -m, so the
    //          accumulators come out as x - m and p = exp2 of them: no per-score arithmetic besides the exponential.
    //          m is not advanced: the probabilities may use a stale reference as long as they fit the packed
    //          half-precision operand of the second MFMA.  That is checked on the row sums (a lane's partial sum above
    //          kStaleLimit, or not finite, means some p may be too large) before anything is added to O; if it fails
    //          (rare) the wave leaves the FAST loop and takes the same tile again in the EXACT form, which advances m.
    //          The normalised result does not depend on which reference the exponentials use.
    // Control flow: an outer loop runs one BIAS / EXACT tile, then an inner loop runs FAST tiles for as long as they
    // are eligible and pass their check.  The inner loop has one body and one exit, so the O accumulators stay in the
    // same registers around it.
    constexpr float kStaleLimit = 1024.0f;  // p up to 2^10: 64 of them still sum far below the half-precision range
    int stage = 0, fill = 2;
    auto enter_tile = [&](int t) __attribute__((always_inline)) {
        // tile t has landed once at most the loads of tile t + 1 are outstanding
        if (t + 1 < n_tiles) {
            if (mb)
                TR_WAIT_VMCNT(LPW + 1);
            else
                TR_WAIT_VMCNT(LPW);
        } else {
            TR_WAIT_VMCNT(0);
        }
        __builtin_amdgcn_s_barrier();  // everyone's part of tile t is in LDS; everyone is done with tile t - 1
        asm volatile("" ::: "memory");  // no LDS access may be moved across the barrier by the compiler
        if (t + 2 < n_tiles)
            issue(t + 2, fill);
    };
    auto leave_tile = [&]() __attribute__((always_inline)) {
        stage = stage == 2 ? 0 : stage + 1;
        fill  = fill == 2 ? 0 : fill + 1;
    };
    // Probabilities -> packed operands of the second MFMA.  Register r of block kt is key kt*32 + 8*(r/4) + 4*g +
    // (r%4): a lane half holds four keys of each 8-key group.  Step st = 2*kt + j uses groups 2j and 2j+1 of the
    // block; after exchanging the packed pairs (group 2j+1 of the lower half <-> group 2j of the upper half) lane half
    // g holds the eight consecutive keys of group 2j + g, i.e. 16-byte chunk 2*st + g of the V^T rows.  The row sum is
    // taken on the exchanged registers (the two halves of a column together hold every key once).
    auto pack_probs = [&](f32x16 (&sacc)[2], u32x4 (&pf)[4], float &rs) __attribute__((always_inline)) {
        rs = 0.f;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int kt = st >> 1, j = st & 1;
            uint32_t w0 = AttnT<DT>::pack_only(sacc[kt][8 * j + 0], sacc[kt][8 * j + 1]);
            uint32_t w1 = AttnT<DT>::pack_only(sacc[kt][8 * j + 2], sacc[kt][8 * j + 3]);
            uint32_t w2 = AttnT<DT>::pack_only(sacc[kt][8 * j + 4], sacc[kt][8 * j + 5]);
            uint32_t w3 = AttnT<DT>::pack_only(sacc[kt][8 * j + 6], sacc[kt][8 * j + 7]);
            if constexpr (PERM) {
                // V^T comes with its keys in the accumulators' order (AttnParams::vt_perm): chunk 2*st + g of its rows
                // holds exactly the eight keys this lane half has just packed
                pf[st][0] = w0, pf[st][1] = w1, pf[st][2] = w2, pf[st][3] = w3;
            } else {
                auto x0 = __builtin_amdgcn_permlane32_swap(w0, w2, false, false);
                auto x1 = __builtin_amdgcn_permlane32_swap(w1, w3, false, false);
                pf[st][0] = x0[0], pf[st][1] = x1[0], pf[st][2] = x0[1], pf[st][3] = x1[1];
            }
#pragma unroll
            for (int e = 0; e < 4; ++e)
                AttnT<DT>::add_packed(pf[st][e], rs);
        }
    };
    // O^T += V^T P^T and the row sum
    auto accumulate = [&](const unsigned char *vtbuf, u32x4 (&pf)[4], float rs, float alpha) __attribute__((always_inline)) {
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const u32x4 vf = *reinterpret_cast<const u32x4 *>(vtbuf + dt * 32 * 128 + frag_off[st]);
                AttnT<DT>::mma(vf, pf[st], oacc[dt]);
            }
        rs  = half_swap_sum(rs);
        l_i = fmaf(l_i, alpha, rs);
    };
    // skip_half0 (wave-uniform): the first 32 keys of the tile are already in O and l (the FAST loop gave the tile up
    // between its halves); their scores are replaced by -inf, so they take no part in the maximum and add nothing
    auto general_tile = [&](auto mode_tag, int t, bool skip_half0) __attribute__((always_inline)) {
        constexpr int MODE = decltype(mode_tag)::value;  // 0 BIAS, 1 EXACT
        const unsigned char *const kbuf  = lds_all + stage * kStage;
        const unsigned char *const vtbuf = kbuf + kTile;
        const int kv0 = t * kTileKV;
        f32x16 sacc[2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                sacc[kt][r] = 0.f;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                u32x4 kf = *reinterpret_cast<const u32x4 *>(kbuf + kt * 32 * 128 + frag_off[kk]);
                AttnT<DT>::mma(kf, qf[kk], sacc[kt]);
            }
        }
        if (skip_half0) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                sacc[0][r] = -INFINITY;
        }
        float mx = -INFINITY;
        if (MODE == 0) {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int key0 = kt * 32 + r4 * 8 + g * 4;
                    // without a mask the three bias rows hold zeros (written once above), so no branch is needed and
                    // the eight reads of a tile go out together
                    const float4 raw = *reinterpret_cast<const float4 *>(&lds_bias[stage][key0]);
                    const float bv[4] = {raw.x * kLog2e, raw.y * kLog2e, raw.z * kLog2e, raw.w * kLog2e};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float be       = kv0 + key0 + e < kv_end ? bv[e] : -INFINITY;
                        float s2             = sacc[kt][r4 * 4 + e] + be;
                        sacc[kt][r4 * 4 + e] = s2;
                        mx                   = fmaxf(mx, s2);
                    }
                }
            }
        } else {
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    mx = fmaxf(mx, sacc[kt][r]);
        }
        mx          = half_swap_max(mx);
        float m_new = fmaxf(m_i, mx);
        float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        float alpha = __builtin_amdgcn_exp2f(m_i - m_use);
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                sacc[kt][r] = __builtin_amdgcn_exp2f(sacc[kt][r] - m_use);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                oacc[dt][r] *= alpha;
        m_i = m_new;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            negm[r] = -m_new;
        // the sixteen registers stay a block of their own (the MFMA reads them as its C operand); without this the
        // compiler keeps one copy and rebuilds the block in front of every tile
        asm volatile("" : "+v"(negm));
        u32x4 pf[4];
        float rs;
        pack_probs(sacc, pf, rs);
        accumulate(vtbuf, pf, rs, alpha);
    };

    // A quarter of that (four accumulator registers: four exponentials, two packs, two additions to the row sum), for
    // the key order in which the packed pairs need no exchange between the lane halves.  Register 4k + i of block kt is
    // element 2*(k&1) + i/2 of the operand of P.V step 2*kt + k/2.
    auto fast_quarter = [&](auto kt_tag, auto k_tag, f32x16 &sk, u32x4 (&pf)[4], float &rs) __attribute__((always_inline)) {
        constexpr int kt = decltype(kt_tag)::value, k = decltype(k_tag)::value;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            sk[4 * k + i] = __builtin_amdgcn_exp2f(sk[4 * k + i]);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t w = AttnT<DT>::pack_only(sk[4 * k + 2 * h], sk[4 * k + 2 * h + 1]);
            pf[2 * kt + (k >> 1)][2 * (k & 1) + h] = w;
            AttnT<DT>::add_packed(w, rs);
        }
    };
    // One half (32 keys, accumulator block kt) of a FAST tile: exponentials, packed operands of the two P.V steps the
    // half feeds, and this lane's part of the row sum.
    auto fast_half = [&](auto kt_tag, f32x16 &sk, u32x4 (&pf)[4], float &rs) __attribute__((always_inline)) {
        constexpr int kt = decltype(kt_tag)::value;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            sk[r] = __builtin_amdgcn_exp2f(sk[r]);
        rs = 0.f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int st = 2 * kt + j;
            uint32_t w0 = AttnT<DT>::pack_only(sk[8 * j + 0], sk[8 * j + 1]);
            uint32_t w1 = AttnT<DT>::pack_only(sk[8 * j + 2], sk[8 * j + 3]);
            uint32_t w2 = AttnT<DT>::pack_only(sk[8 * j + 4], sk[8 * j + 5]);
            uint32_t w3 = AttnT<DT>::pack_only(sk[8 * j + 6], sk[8 * j + 7]);
            if constexpr (PERM) {
                pf[st][0] = w0, pf[st][1] = w1, pf[st][2] = w2, pf[st][3] = w3;
            } else {
                auto x0 = __builtin_amdgcn_permlane32_swap(w0, w2, false, false);
                auto x1 = __builtin_amdgcn_permlane32_swap(w1, w3, false, false);
                pf[st][0] = x0[0], pf[st][1] = x1[0], pf[st][2] = x0[1], pf[st][3] = x1[1];
            }
#pragma unroll
            for (int e = 0; e < 4; ++e)
                AttnT<DT>::add_packed(pf[st][e], rs);
        }
    };
    // the two P.V steps of half kt
    auto pv_half = [&](auto kt_tag, const unsigned char *vtbuf, u32x4 (&pf)[4]) __attribute__((always_inline)) {
        constexpr int kt = decltype(kt_tag)::value;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int dt = 0; dt < 2; ++dt) {
                const u32x4 vf = *reinterpret_cast<const u32x4 *>(vtbuf + dt * 32 * 128 + frag_off[2 * kt + j]);
                AttnT<DT>::mma(vf, pf[2 * kt + j], oacc[dt]);
            }
    };

    int t = 0;
    bool entered = false;  // the FAST loop gave tile t up after entering it: the barrier of tile t is already behind us
    bool half0_done = false;  // ... and after its first 32 keys had gone into O and l
    while (t < n_tiles) {
        if (!entered)
            enter_tile(t);
        entered = false;
        if (mb != nullptr || (t + 1) * kTileKV > kv_end)  // workgroup-uniform
            general_tile(std::integral_constant<int, 0>(), t, false);
        else
            general_tile(std::integral_constant<int, 1>(), t, half0_done);
        half0_done = false;
        leave_tile();
        ++t;
        if (mb != nullptr || !__all(m_i > -INFINITY))  // per wave: FAST needs a finite reference
            continue;
        // FAST tiles.  On one SIMD the matrix pipe and the vector ALU overlap only for independent instruction streams
        // of one wave, and a tile as a whole is a dependent chain (scores -> exponentials -> P.V).  Its two 32-key
        // halves are independent of each other, though, so they are skewed by one step:
        //     scores 0 | scores 1 under the exponentials of half 0 | P.V 0 under the exponentials of half 1 | P.V 1
        // with eight vector instructions behind each MFMA.  The reference is checked per half, before the half's P.V
        // step is issued.
        while (t < n_tiles && (t + 1) * kTileKV <= kv_end) {
            enter_tile(t);
            const unsigned char *const kbuf  = lds_all + stage * kStage;
            const unsigned char *const vtbuf = kbuf + kTile;
            u32x4 pf[4];
            float rs0 = 0.f, rs1 = 0.f;
            f32x16 sacc[2];
            if constexpr (PERM) {
                // The issue order is written out: a fence (nothing may be moved across it by the compiler) after every
                // MFMA-plus-eight-vector-instructions step.
                u32x4 kf[2][4];
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk)
                        kf[kt][kk] = *reinterpret_cast<const u32x4 *>(kbuf + kt * 32 * 128 + frag_off[kk]);
                sacc[0] = AttnT<DT>::mma_from(kf[0][0], qf[0], negm);
#pragma unroll
                for (int kk = 1; kk < 4; ++kk)
                    AttnT<DT>::mma(kf[0][kk], qf[kk], sacc[0]);
                __builtin_amdgcn_sched_barrier(0);
                sacc[1] = AttnT<DT>::mma_from(kf[1][0], qf[0], negm);
                fast_quarter(std::integral_constant<int, 0>(), std::integral_constant<int, 0>(), sacc[0], pf, rs0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kk = 1; kk < 4; ++kk) {
                    AttnT<DT>::mma(kf[1][kk], qf[kk], sacc[1]);
                    if (kk == 1)
                        fast_quarter(std::integral_constant<int, 0>(), std::integral_constant<int, 1>(), sacc[0], pf, rs0);
                    else if (kk == 2)
                        fast_quarter(std::integral_constant<int, 0>(), std::integral_constant<int, 2>(), sacc[0], pf, rs0);
                    else
                        fast_quarter(std::integral_constant<int, 0>(), std::integral_constant<int, 3>(), sacc[0], pf, rs0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    u32x4 kf = *reinterpret_cast<const u32x4 *>(kbuf + kt * 32 * 128 + frag_off[0]);
                    sacc[kt] = AttnT<DT>::mma_from(kf, qf[0], negm);
#pragma unroll
                    for (int kk = 1; kk < 4; ++kk) {
                        kf = *reinterpret_cast<const u32x4 *>(kbuf + kt * 32 * 128 + frag_off[kk]);
                        AttnT<DT>::mma(kf, qf[kk], sacc[kt]);
                    }
                }
                fast_half(std::integral_constant<int, 0>(), sacc[0], pf, rs0);
            }
            if (__builtin_expect(__any(!(rs0 <= kStaleLimit)), 0)) {
                entered = true;
                break;
            }
            if constexpr (PERM) {
                u32x4 vf[2][2];
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int dt = 0; dt < 2; ++dt)
                        vf[j][dt] = *reinterpret_cast<const u32x4 *>(vtbuf + dt * 32 * 128 + frag_off[j]);
                __builtin_amdgcn_sched_barrier(0);
                AttnT<DT>::mma(vf[0][0], pf[0], oacc[0]);
                fast_quarter(std::integral_constant<int, 1>(), std::integral_constant<int, 0>(), sacc[1], pf, rs1);
                __builtin_amdgcn_sched_barrier(0);
                AttnT<DT>::mma(vf[0][1], pf[0], oacc[1]);
                fast_quarter(std::integral_constant<int, 1>(), std::integral_constant<int, 1>(), sacc[1], pf, rs1);
                __builtin_amdgcn_sched_barrier(0);
                AttnT<DT>::mma(vf[1][0], pf[1], oacc[0]);
                fast_quarter(std::integral_constant<int, 1>(), std::integral_constant<int, 2>(), sacc[1], pf, rs1);
                __builtin_amdgcn_sched_barrier(0);
                AttnT<DT>::mma(vf[1][1], pf[1], oacc[1]);
                fast_quarter(std::integral_constant<int, 1>(), std::integral_constant<int, 3>(), sacc[1], pf, rs1);
                __builtin_amdgcn_sched_barrier(0);
            } else {
                pv_half(std::integral_constant<int, 0>(), vtbuf, pf);
                fast_half(std::integral_constant<int, 1>(), sacc[1], pf, rs1);
            }
            if (__builtin_expect(__any(!(rs1 <= kStaleLimit)), 0)) {
                l_i += half_swap_sum(rs0);
                entered    = true;
                half0_done = true;
                break;
            }
            pv_half(std::integral_constant<int, 1>(), vtbuf, pf);
            l_i += half_swap_sum(rs0 + rs1);
            leave_tile();
            ++t;
        }
    }

    // ---- normalise and store (see attention_kernel)
    __syncthreads();
    {
        unsigned char *const stg = lds_all + wave * 32 * kRowBytes;
        const float inv          = l_i > 0.f ? 1.0f / l_i : 0.f;
#pragma unroll
        for (int dt = 0; dt < 2; ++dt)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                u32x2 w;
                w[0] = AttnT<DT>::pack2(oacc[dt][r4 * 4 + 0] * inv, oacc[dt][r4 * 4 + 1] * inv);
                w[1] = AttnT<DT>::pack2(oacc[dt][r4 * 4 + 2] * inv, oacc[dt][r4 * 4 + 3] * inv);
                *reinterpret_cast<u32x2 *>(stg + lq * kRowBytes + (dt * 32 + r4 * 8 + g * 4) * 2) = w;
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int r    = pass * 8 + (lane >> 3);
            const int qrow = q0 + r;
            if (qrow < S) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(stg + r * kRowBytes + (lane & 7) * 16);
                store_out16(ob + (size_t)qrow * p.o_ss + (lane & 7) * 8, v);
                if (p.oq) {
                    u32x2 q8;
#pragma unroll
                    for (int w = 0; w < 2; ++w) {
                        uint32_t packed = 0;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const uint32_t word = v[w * 2 + (e >> 1)];
                            const float f       = AttnT<DT>::to_float((uint16_t)(e & 1 ? word >> 16 : word & 0xffffu));
                            packed |= (uint32_t)(uint8_t)float2int8_ref(__fmul_rn(f, p.q_inv)) << (8 * e);
                        }
                        q8[w] = packed;
                    }
                    int8_t *oqb = p.oq + (size_t)b * p.o_sb + (size_t)head * p.o_sh;
                    store_out8(oqb + (size_t)qrow * p.o_ss + (lane & 7) * 8, q8);
                }
            }
        }
    }
}

// One wave per batch row, two passes over it (the second finds the row in cache): the row's largest value, then the
// largest index whose mask value is above (largest value + threshold) and the smallest index whose value is not
// exactly zero.  The cut is relative to the row's maximum because softmax is: a key whose bias lies `threshold` (a
// large negative number) below the best key's contributes exp(threshold + score difference) = 0 in fp32, whatever
// constant the whole row carries.  Row b is read at mask + b * src_stride (0: one row serves every sequence); with
// mask_f32 given, the row is also written there in fp32, densely (what the attention kernels read).
template <int DT>
__global__ void mask_to_kv_len_kernel(const typename Elem<DT>::type *__restrict__ mask, long src_stride,
                                      float *__restrict__ mask_f32, int32_t *__restrict__ kv_len, int S, float threshold,
                                      int flag_zero_rows) {
    const int b    = blockIdx.x;
    const int lane = threadIdx.x;
    const typename Elem<DT>::type *row = mask + (size_t)b * src_stride;
    float top = -INFINITY;
    for (int j = lane; j < S; j += 64) {
        const float v = Elem<DT>::ld(&row[j]);
        if (mask_f32)
            mask_f32[(size_t)b * S + j] = v;
        top = v > top ? v : top;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float other = __shfl_xor(top, o, 64);
        top               = other > top ? other : top;
    }
    const float cut = top + threshold;
    int last = -1, first_nonzero = S;
    for (int j = lane; j < S; j += 64) {
        const float v = Elem<DT>::ld(&row[j]);
        if (v > cut)
            last = j;
        if (v != 0.0f && j < first_nonzero)
            first_nonzero = j;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const int other = __shfl_xor(last, o, 64), other_nz = __shfl_xor(first_nonzero, o, 64);
        last            = other > last ? other : last;
        first_nonzero   = other_nz < first_nonzero ? other_nz : first_nonzero;
    }
    // No key above the cut (a row of -inf or NaN only): the reference still runs softmax(scores + mask) over all S
    // keys, so every key stays in, with its bias.  A row that masks every key with the same finite value keeps all
    // its keys by the rule itself: each one is the row's maximum.
    int len = last < 0 ? S : last + 1;
    // a plain padding mask is exactly 0 on every visible key: the attention kernel then needs the length only
    if (flag_zero_rows && first_nonzero >= len)
        len |= kKvLenMaskZero;
    if (lane == 0)
        kv_len[b] = len;
}

// 128-row query blocks when that already gives >= 2 workgroups per CU, else 64-row blocks
std::atomic<int> g_attention_dma{1};  // experiment hook: 0 keeps the register-staged kernel for the V^T layout as well

template <bool VT> int launch_attention(hipStream_t s, int dtype, const AttnParams &p, int B, int heads, int S) {
    long blocks128 = (long)((S + 127) / 128) * heads * B;
    auto padded = [&](long n_q) { return dim3((unsigned)(((n_q * heads * B + 7) / 8) * 8)); };
    if (VT && g_attention_dma) {
#define TR_LAUNCH_DMA(NWv, THREADS)                                                                                   \
    do {                                                                                                              \
        if (dtype == TNN_ROCM_F16 && p.vt_perm)                                                                       \
            hipLaunchKernelGGL((attention_dma_kernel<TNN_ROCM_F16, NWv, true>), grid, dim3(THREADS), 0, s, p);        \
        else if (dtype == TNN_ROCM_F16)                                                                               \
            hipLaunchKernelGGL((attention_dma_kernel<TNN_ROCM_F16, NWv, false>), grid, dim3(THREADS), 0, s, p);       \
        else if (p.vt_perm)                                                                                           \
            hipLaunchKernelGGL((attention_dma_kernel<TNN_ROCM_BF16, NWv, true>), grid, dim3(THREADS), 0, s, p);       \
        else                                                                                                          \
            hipLaunchKernelGGL((attention_dma_kernel<TNN_ROCM_BF16, NWv, false>), grid, dim3(THREADS), 0, s, p);      \
    } while (0)
        if (blocks128 >= 512) {
            dim3 grid = padded((S + 127) / 128);
            TR_LAUNCH_DMA(4, 256);
        } else {
            dim3 grid = padded((S + 63) / 64);
            TR_LAUNCH_DMA(2, 128);
        }
#undef TR_LAUNCH_DMA
        TR_CHECK_LAUNCH();
        return 0;
    }
    if (blocks128 >= 512) {
        dim3 grid = padded((S + 127) / 128);
        if (dtype == TNN_ROCM_F16)
            hipLaunchKernelGGL((attention_kernel<TNN_ROCM_F16, 4, VT>), grid, dim3(256), 0, s, p);
        else
            hipLaunchKernelGGL((attention_kernel<TNN_ROCM_BF16, 4, VT>), grid, dim3(256), 0, s, p);
    } else {
        dim3 grid = padded((S + 63) / 64);
        if (dtype == TNN_ROCM_F16)
            hipLaunchKernelGGL((attention_kernel<TNN_ROCM_F16, 2, VT>), grid, dim3(128), 0, s, p);
        else
            hipLaunchKernelGGL((attention_kernel<TNN_ROCM_BF16, 2, VT>), grid, dim3(128), 0, s, p);
    }
    TR_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" {

int tnn_rocm_attention(void *stream, int dtype, const void *q, const void *k, const void *v, void *out, int B,
                       int heads, int S, int head_dim, long q_sb, long q_sh, long q_ss, long kv_sb, long kv_sh,
                       long kv_ss, long o_sb, long o_sh, long o_ss, float scale, const float *mask,
                       const int32_t *kv_len) {
    TR_REQUIRE(B >= 0 && heads >= 0 && S >= 0, TNN_ROCM_ESHAPE, "attention: negative size");
    if (B == 0 || heads == 0 || S == 0)
        return 0;
    TR_REQUIRE(q && k && v && out, TNN_ROCM_EINVAL, "attention: null pointer");
    TR_REQUIRE(head_dim == kD, TNN_ROCM_ESHAPE, "attention: head_dim %d unsupported (64 only)", head_dim);
    TR_REQUIRE(dtype == TNN_ROCM_F16 || dtype == TNN_ROCM_BF16, TNN_ROCM_EDTYPE,
               "attention: dtype %d unsupported (F16 or BF16)", dtype);
    TR_REQUIRE(B <= 65535 && heads <= 65535, TNN_ROCM_ESHAPE, "attention: batch/heads exceed the grid limit");
    auto ok = [](const void *ptr, long a, long b2, long c) {
        return ((((uintptr_t)ptr) & 15u) == 0) && a % 8 == 0 && b2 % 8 == 0 && c % 8 == 0;
    };
    TR_REQUIRE(ok(q, q_sb, q_sh, q_ss) && ok(k, kv_sb, kv_sh, kv_ss) && ok(v, kv_sb, kv_sh, kv_ss) &&
                   ok(out, o_sb, o_sh, o_ss),
               TNN_ROCM_EALIGN, "attention: pointers must be 16-byte aligned and strides multiples of 8 elements");
    TR_REQUIRE(q_ss >= kD && kv_ss >= kD && o_ss >= kD, TNN_ROCM_ESHAPE, "attention: row stride below head_dim");
    TR_REQUIRE((long)S * kv_ss < (1l << 31), TNN_ROCM_ESHAPE, "attention: S * row stride exceeds 32-bit tile offsets");
    AttnParams p;
    p.q = (const uint16_t *)q;
    p.k = (const uint16_t *)k;
    p.v = (const uint16_t *)v;
    p.o = (uint16_t *)out;
    p.q_sb = q_sb, p.q_sh = q_sh, p.q_ss = q_ss;
    p.kv_sb = kv_sb, p.kv_sh = kv_sh, p.kv_ss = kv_ss;
    p.o_sb = o_sb, p.o_sh = o_sh, p.o_ss = o_ss;
    p.S           = S;
    p.B           = B;
    p.heads       = heads;
    p.scale_log2e = scale * kLog2e;
    p.mask        = mask;
    p.kv_len      = kv_len;
    p.vt_sb = p.vt_sh = p.vt_sd = 0;
    p.oq      = nullptr;
    p.q_inv   = 0.f;
    p.vt_perm = 0;
    return launch_attention<false>((hipStream_t)stream, dtype, p, B, heads, S);
}

int tnn_rocm_attention_vt(void *stream, int dtype, const void *q, const void *k, const void *vt, void *out, int B,
                          int heads, int S, int head_dim, long q_sb, long q_sh, long q_ss, long k_sb, long k_sh,
                          long k_ss, long vt_sb, long vt_sh, long vt_sd, long o_sb, long o_sh, long o_ss, float scale,
                          const float *mask, const int32_t *kv_len) {
    return tnn_rocm_attention_vt_q8(stream, dtype, q, k, vt, out, nullptr, 0.f, B, heads, S, head_dim, q_sb, q_sh, q_ss, k_sb,
                                    k_sh, k_ss, vt_sb, vt_sh, vt_sd, o_sb, o_sh, o_ss, scale, mask, kv_len, 0);
}

int tnn_rocm_attention_vt_q8(void *stream, int dtype, const void *q, const void *k, const void *vt, void *out,
                             int8_t *out_q, float out_q_inv_scale, int B, int heads, int S, int head_dim, long q_sb,
                             long q_sh, long q_ss, long k_sb, long k_sh, long k_ss, long vt_sb, long vt_sh, long vt_sd,
                             long o_sb, long o_sh, long o_ss, float scale, const float *mask, const int32_t *kv_len,
                             int vt_key_order) {
    TR_REQUIRE(B >= 0 && heads >= 0 && S >= 0, TNN_ROCM_ESHAPE, "attention_vt: negative size");
    TR_REQUIRE(vt_key_order == 0 || (vt_key_order == 1 && S % 16 == 0), TNN_ROCM_EINVAL,
               "attention_vt: V^T key order %d (0 natural, 1 accumulator order, which needs S %% 16 == 0; S=%d)", vt_key_order, S);
    if (B == 0 || heads == 0 || S == 0)
        return 0;
    TR_REQUIRE(q && k && vt && out, TNN_ROCM_EINVAL, "attention_vt: null pointer");
    TR_REQUIRE(head_dim == kD, TNN_ROCM_ESHAPE, "attention_vt: head_dim %d unsupported (64 only)", head_dim);
    TR_REQUIRE(dtype == TNN_ROCM_F16 || dtype == TNN_ROCM_BF16, TNN_ROCM_EDTYPE,
               "attention_vt: dtype %d unsupported (F16 or BF16)", dtype);
    TR_REQUIRE(B <= 65535 && heads <= 65535, TNN_ROCM_ESHAPE, "attention_vt: batch/heads exceed the grid limit");
    TR_REQUIRE(S % 8 == 0, TNN_ROCM_ESHAPE, "attention_vt: S=%d must be a multiple of 8 (16-byte V^T vectors)", S);
    auto ok = [](const void *ptr, long a, long b2, long c) {
        return ((((uintptr_t)ptr) & 15u) == 0) && a % 8 == 0 && b2 % 8 == 0 && c % 8 == 0;
    };
    TR_REQUIRE(ok(q, q_sb, q_sh, q_ss) && ok(k, k_sb, k_sh, k_ss) && ok(vt, vt_sb, vt_sh, vt_sd) &&
                   ok(out, o_sb, o_sh, o_ss),
               TNN_ROCM_EALIGN, "attention_vt: pointers must be 16-byte aligned and strides multiples of 8 elements");
    TR_REQUIRE(q_ss >= kD && k_ss >= kD && o_ss >= kD && vt_sd >= S, TNN_ROCM_ESHAPE, "attention_vt: stride too small");
    TR_REQUIRE((long)S * k_ss < (1l << 31) && (long)kD * vt_sd + S < (1l << 31), TNN_ROCM_ESHAPE,
               "attention_vt: per-head extent exceeds 32-bit tile offsets");
    AttnParams p;
    p.q = (const uint16_t *)q;
    p.k = (const uint16_t *)k;
    p.v = (const uint16_t *)vt;
    p.o = (uint16_t *)out;
    p.q_sb = q_sb, p.q_sh = q_sh, p.q_ss = q_ss;
    p.kv_sb = k_sb, p.kv_sh = k_sh, p.kv_ss = k_ss;
    p.vt_sb = vt_sb, p.vt_sh = vt_sh, p.vt_sd = vt_sd;
    p.o_sb = o_sb, p.o_sh = o_sh, p.o_ss = o_ss;
    p.S           = S;
    p.B           = B;
    p.heads       = heads;
    p.scale_log2e = scale * kLog2e;
    p.mask        = mask;
    p.kv_len      = kv_len;
    TR_REQUIRE(!out_q || (((uintptr_t)out_q) & 7u) == 0, TNN_ROCM_EALIGN, "attention_vt: int8 output must be 8-byte aligned");
    p.oq      = out_q;
    p.q_inv   = out_q_inv_scale;
    p.vt_perm = vt_key_order;
    return launch_attention<true>((hipStream_t)stream, dtype, p, B, heads, S);
}

TR_DEFINE_STORE_THROUGH_SETTER(attention_set_store_through)
__attribute__((visibility("default"))) int tnn_rocm_debug_set_attention_dma(int on) {
    g_attention_dma = on;
    return 0;
}

int tnn_rocm_mask_to_kv_len(void *stream, const float *mask, int32_t *kv_len, int B, int S, float threshold) {
    TR_REQUIRE(B >= 0 && S >= 0, TNN_ROCM_ESHAPE, "mask_to_kv_len: negative size");
    if (B == 0)
        return 0;
    TR_REQUIRE(mask && kv_len, TNN_ROCM_EINVAL, "mask_to_kv_len: null pointer");
    hipLaunchKernelGGL(mask_to_kv_len_kernel<TNN_ROCM_F32>, dim3(B), dim3(64), 0, (hipStream_t)stream, mask, (long)S, nullptr,
                       kv_len, S, threshold, 0);
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_mask_to_kv_len_flagged(void *stream, const float *mask, int32_t *kv_len, int B, int S, float threshold) {
    return tnn_rocm_mask_prepare(stream, TNN_ROCM_F32, mask, nullptr, kv_len, B, S, threshold);
}

int tnn_rocm_mask_prepare_strided(void *stream, int dtype, const void *mask, long mask_batch_stride, float *mask_f32,
                                  int32_t *kv_len, int B, int S, float threshold) {
    TR_REQUIRE(B >= 0 && S >= 0 && S < kKvLenMaskZero, TNN_ROCM_ESHAPE, "mask_prepare: bad size");
    TR_REQUIRE(mask_batch_stride == 0 || mask_batch_stride >= S, TNN_ROCM_ESHAPE, "mask_prepare: batch stride %ld below S",
               mask_batch_stride);
    if (B == 0)
        return 0;
    TR_REQUIRE(mask && kv_len, TNN_ROCM_EINVAL, "mask_prepare: null pointer");
    TR_REQUIRE((dtype == TNN_ROCM_F32 && mask_batch_stride == S) || mask_f32, TNN_ROCM_EINVAL,
               "mask_prepare: a half-precision or strided mask needs the fp32 buffer");
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case TNN_ROCM_F32:
            hipLaunchKernelGGL(mask_to_kv_len_kernel<TNN_ROCM_F32>, dim3(B), dim3(64), 0, s, (const float *)mask,
                               mask_batch_stride, mask_f32, kv_len, S, threshold, 1);
            break;
        case TNN_ROCM_F16:
            hipLaunchKernelGGL(mask_to_kv_len_kernel<TNN_ROCM_F16>, dim3(B), dim3(64), 0, s, (const half_t *)mask,
                               mask_batch_stride, mask_f32, kv_len, S, threshold, 1);
            break;
        case TNN_ROCM_BF16:
            hipLaunchKernelGGL(mask_to_kv_len_kernel<TNN_ROCM_BF16>, dim3(B), dim3(64), 0, s, (const bf16_bits *)mask,
                               mask_batch_stride, mask_f32, kv_len, S, threshold, 1);
            break;
        default:
            TR_REQUIRE(false, TNN_ROCM_EDTYPE, "mask_prepare: dtype %d unsupported", dtype);
    }
    TR_CHECK_LAUNCH();
    return 0;
}

int tnn_rocm_mask_prepare(void *stream, int dtype, const void *mask, float *mask_f32, int32_t *kv_len, int B, int S,
                          float threshold) {
    // an fp32 mask is used where it lies: no copy
    return tnn_rocm_mask_prepare_strided(stream, dtype, mask, (long)S, dtype == TNN_ROCM_F32 ? nullptr : mask_f32, kv_len, B, S,
                                         threshold);
}

}  // extern "C"
