// Stand-alone micro-benchmark of one gfx950 SIMD: how the matrix pipe (MFMA), the vector ALU and the operand reads
// from LDS share a SIMD's time.  It is the evidence behind the ceilings quoted for the attention kernel and the GEMM
// main loop; nothing in the library uses it.
//
//   hipcc --offload-arch=gfx950 -O3 -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops \
//         tnn_amd/csrc/probe_simd.hip -o tnn_amd/lib/probe_simd && tnn_amd/lib/probe_simd
//
// One "tile" is what a wave of the attention kernel does per 64-key tile of a 32-query block at head size 64:
//   8 score MFMAs (two dependent chains of four, 32x32x16 f16), 32 v_exp_f32, 16 packs to half precision, 16 dot2 for
//   the row sum, 8 lane-half swaps, 8 MFMAs for P.V (two accumulators), and sixteen 16-byte-per-lane fragment reads
//   from LDS (conflict-free: the kernel's XOR swizzle).
// Variants:
//   mfma      the 16 MFMAs alone                      valu      the vector work alone (on independent registers)
//   chain     MFMAs + vector work, dependent as in the kernel, operands from registers
//   lds       the sixteen fragment reads alone
//   tile      chain + fragment reads feeding the MFMAs (the whole tile)
//   ahead     tile with every fragment requested before the first MFMA that needs one (latency taken out)
//   pipe      the same instruction counts as chain, software-pipelined inside ONE wave: while the vector work of tile i
//             runs, the matrix pipe is given the score MFMAs of tile i + 1 and the P.V MFMAs of tile i - 1, all on
//             registers the vector work does not touch (one MFMA, then four vector instructions, sixteen times per
//             tile; two register sets, the loop unrolled twice so that no set is copied).  Operands from registers.
//   pipe+lds  pipe with the sixteen fragment reads of the MFMAs it issues, requested one group ahead
//   skew      the overlap available INSIDE one tile, no state carried between tiles: the two 32-key halves are skewed
//             by one step -- scores of half 0 | scores of half 1 under the vector work of half 0 | P.V of half 0 under
//             the vector work of half 1 | P.V of half 1.  Same instruction counts as chain, operands from registers.
//   skew+lds  skew with the fragment reads from LDS
// Each is run with 1, 2 and 3 waves per SIMD (256 x k workgroups of four waves, one wave per SIMD each) and reported
// as nanoseconds per tile and SIMD, i.e. the time divided by the waves per SIMD.
// A second table gives the matrix rate the whole chip sustains: one wave per SIMD that issues nothing but independent
// MFMAs (sixteen accumulators, eight operand fragments loaded once), about a millisecond per launch, with operands that
// are all zero, all one, or normally distributed.  The power the matrix pipe draws depends on the operand bits, and the
// clock follows the power: that rate, not the data-sheet figure, is what a GEMM main loop can be held against.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

enum { MFMA_ONLY, VALU_ONLY, CHAIN, LDS_ONLY, TILE, TILE_AHEAD, PIPE, PIPE_LDS, SKEW, SKEW_LDS };

template <int MODE> __global__ void __launch_bounds__(256) probe(float *out, int iters, float seed) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[32768];
    for (int i = threadIdx.x; i < 8192; i += 256)
        ((float *)lds)[i] = seed * 1e-3f * (i & 15);
    __syncthreads();
    const unsigned lq = threadIdx.x & 31, g = (threadIdx.x >> 5) & 1;
    unsigned fo[4];  // fragment chunk 2x + g of row lq, chunk positions XOR-swizzled by the row
    for (int x = 0; x < 4; ++x)
        fo[x] = lq * 128 + (((2 * x + g) ^ ((lq >> 1) & 7)) * 16);
    f32x16 o0, o1, s0, s1, z;
    for (int r = 0; r < 16; ++r)
        o0[r] = 0.f, o1[r] = 0.f, z[r] = -seed;
    f16x8 kreg, q;
    for (int r = 0; r < 8; ++r)
        kreg[r] = (_Float16)(seed * 0.01f + r * 0.001f), q[r] = (_Float16)(seed * 0.02f - r * 0.001f);
    float ind[32];
    for (int r = 0; r < 32; ++r)
        ind[r] = seed * 0.001f * r;
    float rs          = 0.f;
    const f16x2 ones  = {(_Float16)1.0f, (_Float16)1.0f};
    constexpr bool kMfma = MODE != VALU_ONLY && MODE != LDS_ONLY;
    constexpr bool kValu = MODE != MFMA_ONLY && MODE != LDS_ONLY;
    constexpr bool kLds  = MODE == LDS_ONLY || MODE == TILE || MODE == TILE_AHEAD;
    for (int i = 0; i < iters; ++i) {
        const unsigned char *kb = lds + (i & 1) * 16384, *vb = kb + 8192;
        if (MODE == LDS_ONLY) {
            u32x4 acc = {0, 0, 0, 0};
#pragma unroll
            for (int x = 0; x < 4; ++x)
#pragma unroll
                for (int part = 0; part < 4; ++part)
                    acc ^= *reinterpret_cast<const u32x4 *>(kb + part * 4096 + fo[x]);
            rs += __builtin_bit_cast(float, acc[0] ^ acc[1] ^ acc[2] ^ acc[3]);
            continue;
        }
        f16x8 kf[8], vf[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) {  // distinct values, so that no two MFMAs compute the same thing
            kf[x] = kreg, vf[x] = kreg;
            kf[x][x] = (_Float16)(float)(i + x);
            vf[x][7 - x] = (_Float16)(float)(i - x);
        }
        if (MODE == TILE_AHEAD) {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                kf[2 * x]     = *reinterpret_cast<const f16x8 *>(kb + fo[x]);
                kf[2 * x + 1] = *reinterpret_cast<const f16x8 *>(kb + 4096 + fo[x]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (kMfma) {
            s0 = z, s1 = z;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                if (MODE == TILE) {
                    kf[2 * x]     = *reinterpret_cast<const f16x8 *>(kb + fo[x]);
                    kf[2 * x + 1] = *reinterpret_cast<const f16x8 *>(kb + 4096 + fo[x]);
                }
                s0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[2 * x], q, s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[2 * x + 1], q, s1, 0, 0, 0);
            }
        }
        if (MODE == TILE_AHEAD) {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                vf[2 * x]     = *reinterpret_cast<const f16x8 *>(vb + fo[x]);
                vf[2 * x + 1] = *reinterpret_cast<const f16x8 *>(vb + 4096 + fo[x]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        u32x4 pf[4];
#pragma unroll
        for (int st = 0; st < 4; ++st)
            pf[st] = __builtin_bit_cast(u32x4, kreg);
        if (kValu) {
            if (MODE == VALU_ONLY) {  // the same instructions on registers no MFMA touches
#pragma unroll
                for (int r = 0; r < 32; ++r)
                    ind[r] = __builtin_amdgcn_exp2f(ind[r]);
#pragma unroll
                for (int st = 0; st < 4; ++st)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        pf[st][e] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(ind[st * 8 + 2 * e], ind[st * 8 + 2 * e + 1]));
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    s0[r] = __builtin_amdgcn_exp2f(s0[r]), s1[r] = __builtin_amdgcn_exp2f(s1[r]);
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    f32x16 &s = st < 2 ? s0 : s1;
                    const int j = st & 1;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        pf[st][e] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(s[8 * j + 2 * e], s[8 * j + 2 * e + 1]));
                }
            }
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                auto x0 = __builtin_amdgcn_permlane32_swap(pf[st][0], pf[st][2], false, false);
                auto x1 = __builtin_amdgcn_permlane32_swap(pf[st][1], pf[st][3], false, false);
                pf[st][0] = x0[0], pf[st][1] = x1[0], pf[st][2] = x0[1], pf[st][3] = x1[1];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    rs = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pf[st][e]), ones, rs, false);
            }
        }
        if (kMfma) {
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                if (MODE == TILE) {
                    vf[2 * st]     = *reinterpret_cast<const f16x8 *>(vb + fo[st]);
                    vf[2 * st + 1] = *reinterpret_cast<const f16x8 *>(vb + 4096 + fo[st]);
                }
                const f16x8 p = MODE == MFMA_ONLY ? q : __builtin_bit_cast(f16x8, pf[st]);
                o0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * st], p, o0, 0, 0, 0);
                o1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * st + 1], p, o1, 0, 0, 0);
            }
        } else {
            asm volatile("" ::"v"(pf[0]), "v"(pf[1]), "v"(pf[2]), "v"(pf[3]));
        }
        if (MODE == MFMA_ONLY)
            asm volatile("" ::"v"(s0), "v"(s1));  // the score MFMAs stay although nothing reads their result
        (void)kLds;
    }
    float t = rs;
    for (int r = 0; r < 16; ++r)
        t += o0[r] + o1[r];
    for (int r = 0; r < 32; ++r)
        t += ind[r];
    if (t == 12345.678f)
        out[0] = t;
}

// The pipelined variants.  Per tile and wave: 16 MFMAs (8 for the scores of the NEXT tile into s_next, 8 for P.V of the
// PREVIOUS tile from pf_prev into o0 / o1) and the 64 vector instructions of the CURRENT tile (32 exp2 on s_cur, 16
// packs into pf_cur, 16 dot2 for the row sum); nothing issued in one half depends on the other half within the tile.
// sched_group_barrier pins the order: one MFMA, four vector instructions, and so on.
template <bool WITH_LDS> __global__ void __launch_bounds__(256) probe_pipe(float *out, int iters, float seed) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[32768];
    for (int i = threadIdx.x; i < 8192; i += 256)
        ((float *)lds)[i] = seed * 1e-3f * (i & 15);
    __syncthreads();
    const unsigned lq = threadIdx.x & 31, g = (threadIdx.x >> 5) & 1;
    unsigned fo[4];
    for (int x = 0; x < 4; ++x)
        fo[x] = lq * 128 + (((2 * x + g) ^ ((lq >> 1) & 7)) * 16);
    f32x16 o0, o1, z, sa0, sa1, sb0, sb1;
    for (int r = 0; r < 16; ++r)
        o0[r] = 0.f, o1[r] = 0.f, z[r] = -seed, sa0[r] = seed * r, sa1[r] = -seed * r, sb0[r] = seed, sb1[r] = seed;
    f16x8 kreg, q;
    for (int r = 0; r < 8; ++r)
        kreg[r] = (_Float16)(seed * 0.01f + r * 0.001f), q[r] = (_Float16)(seed * 0.02f - r * 0.001f);
    u32x4 pa[4], pb[4];
    for (int st = 0; st < 4; ++st)
        pa[st] = __builtin_bit_cast(u32x4, kreg), pb[st] = __builtin_bit_cast(u32x4, kreg);
    float rs         = 0.f;
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    // one tile: vector work on (s0, s1) -> pf_cur; MFMAs: scores of the next tile -> (n0, n1), P.V of pf_prev -> o
    auto tile = [&](int i, f32x16 &s0, f32x16 &s1, f32x16 &n0, f32x16 &n1, u32x4 (&pf_prev)[4], u32x4 (&pf_cur)[4])
                    __attribute__((always_inline)) {
        const unsigned char *kb = lds + (i & 1) * 16384, *vb = kb + 8192;
        f16x8 kf[8], vf[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            if (WITH_LDS) {
                kf[x] = *reinterpret_cast<const f16x8 *>(kb + (x & 1) * 4096 + fo[x >> 1]);
                vf[x] = *reinterpret_cast<const f16x8 *>(vb + (x & 1) * 4096 + fo[x >> 1]);
            } else {
                kf[x] = kreg, vf[x] = kreg;
                kf[x][x] = (_Float16)(float)(i + x);
                vf[x][7 - x] = (_Float16)(float)(i - x);
            }
        }
        n0 = z, n1 = z;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            n0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[2 * x], q, n0, 0, 0, 0);
            n1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[2 * x + 1], q, n1, 0, 0, 0);
        }
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const f16x8 p = __builtin_bit_cast(f16x8, pf_prev[st]);
            o0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * st], p, o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * st + 1], p, o1, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r)
            s0[r] = __builtin_amdgcn_exp2f(s0[r]), s1[r] = __builtin_amdgcn_exp2f(s1[r]);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            f32x16 &s = st < 2 ? s0 : s1;
            const int j = st & 1;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                pf_cur[st][e] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(s[8 * j + 2 * e], s[8 * j + 2 * e + 1]));
                rs = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pf_cur[st][e]), ones, rs, false);
            }
        }
        // the issue order: (LDS reads first,) then one MFMA followed by four vector instructions, sixteen times
        if (WITH_LDS)
            __builtin_amdgcn_sched_group_barrier(0x100, 16, 0);  // DS reads
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // VALU
        }
    };
    for (int i = 0; i < iters; i += 2) {
        tile(i, sa0, sa1, sb0, sb1, pb, pa);      // vector work on set a; scores into set b; P.V from the pairs of b
        tile(i + 1, sb0, sb1, sa0, sa1, pa, pb);  // and the other way round
    }
    float t = rs;
    for (int r = 0; r < 16; ++r)
        t += o0[r] + o1[r] + sa0[r] + sb0[r] + sa1[r] + sb1[r];
    if (t == 12345.678f)
        out[0] = t;
}

// Half-tile skew: see the variant list at the top.
template <bool WITH_LDS> __global__ void __launch_bounds__(256) probe_skew(float *out, int iters, float seed) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[32768];
    for (int i = threadIdx.x; i < 8192; i += 256)
        ((float *)lds)[i] = seed * 1e-3f * (i & 15);
    __syncthreads();
    const unsigned lq = threadIdx.x & 31, g = (threadIdx.x >> 5) & 1;
    unsigned fo[4];
    for (int x = 0; x < 4; ++x)
        fo[x] = lq * 128 + (((2 * x + g) ^ ((lq >> 1) & 7)) * 16);
    f32x16 o0, o1, z, s0, s1;
    for (int r = 0; r < 16; ++r)
        o0[r] = 0.f, o1[r] = 0.f, z[r] = -seed;
    f16x8 kreg, q;
    for (int r = 0; r < 8; ++r)
        kreg[r] = (_Float16)(seed * 0.01f + r * 0.001f), q[r] = (_Float16)(seed * 0.02f - r * 0.001f);
    float rs         = 0.f;
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    for (int i = 0; i < iters; ++i) {
        const unsigned char *kb = lds + (i & 1) * 16384, *vb = kb + 8192;
        f16x8 kf[8], vf[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            if (WITH_LDS) {
                kf[x] = *reinterpret_cast<const f16x8 *>(kb + (x >> 2) * 4096 + fo[x & 3]);   // half x/4, k-step x%4
                vf[x] = *reinterpret_cast<const f16x8 *>(vb + (x & 1) * 4096 + fo[x >> 1]);   // step x/2, d block x%2
            } else {
                kf[x] = kreg, vf[x] = kreg;
                kf[x][x] = (_Float16)(float)(i + x);
                vf[x][7 - x] = (_Float16)(float)(i - x);
            }
        }
        u32x4 pf[4];
        s0 = z, s1 = z;
#pragma unroll
        for (int x = 0; x < 4; ++x)
            s0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[x], q, s0, 0, 0, 0);
#pragma unroll
        for (int x = 0; x < 4; ++x)
            s1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[4 + x], q, s1, 0, 0, 0);
        auto softmax_half = [&](f32x16 &s, int half) __attribute__((always_inline)) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                s[r] = __builtin_amdgcn_exp2f(s[r]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pf[2 * half + j][e] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(s[8 * j + 2 * e], s[8 * j + 2 * e + 1]));
                    rs = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pf[2 * half + j][e]), ones, rs, false);
                }
        };
        softmax_half(s0, 0);
        softmax_half(s1, 1);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const f16x8 p = __builtin_bit_cast(f16x8, pf[st]);
            o0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * st], p, o0, 0, 0, 0);
            o1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * st + 1], p, o1, 0, 0, 0);
        }
        // issue order: (reads,) 4 MFMA [scores 0]; 4 x {MFMA [scores 1], 8 VALU [half 0]}; 4 x {MFMA [P.V 0], 8 VALU
        // [half 1]}; 4 MFMA [P.V 1]
        if (WITH_LDS)
            __builtin_amdgcn_sched_group_barrier(0x100, 16, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    }
    float t = rs;
    for (int r = 0; r < 16; ++r)
        t += o0[r] + o1[r] + s0[r] + s1[r];
    if (t == 12345.678f)
        out[0] = t;
}

// ORDER: the sequence in which the sixteen accumulators take their MFMA within one iteration.  0 row-major (the A
// fragment stays on its port for four MFMAs in a row), 1 diagonals (both operand ports change with every MFMA), 2
// boustrophedon (exactly one port changes with every MFMA)
template <int ORDER>
__global__ void __launch_bounds__(256) matrix_rate(const u32x4 *__restrict__ operands, float *out, int iters) {
    f16x8 a[4], b[4];
    for (int i = 0; i < 4; ++i) {
        a[i] = __builtin_bit_cast(f16x8, operands[(i * 2 + 0) * 64 + (threadIdx.x & 63)]);
        b[i] = __builtin_bit_cast(f16x8, operands[(i * 2 + 1) * 64 + (threadIdx.x & 63)]);
    }
    f32x16 acc[4][4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            const int i = ORDER == 1 ? (s & 3) : (s >> 2);
            const int j = ORDER == 1 ? ((s & 3) + (s >> 2)) & 3 : (ORDER == 2 && ((s >> 2) & 1) ? 3 - (s & 3) : (s & 3));
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[j], a[i], acc[i][j], 0, 0, 0);
        }
    }
    float t = 0.f;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r)
                t += acc[i][j][r];
    if (t == 12345.678f)
        out[0] = t;
}

// the int8 counterpart: sixteen independent v_mfma_i32_32x32x32_i8 per iteration
__global__ void __launch_bounds__(256) matrix_rate_i8(const u32x4 *__restrict__ operands, int *out, int iters) {
    i32x4 a[4], b[4];
    for (int i = 0; i < 4; ++i) {
        a[i] = __builtin_bit_cast(i32x4, operands[(i * 2 + 0) * 64 + (threadIdx.x & 63)]);
        b[i] = __builtin_bit_cast(i32x4, operands[(i * 2 + 1) * 64 + (threadIdx.x & 63)]);
    }
    i32x16 acc[4][4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[j], a[i], acc[i][j], 0, 0, 0);
    }
    int t = 0;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j)
            for (int r = 0; r < 16; ++r)
                t += acc[i][j][r];
    if (t == 123456789)
        out[0] = t;
}

// POP/s of the chip with every SIMD issuing int8 MFMAs only; data: 0 zeros, 1 ones, 2 uniform in [-127, 127] (quantised
// activations and weights use the whole range)
double matrix_rate_i8_pops(int data) {
    const int n = 8 * 64 * 16;  // eight fragments of 64 lanes x 16 bytes
    signed char *h = (signed char *)malloc(n);
    unsigned long long st = 1442695040888963407ull;
    for (int i = 0; i < n; ++i) {
        st = st * 6364136223846793005ull + 1442695040888963407ull;
        h[i] = data == 0 ? 0 : data == 1 ? 1 : (signed char)((int)((st >> 33) % 255) - 127);
    }
    u32x4 *d = nullptr;
    int *o   = nullptr;
    if (hipMalloc(&d, n) != hipSuccess || hipMalloc(&o, 4) != hipSuccess)
        return -1.0;
    (void)hipMemcpy(d, h, n, hipMemcpyHostToDevice);
    free(h);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    const int iters = 4000, reps = 6;
    dim3 grid(256), block(256);
    hipLaunchKernelGGL(matrix_rate_i8, grid, block, 0, 0, d, o, iters);
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0);
    for (int r = 0; r < reps; ++r)
        hipLaunchKernelGGL(matrix_rate_i8, grid, block, 0, 0, d, o, iters);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipFree(d);
    (void)hipFree(o);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    const double ops = 1024.0 * 16.0 * iters * reps * 65536.0;  // 1024 waves x 16 MFMAs x 32*32*32*2
    return ops / (ms * 1e-3) / 1e15;
}

// PFLOP/s of the chip with every SIMD issuing MFMAs only; data: 0 zeros, 1 ones, 2 normal (sigma 0.5 x sigma 0.02, the
// scale of activations times weights)
double matrix_rate_pflops(int data, int order = 0) {
    const int n = 8 * 64 * 8;  // eight fragments of 64 lanes x 8 halves
    _Float16 *h = (_Float16 *)malloc(n * sizeof(_Float16));
    unsigned long long st = 88172645463325252ull;
    auto uni = [&]() {
        st = st * 6364136223846793005ull + 1442695040888963407ull;
        return (double)((st >> 11) + 1) / 9007199254740994.0;
    };
    for (int i = 0; i < n; ++i) {
        const double g = sqrt(-2.0 * log(uni())) * cos(6.283185307179586 * uni());
        const bool is_b = (i / 512) & 1;
        h[i] = data == 0 ? (_Float16)0.f : data == 1 ? (_Float16)1.f : (_Float16)(g * (is_b ? 0.02 : 0.5));
    }
    u32x4 *d = nullptr;
    float *o = nullptr;
    if (hipMalloc(&d, n * sizeof(_Float16)) != hipSuccess || hipMalloc(&o, 4) != hipSuccess)
        return -1.0;
    (void)hipMemcpy(d, h, n * sizeof(_Float16), hipMemcpyHostToDevice);
    free(h);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    const int iters = 4000, reps = 6;  // 64 000 MFMAs per wave and launch: about 0.8 ms
    dim3 grid(256), block(256);
    auto launch = [&]() {
        if (order == 1)
            hipLaunchKernelGGL(matrix_rate<1>, grid, block, 0, 0, d, o, iters);
        else if (order == 2)
            hipLaunchKernelGGL(matrix_rate<2>, grid, block, 0, 0, d, o, iters);
        else
            hipLaunchKernelGGL(matrix_rate<0>, grid, block, 0, 0, d, o, iters);
    };
    launch();
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0);
    for (int r = 0; r < reps; ++r)
        launch();
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipFree(d);
    (void)hipFree(o);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    const double flop = 1024.0 * 16.0 * iters * reps * 32768.0;  // 1024 waves x 16 MFMAs x 32*32*16*2
    return flop / (ms * 1e-3) / 1e15;
}

template <int MODE> double ns_per_tile_and_simd(int waves_per_simd, int iters) {
    float *d = nullptr;
    if (hipMalloc(&d, 4) != hipSuccess)
        return -1.0;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    dim3 grid(256 * waves_per_simd), block(256);
    auto launch = [&](int n) {
        if (MODE == PIPE)
            hipLaunchKernelGGL((probe_pipe<false>), grid, block, 0, 0, d, n, 0.5f);
        else if (MODE == PIPE_LDS)
            hipLaunchKernelGGL((probe_pipe<true>), grid, block, 0, 0, d, n, 0.5f);
        else if (MODE == SKEW)
            hipLaunchKernelGGL((probe_skew<false>), grid, block, 0, 0, d, n, 0.5f);
        else if (MODE == SKEW_LDS)
            hipLaunchKernelGGL((probe_skew<true>), grid, block, 0, 0, d, n, 0.5f);
        else
            hipLaunchKernelGGL((probe<(MODE >= PIPE ? (int)CHAIN : MODE)>), grid, block, 0, 0, d, n, 0.5f);
    };
    launch(10);
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0);
    launch(iters);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    (void)hipFree(d);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return ms * 1e6 / iters / waves_per_simd;
}

int main() {
    const int iters = 20000;
    printf("ns per tile and SIMD (time of one wave's tile divided by the waves sharing the SIMD)\n");
    printf("%-11s %9s %9s %9s %9s %9s %9s %9s %9s %9s %9s\n", "waves/SIMD", "mfma", "valu", "chain", "lds", "tile", "ahead",
           "pipe", "pipe+lds", "skew", "skew+lds");
    for (int w = 1; w <= 3; ++w)
        printf("%-11d %9.1f %9.1f %9.1f %9.1f %9.1f %9.1f %9.1f %9.1f %9.1f %9.1f\n", w, ns_per_tile_and_simd<MFMA_ONLY>(w, iters),
               ns_per_tile_and_simd<VALU_ONLY>(w, iters), ns_per_tile_and_simd<CHAIN>(w, iters),
               ns_per_tile_and_simd<LDS_ONLY>(w, iters), ns_per_tile_and_simd<TILE>(w, iters),
               ns_per_tile_and_simd<TILE_AHEAD>(w, iters), ns_per_tile_and_simd<PIPE>(w, iters),
               ns_per_tile_and_simd<PIPE_LDS>(w, iters), ns_per_tile_and_simd<SKEW>(w, iters),
               ns_per_tile_and_simd<SKEW_LDS>(w, iters));
    printf("\nmatrix rate of the chip, one wave per SIMD issuing independent MFMAs 32x32x16 f16 only (PFLOP/s; the clock it implies\n"
           "at 1024 FLOP per clock and SIMD over 1024 SIMDs)\n");
    const char *names[3] = {"operands all zero", "operands all one", "operands normally distributed"};
    for (int data = 0; data < 3; ++data) {
        const double pf = matrix_rate_pflops(data);
        printf("%-32s %6.3f PFLOP/s   %5.2f GHz\n", names[data], pf, pf * 1e15 / (1024.0 * 1024.0) / 1e9);
    }
    printf("\nthe same on normally distributed operands, by the order of the sixteen MFMAs of an iteration\n");
    const char *orders[3] = {"row-major (A kept for four)", "diagonals (both ports change)", "boustrophedon (one port changes)"};
    for (int rep = 0; rep < 2; ++rep)
        for (int order = 0; order < 3; ++order) {
            const double pf = matrix_rate_pflops(2, order);
            printf("%-36s %6.3f PFLOP/s   %5.2f GHz\n", orders[order], pf, pf * 1e15 / (1024.0 * 1024.0) / 1e9);
        }
    printf("\nint8: sixteen independent v_mfma_i32_32x32x32_i8 per iteration (5.0 POP/s dense peak = 2048 OP per clock and SIMD)\n");
    const char *names8[3] = {"operands all zero", "operands all one", "operands uniform in [-127,127]"};
    for (int data = 0; data < 3; ++data) {
        const double po = matrix_rate_i8_pops(data);
        printf("%-32s %6.3f POP/s    %5.2f GHz\n", names8[data], po, po * 1e15 / (2048.0 * 1024.0) / 1e9);
    }
    return 0;
}
