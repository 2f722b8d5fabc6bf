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
// Each is run with 1, 2 and 3 waves per SIMD (256 x k workgroups of four waves, one wave per SIMD each) and reported
// as nanoseconds per tile and SIMD, i.e. the time divided by the waves per SIMD.
#include <hip/hip_runtime.h>

#include <cstdio>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

enum { MFMA_ONLY, VALU_ONLY, CHAIN, LDS_ONLY, TILE, TILE_AHEAD };

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

template <int MODE> double ns_per_tile_and_simd(int waves_per_simd, int iters) {
    float *d = nullptr;
    if (hipMalloc(&d, 4) != hipSuccess)
        return -1.0;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    dim3 grid(256 * waves_per_simd), block(256);
    hipLaunchKernelGGL((probe<MODE>), grid, block, 0, 0, d, 10, 0.5f);
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0);
    hipLaunchKernelGGL((probe<MODE>), grid, block, 0, 0, d, iters, 0.5f);
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
    printf("%-11s %9s %9s %9s %9s %9s %9s\n", "waves/SIMD", "mfma", "valu", "chain", "lds", "tile", "ahead");
    for (int w = 1; w <= 3; ++w)
        printf("%-11d %9.1f %9.1f %9.1f %9.1f %9.1f %9.1f\n", w, ns_per_tile_and_simd<MFMA_ONLY>(w, iters),
               ns_per_tile_and_simd<VALU_ONLY>(w, iters), ns_per_tile_and_simd<CHAIN>(w, iters),
               ns_per_tile_and_simd<LDS_ONLY>(w, iters), ns_per_tile_and_simd<TILE>(w, iters),
               ns_per_tile_and_simd<TILE_AHEAD>(w, iters));
    return 0;
}
