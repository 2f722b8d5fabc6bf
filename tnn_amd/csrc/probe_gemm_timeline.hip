// Stand-alone timeline of the tiled projection GEMM: where one launch spends its time (entry, first slab landed, main
// loop, epilogue / C stores, LayerNorm output) and how much of the launch-to-launch period lies outside the kernel's own
// code (dispatch, cache write-back at the kernel's end).  Nothing in the library uses it.
//
//   cd tnn_amd/csrc && hipcc --offload-arch=gfx950 -O3 -std=c++17 -ffp-contract=off -Xclang -target-feature -Xclang \
//       -packed-fp32-ops -I ../../include -I . probe_gemm_timeline.hip runtime.hip -o ../lib/probe_gemm_timeline
//   ../lib/probe_gemm_timeline N K mode        (M = 3072 tokens; mode 0 bias, 1 bias + GELU, 2 LayerNorm folded +
//                                               GELU + LayerNorm output, 3 bias + residual, 4 as 2 with the row
//                                               statistics instead of the LayerNorm output, 5 bias + a residual
//                                               rebuilt from the raw tensor and the row statistics, 6 as 4 with the
//                                               statistics from handed-over row sums, 7 as 5 leaving such sums)
// The kernels are compiled from gemm.hip itself with the timeline stamps switched on.
#define TNN_ROCM_TIMELINE 1
#include "gemm.hip"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

int main(int argc, char **argv) {
    if (argc < 4) {
        fprintf(stderr, "usage: %s N K mode\n", argv[0]);
        return 2;
    }
    const int M = 3072, N = atoi(argv[1]), K = atoi(argv[2]), mode = atoi(argv[3]);
    _Float16 *A, *B, *C, *Y, *R;
    float *bias, *cs, *g, *be, *stats, *gn, *bn, *sums;
    (void)hipMalloc(&A, (size_t)M * K * 2);
    (void)hipMalloc(&B, (size_t)N * K * 2);
    (void)hipMalloc(&C, (size_t)M * N * 2);
    (void)hipMalloc(&Y, (size_t)M * K * 2);
    (void)hipMalloc(&R, (size_t)M * N * 2);
    (void)hipMalloc(&bias, N * 4);
    (void)hipMalloc(&cs, N * 4);
    (void)hipMalloc(&g, K * 4);
    (void)hipMalloc(&be, K * 4);
    (void)hipMemset(A, 0x11, (size_t)M * K * 2);
    (void)hipMemset(B, 0x11, (size_t)N * K * 2);
    (void)hipMemset(R, 0, (size_t)M * N * 2);
    (void)hipMemset(bias, 0, N * 4);
    (void)hipMemset(cs, 0, N * 4);
    (void)hipMemset(g, 0, K * 4);
    (void)hipMemset(be, 0, K * 4);
    (void)hipMalloc(&stats, (size_t)M * 8);
    (void)hipMalloc(&gn, N * 4);
    (void)hipMalloc(&bn, N * 4);
    (void)hipMemset(stats, 0, (size_t)M * 8);
    // TNN_PROBE_SUMS_BEHIND_A=1: the row sums sit in the allocation of A, right behind it (address translation shared)
    if (getenv("TNN_PROBE_SUMS_BEHIND_A")) {
        (void)hipFree(A);
        (void)hipMalloc(&A, (size_t)M * K * 2 + (size_t)TNN_ROCM_MAX_ROW_SUM_BLOCKS * M * 8);
        (void)hipMemset(A, 0x11, (size_t)M * K * 2);
        sums = (float *)((char *)A + (size_t)M * K * 2);
    } else
        (void)hipMalloc(&sums, (size_t)TNN_ROCM_MAX_ROW_SUM_BLOCKS * M * 8);
    (void)hipMemset(sums, 0, (size_t)TNN_ROCM_MAX_ROW_SUM_BLOCKS * M * 8);
    (void)hipMemset(gn, 0, N * 4);
    (void)hipMemset(bn, 0, N * 4);
    // TNN_PROBE_WRITE_BACK=1: ordinary write-back stores for the results instead of the device-scope stores
    if (getenv("TNN_PROBE_WRITE_BACK"))
        (void)tnn_rocm_debug_set_store_through(0);
    hipStream_t s;
    (void)hipStreamCreate(&s);
    auto call = [&]() {
        if (mode == 2 || mode == 4 || mode == 6)  // LayerNorm folded in; 2: its output written, 4: the row statistics
            // handed on instead, 6: as 4 with the statistics taken from the producer's row sums (twelve blocks)
            return tnn_rocm_gemm_ln(s, TNN_ROCM_F16, A, B, bias, cs, g, be, 1e-12f, C, mode == 2 ? Y : nullptr,
                                    mode != 2 ? stats : nullptr, mode == 6 ? sums : nullptr, mode == 6 ? 12 : 0, M, N, K,
                                    TNN_ROCM_EPI_GELU, nullptr);
        if (mode == 5 || mode == 7) {  // bias + a LayerNorm output rebuilt from the raw tensor as the residual; 7: also
            int blocks = 0;            // leaves the row sums of its output
            return tnn_rocm_gemm_residual_ln(s, TNN_ROCM_F16, A, B, bias, C, R, stats, gn, bn, M, N, K, TNN_ROCM_EPI_BIAS,
                                             mode == 7 ? sums : nullptr, mode == 7 ? &blocks : nullptr);
        }
        const int fl = TNN_ROCM_EPI_BIAS | (mode == 1 ? TNN_ROCM_EPI_GELU : 0) | (mode == 3 ? TNN_ROCM_EPI_RESIDUAL : 0);
        return tnn_rocm_gemm(s, TNN_ROCM_F16, 1, A, B, C, M, N, K, K, K, N, 1, 1, 1, fl, bias, mode == 3 ? R : nullptr, N);
    };
    for (int i = 0; i < 20; i++)
        if (call()) {
            printf("error: %s\n", tnn_rocm_last_error());
            return 1;
        }
    (void)hipStreamSynchronize(s);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    (void)hipEventRecord(e0, s);
    for (int i = 0; i < 200; i++)
        call();
    (void)hipEventRecord(e1, s);
    (void)hipStreamSynchronize(s);
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    printf("M=%d N=%d K=%d mode=%d: %.2f us launch to launch (200 back-to-back launches)\n", M, N, K, mode, ms * 1000 / 200);
    std::vector<unsigned long long> tl(4096 * 8);
    (void)hipMemcpyFromSymbol(tl.data(), HIP_SYMBOL(g_gemm_timeline), tl.size() * 8);  // the last launch's stamps
    unsigned long long t0 = ~0ull;
    int nb = 0;
    for (int b = 0; b < 4096; b++)
        if (tl[b * 8]) {
            t0 = std::min(t0, tl[b * 8]);
            nb = b + 1;
        }
    // stamp slots roughly in the order the kernel passes them (the row sums are added up before the first slab has
    // landed in tile shapes that share a CU, after the main loop in those that have one to themselves)
    const int order[7] = {0, 5, 1, 6, 2, 3, 4};
    const char *nm[7]  = {"entry", "first slabs requested", "first slab landed", "row sums added up", "main loop done",
                          "C stored", "kernel end"};
    double sum[7] = {0}, mx[7] = {0}, mn[7] = {1e9, 1e9, 1e9, 1e9, 1e9, 1e9, 1e9};
    int cnt = 0;
    for (int b = 0; b < nb; b++) {
        if (!tl[b * 8 + 4])
            continue;
        cnt++;
        for (int i = 0; i < 7; i++) {
            const double v = tl[b * 8 + order[i]] ? (tl[b * 8 + order[i]] - t0) * 0.01 : 0.0;  // 100 MHz counter -> us
            sum[i] += v, mx[i] = std::max(mx[i], v), mn[i] = std::min(mn[i], v);
        }
    }
    for (int i = 0; i < 7; i++)
        if (sum[i] > 0 || i == 0)  // the direct-to-LDS pipeline stamps all seven; the register-staged one five
            printf("  %-22s mean %6.2f us  min %6.2f  max %6.2f   (%d workgroups, from the first workgroup's entry)\n", nm[i],
                   sum[i] / cnt, mn[i], mx[i], cnt);
    printf("  %-22s %6.2f us   (launch to launch minus the last workgroup's end)\n", "until the next launch",
           ms * 1000 / 200 - mx[6]);
    return 0;
}
