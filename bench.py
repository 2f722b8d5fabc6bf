#!/usr/bin/env python3
"""Benchmark of the transformer-encoder hot path on one MI355X.

A "step" is one Instance::Forward() of the DEVICE_ROCM backend on the 12-layer BERT-base encoder (hidden 768,
12 heads, FFN 3072, post-LN; fp16 activations/weights, fp32 accumulation) over one synthetic batch of 8 sequences
of 384 tokens with per-sequence valid lengths uniform in [200, 384]: token ids -> last hidden state.  The model is
written as .tnnproto/.tnnmodel (the decomposed op graph), loaded by the C++ host, rewritten by the ROCm fusion pass
and executed layer by layer; inputs are resident in their HBM blobs when the timed region starts.

Prints ONE JSON line: sequences/s, the roofline of the dominant kernel (events on the instance's stream inside the
timed region) and the CPU baseline (the reference engine's own DEVICE_X86 path, when its prebuilt library is
present) timed on this box's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
SUSTAINED_FP16_TFLOPS = 1692.0  # measured: MFMA-only loop on every SIMD, normally distributed operands (the SIMD probe)
SUSTAINED_INT8_TOPS = 3439.0    # the same loop with v_mfma_i32_32x32x32_i8 on operands uniform in [-127, 127]

# HBM bytes per launch (fetched + written) of the projection GEMMs at the batch-8 / seq-384 workload, from two
# rocprofv3 --pmc runs of this command (FETCH_SIZE, WRITE_SIZE), each scaled by what the same counter reads for the
# --counter-reference kernel (64 MiB in, 64 MiB out): FETCH_SIZE reads half the bytes, WRITE_SIZE all of them.
MEASURED_HBM_BYTES_PER_LAUNCH = {
    "gemm_qkv": int((2 * 14212.5 + 13868.7) * 1024),   # algorithmic: 4.5 + 3.4 in, 13.5 out MiB (+ row sums / statistics: 0.2)
    "gemm_out": int((2 * 10458.5 + 4896.0) * 1024),    # algorithmic: 4.5 + 1.1 + 4.5 in, 4.5 (+ 0.3 row sums) out MiB
    "gemm_ffn1": int((2 * 16752.0 + 18456.0) * 1024),  # algorithmic: 4.5 + 4.5 (+ 0.3 row sums) in, 18 out MiB
    "gemm_ffn2": int((2 * 37176.5 + 4807.6) * 1024),   # algorithmic: 18 + 4.5 + 4.5 in, 4.5 (+ 0.2 row sums) out MiB
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--seq", type=int, default=384)
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-second-instance", action="store_true",
                    help="leave out the untimed two-instances-at-once leg (kernel traces: its overlapping launches would "
                         "mix into the per-kernel averages)")
    ap.add_argument("--cpu-seqs", type=int, default=2, help="sequences in the bounded CPU-baseline sample")
    ap.add_argument("--counter-reference", action="store_true",
                    help="also launch one element-wise kernel of known size (64 MiB read, 64 MiB written) so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command carries its own scale factor")
    return ap.parse_args()


def cpu_baseline(cfg, weights, ids, seg, mask, n_seqs):
    """Bounded CPU sample: n_seqs sequences through all layers.  "reference" = the reference engine's DEVICE_X86 path
    (oracle/_ref, prebuilt) timed with the reference benchmark tool's own loop (5 warm-up + 20 timed iterations of
    SetInputMat + Forward + GetOutputMat) on all host cores, plus a reduced loop on one thread; "port" = the plain-C
    restatement under oracle/ when that library is absent."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    B, S = ids.shape
    n = min(n_seqs, B)
    try:
        import ref_driver
        if ref_driver.available():
            return ref_driver.time_encoder(cfg, weights, ids[:n], seg[:n], mask[:n])
    except (ImportError, OSError) as e:  # library missing or not loadable on this box
        print("bench.py: reference CPU library unavailable (%s); timing the restatement" % e, file=sys.stderr)
    import encoder_ref
    t0 = time.perf_counter()
    x0 = encoder_ref.embed(weights, ids[:n], seg[:n], cfg.eps)
    encoder_ref.encoder(weights, cfg, x0, n, S, mask[:n])
    dt = time.perf_counter() - t0
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {"value": n / dt, "unit": "sequences/s", "cores": cores, "kind": "port",
            "sample": "%d of %d sequences (S=%d) through all %d layers, fp32 restatement of the reference's "
                      "DEVICE_NAIVE graph, OpenMP over rows" % (n, B, S, cfg.layers)}


def classify(layer_name):
    for key in ("_ffn1_", "_ffn2_", "_o_mm"):
        if key in layer_name:
            return {"_ffn1_": "gemm_ffn1", "_ffn2_": "gemm_ffn2", "_o_mm": "gemm_out"}[key]
    return "other"


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs the hot path on ONE GPU; --gpus %d is not supported (the path shards by "
              "batch with no exchange: one process per GPU, each on its own share of the batch)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    from tnn_amd import host, ops, tnnmodel
    from tnn_amd.encoder import EncoderConfig, make_weights, make_inputs

    host.load()  # fails loudly if the HIP library or the host library is not built
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    cfg = EncoderConfig.bert_base(args.layers)
    B, S = args.batch, args.seq
    weights = make_weights(cfg, seed=20240601)
    ids, seg, lens, mask = make_inputs(cfg, B, S, min(200, S), min(384, S), seed=20240602)
    graph = tnnmodel.encoder_graph(cfg, weights, B, S)
    inst = host.RocmInstance.from_graph(graph, "fp16")
    layer_types = [t for t, _ in inst.layers()]
    inst.set_input("input_ids", ids)
    inst.set_input("token_type_ids", seg)
    inst.set_input("attention_bias", mask.reshape(B, 1, 1, S))

    # warm-up: the first forwards perform every lazy allocation (and, with TNN_ROCM_GRAPH=1, the third records the graph)
    for _ in range(max(args.warmup, 3)):
        inst.forward()

    # ---- timed region: exactly K Instance::Forward() calls (the layer loop + the engine's per-forward synchronise)
    step_s = []
    inst.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ts = time.perf_counter()
        inst.forward()          # returns after the forward's own synchronise
        step_s.append(time.perf_counter() - ts)
    inst.sync()
    dt = time.perf_counter() - t0

    # ---- untimed for `value`: the loop of the reference's benchmark tool (test/test.cc:101-152), i.e. the host Mats
    # go in and the output Mat comes out every iteration: SetInputMat x3 (25 KB over PCIe) + Forward + GetOutputMat
    # (the [8,384,768] result cast to fp32 on the device and copied to the host), 5 warm-up + 20 timed iterations
    inst.set_input("input_ids", ids)
    inst.set_input("token_type_ids", seg)
    inst.set_input("attention_bias", mask.reshape(B, 1, 1, S))
    io_min, io_avg, io_max = inst.time_loop(5, 20, "last_hidden")   # native loop, as the CPU baseline's
    # the same loop for a caller whose data is on the device already: Mats in device memory in (Mat(DEVICE_ROCM, ...)) and
    # the result out as a half Mat in device memory; nothing crosses the bus
    d_in = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in
            (ids.astype(np.int32), seg.astype(np.int32), mask.reshape(B, 1, 1, S).astype(np.float32))]
    torch.cuda.synchronize()
    inst.set_input_device("input_ids", d_in[0].data_ptr(), np.int32, [B, S])
    inst.set_input_device("token_type_ids", d_in[1].data_ptr(), np.int32, [B, S])
    inst.set_input_device("attention_bias", d_in[2].data_ptr(), np.float32, [B, 1, 1, S])
    dev_min, dev_avg, dev_max = inst.time_loop_device(5, 20, "last_hidden", np.float16)

    # ---- untimed for `value`: two instances of the same model driven from two host threads at once, each on its own
    # stream with its own batch of 8 resident in HBM.  One forward is a chain of dependent launches, each with a ramp, a
    # tail and a gap in front of it; a second chain fills them.  Sequences/s over both instances; the latency of one
    # forward roughly doubles.
    pair_dt = None
    if not args.no_second_instance:
        import threading
        inst_b = host.RocmInstance.from_graph(graph, "fp16")
        inst_b.set_input("input_ids", ids)
        inst_b.set_input("token_type_ids", seg)
        inst_b.set_input("attention_bias", mask.reshape(B, 1, 1, S))
        for _ in range(max(args.warmup, 3)):
            inst_b.forward()
        pair = [inst, inst_b]

        def drive(i):
            for _ in range(args.steps):
                pair[i].forward()
        inst.sync()
        inst_b.sync()
        tp0 = time.perf_counter()
        threads = [threading.Thread(target=drive, args=(i,)) for i in range(2)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        inst.sync()
        inst_b.sync()
        pair_dt = time.perf_counter() - tp0
        inst_b.close()

    ms_per_step = dt / args.steps * 1e3
    seqs_per_s = B * args.steps / dt
    T, H, F = B * S, cfg.hidden, cfg.ffn

    # ---- per-launch duration of the four projection GEMMs.  A captured graph cannot carry per-launch events and an
    # event pair around one 10-30 us launch in the eager layer loop also times the launch gap, so each GEMM is
    # launched back to back (same shapes, same fused epilogue, through the same C entry point the layers call)
    # between two events on the launch stream; rocprofv3's kernel trace of this command reports the same averages.
    def timed(fn, n):
        for _ in range(5):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    n_gemm = max(args.steps, 20) * cfg.layers
    x_h = torch.randn(T, H, device="cuda").half()
    x_f = torch.randn(T, F, device="cuda").half()
    res = torch.randn(T, H, device="cuda").half()
    w_qkv, w_o = (torch.randn(3 * H, H, device="cuda") * 0.02).half(), (torch.randn(H, H, device="cuda") * 0.02).half()
    w_1, w_2 = (torch.randn(F, H, device="cuda") * 0.02).half(), (torch.randn(H, F, device="cuda") * 0.02).half()
    b_qkv, b_h, b_f = (torch.randn(n, device="cuda") * 0.02 for n in (3 * H, H, F))
    o_h = torch.empty(T, H, device="cuda", dtype=torch.float16)
    o_f = torch.empty(T, F, device="cuda", dtype=torch.float16)
    # the forms the fused graph launches: QKV and FFN1 read a LayerNorm output, so they run on the raw tensor with the
    # normalisation folded into the GEMM and leave the rows' {rstd, mean} behind; the out-projection and FFN2, whose
    # residual operand is that LayerNorm output, rebuild it from the raw tensor and those statistics
    ln_g, ln_b = torch.ones(H, device="cuda"), torch.zeros(H, device="cuda")
    cs_qkv, cs_f = w_qkv.float().sum(1).contiguous(), w_1.float().sum(1).contiguous()
    stats = ops.gemm_ln(x_h, w_1, b_f, cs_f, cfg.eps, want_stats=True)[1]
    # ... and leave the row sums of their output for the folding GEMM that reads it next (FFN1 after the out-projection,
    # the next layer's QKV after FFN2), which then does not take the statistics from its own operand
    _, sums_o = ops.gemm_residual_ln(x_h, w_o, res, stats, ln_g, ln_b, bias=b_h, out=o_h, want_row_sums=True)
    _, sums_2 = ops.gemm_residual_ln(x_f, w_2, res, stats, ln_g, ln_b, bias=b_h, out=o_h, want_row_sums=True)
    gemm_ms = {
        "gemm_qkv": timed(lambda: ops.qkv_split_ln(x_h, w_qkv, b_qkv, cs_qkv, cfg.eps, B, S, cfg.heads, want_stats=True,
                                                   row_sums=sums_2, vt_key_order=1 if S % 16 == 0 else 0), n_gemm),
        "gemm_out": timed(lambda: ops.gemm_residual_ln(x_h, w_o, res, stats, ln_g, ln_b, bias=b_h, out=o_h,
                                                       want_row_sums=True, row_sums_out=sums_o[0]), n_gemm),
        "gemm_ffn1": timed(lambda: ops.gemm_ln(x_h, w_1, b_f, cs_f, cfg.eps, gelu=True, want_stats=True, row_sums=sums_o),
                           n_gemm),
        "gemm_ffn2": timed(lambda: ops.gemm_residual_ln(x_f, w_2, res, stats, ln_g, ln_b, bias=b_h, out=o_h,
                                                        want_row_sums=True, row_sums_out=sums_2[0]), n_gemm),
    }
    gemm_flops = {"gemm_qkv": 2.0 * T * 3 * H * H, "gemm_out": 2.0 * T * H * H, "gemm_ffn1": 2.0 * T * F * H,
                  "gemm_ffn2": 2.0 * T * H * F}
    gemm_shape = {"gemm_qkv": (T, 3 * H, H), "gemm_out": (T, H, H), "gemm_ffn1": (T, F, H), "gemm_ffn2": (T, H, F)}
    dominant = max(gemm_ms, key=lambda k: gemm_ms[k])
    dom_ms = gemm_ms[dominant]
    achieved = gemm_flops[dominant] / (dom_ms * 1e-3) / 1e12

    # ---- untimed: per-layer profile of the eager layer loop (events around every layer; includes launch gaps)
    full = inst.profile(5)
    breakdown = {}
    for t, name, ms in full:
        key = classify(name) if t == "RocmFusedLinear" else t
        breakdown[key] = breakdown.get(key, 0.0) + ms
    out_final = inst.output("last_hidden")
    assert np.isfinite(out_final).all()

    # the attention kernel on its own, in the layout the fused layer uses (Q|K row-major, V transposed per head):
    # this workload's shape, and the variable-length stress shape (B32, 12 heads x 64, S 512, lengths U[16,512])
    def attention_tflops(B_, S_, lens_):
        d_lens = torch.from_numpy(lens_.astype(np.int32)).cuda()
        qk = torch.randn(B_ * S_, 2 * H, device="cuda").half()
        vt = torch.randn(B_, cfg.heads, 64, S_, device="cuda").half()
        ctx = torch.empty(B_ * S_, H, device="cuda", dtype=torch.float16)
        # (V^T with its keys in the order the fused layer's projection leaves them whenever S is a multiple of 16)
        ms = timed(lambda: ops.attention_qk_vt(qk, vt, B_, S_, cfg.heads, 0.125, kv_len=d_lens, out=ctx,
                                               vt_key_order=1 if S_ % 16 == 0 else 0), 100)
        eff, pad = 4.0 * H * S_ * float(lens_.sum()), 4.0 * B_ * S_ * S_ * H
        return {"effective": round(eff / (ms * 1e-3) / 1e12, 2), "padded": round(pad / (ms * 1e-3) / 1e12, 2),
                "us_per_launch": round(ms * 1e3, 2),
                "frac_of_fp16_peak_effective": round(eff / (ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 4)}

    # ---- the int8 path's dominant kernel on its own workload (config 4: B16 S256 -> 4096 tokens): FFN1 as the
    # quantised graph launches it (int8 x int8 -> int32, requantise, the GELU chain as a table in the epilogue)
    def int8_roofline():
        T8 = 16 * 256
        a8 = torch.randint(-128, 128, (T8, H), device="cuda", dtype=torch.int8)
        w8 = torch.randint(-127, 128, (F, H), device="cuda", dtype=torch.int8)
        b8 = torch.randint(-500, 500, (F,), device="cuda", dtype=torch.int32)
        sc = (torch.rand(F, device="cuda") * 2e-4 + 1e-4).float()
        iota = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8).cuda()
        lut = ops.gelu_i8(iota, 0.05, 20.0)
        o8 = torch.empty(T8, F, device="cuda", dtype=torch.int8)
        ms = timed(lambda: ops.gemm_i8_lut(a8, w8, b8, sc, lut, out=o8), n_gemm)
        opsn = 2.0 * T8 * F * H
        return {"bound": "mfma", "kernel": "gemm_nk_tiled_kernel<int8> (config 4 FFN1: M=%d N=%d K=%d, requantise + GELU "
                                           "table epilogue)" % (T8, F, H),
                "achieved": round(opsn / (ms * 1e-3) / 1e12, 2), "peak": 5000.0, "unit": "TOP/s",
                "frac": round(opsn / (ms * 1e-3) / 1e12 / 5000.0, 4), "traffic": None,
                "us_per_launch": round(ms * 1e3, 2), "ops_per_launch": opsn,
                "sustained_matrix_rate": {"tops": SUSTAINED_INT8_TOPS,
                                          "frac": round(opsn / (ms * 1e-3) / 1e12 / SUSTAINED_INT8_TOPS, 4),
                                          "what": "what the chip holds with every SIMD issuing nothing but independent int8 "
                                                  "MFMAs on operands that use the whole int8 range (4897 on all-zero ones); "
                                                  "context only, frac above stays on the data-sheet peak",
                                          "source": "profiles/simd_probe_mfma_valu_lds.txt (python -m tnn_amd.bench_ops "
                                                    "--simd-probe), typed into bench.py, not measured by this run"}}

    # the dominant GEMM inside the forward: the event pair the eager layer loop puts around its layer (profile pass above),
    # averaged over the layers.  It spans from the previous layer's last kernel to this layer's last kernel on the
    # stream, i.e. the kernel plus the gap in front of it with the weights as the previous layers left them in the
    # caches; the profile pass synchronises per layer, so the host-side launch cost can widen that gap.  The QKV
    # projection shares its layer with the attention kernel and has no figure of its own.
    dom_in_forward_ms = breakdown[dominant] / cfg.layers if dominant in breakdown else None

    roof_i8 = int8_roofline()
    attn_here = attention_tflops(B, S, lens)
    stress_lens = np.random.default_rng(20240603).integers(16, 513, 32)
    attn_stress = attention_tflops(32, 512, stress_lens)
    attn_stress["workload"] = "B32 h12 d64 S512, valid lengths U[16,512] (BASELINE.json configs[2])"

    if args.counter_reference:
        big = torch.randn(16 * 1024 * 1024, device="cuda", dtype=torch.float32)
        torch.cuda.synchronize()
        ops.gelu(big)  # unary_kernel: reads 64 MiB, writes 64 MiB
        torch.cuda.synchronize()

    full_cfg = (B, S, args.layers) == (8, 384, 12)
    out = {
        "metric": "BERT-base seq384 fp16 sequences/sec on 1 MI355X; fused-attention TFLOP/s",
        "value": round(seqs_per_s, 2), "unit": "sequences/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "ms_per_step_min_avg_max": [round(min(step_s) * 1e3, 4), round(sum(step_s) / len(step_s) * 1e3, 4),
                                    round(max(step_s) * 1e3, 4)],
        "with_mat_io": {"loop": "SetInputMat x3 + Forward + GetOutputMat, 5 warm-up + 20 timed (test/test.cc:101-152)",
                        "ms_min_avg_max": [round(io_min * 1e3, 4), round(io_avg * 1e3, 4), round(io_max * 1e3, 4)],
                        "sequences_per_s": round(B / io_avg, 2),
                        "device_mats": {"loop": "the same loop with Mats in device memory (DEVICE_ROCM Mats in, a half "
                                                "Mat in device memory out): nothing crosses the bus",
                                        "ms_min_avg_max": [round(dev_min * 1e3, 4), round(dev_avg * 1e3, 4),
                                                           round(dev_max * 1e3, 4)],
                                        "sequences_per_s": round(B / dev_avg, 2)}},
        "two_instances_at_once": None if pair_dt is None else {
            "what": "two Instances of this model, each with its own batch of %d, driven from two host threads on two "
                    "streams: %d forwards each; not `value` (two batches in flight, a forward's latency about doubles)"
                    % (B, args.steps),
            "sequences_per_s": round(2 * B * args.steps / pair_dt, 2),
            "ms_per_forward_per_instance": round(pair_dt / args.steps * 1e3, 4)},
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": ("12-layer BERT-base encoder fp16, batch 8, seq 384, valid lengths U[200,384] "
                                "(BASELINE.json configs[1])") if full_cfg else
                   "%d-layer BERT-base encoder fp16, batch %d, seq %d" % (args.layers, B, S),
                   "path": "Instance::Forward on DEVICE_ROCM from .tnnproto/.tnnmodel, ROCm fusion pass on, " +
                           ("whole-forward graph replay" if os.environ.get("TNN_ROCM_GRAPH", "0") not in ("", "0") else
                            "eager layer loop on one stream (graph replay behind TNN_ROCM_GRAPH=1 measured 0.5-1.8 % slower)"),
                   "layers": args.layers, "batch": B, "seq_len": S, "hidden": H, "heads": cfg.heads, "ffn": F,
                   "sum_valid_len": int(lens.sum()), "host_layers": len(layer_types)},
        "model_tflops": round(cfg.flops_per_sequence(S) * seqs_per_s / 1e12, 2),
        "attention_tflops": attn_here,
        "attention_tflops_varlen_stress": attn_stress,
        "roofline": {"bound": "mfma",
                     "kernel": "gemm_nk_tiled_kernel (%s: M=%d N=%d K=%d, fused epilogue)" % ((dominant,) + gemm_shape[dominant]),
                     "achieved": round(achieved, 2), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP16_TFLOPS, 4),
                     "traffic": MEASURED_HBM_BYTES_PER_LAUNCH.get(dominant) if full_cfg else None,
                     "traffic_source": ("profiles/bench_c2_bert_base_b8_s384_hbm_traffic_counters.txt: rocprofv3 --pmc "
                                        "FETCH_SIZE and WRITE_SIZE runs of this command, typed into bench.py, not "
                                        "measured by this run") if full_cfg else None,
                     "us_per_launch": round(dom_ms * 1e3, 2),
                     "us_in_forward": None if dom_in_forward_ms is None else round(dom_in_forward_ms * 1e3, 2),
                     "frac_in_forward": None if dom_in_forward_ms is None else round(
                         gemm_flops[dominant] / (dom_in_forward_ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 4),
                     "in_forward_is": "this GEMM's layer between the event pair of the eager layer loop, mean over the "
                                      "layers: kernel + the gap in front of it (frac stays on the back-to-back figure)",
                     "timed_over": "%d back-to-back launches between two events on the launch stream, right after "
                                   "the timed region" % n_gemm,
                     "flops_per_launch": gemm_flops[dominant],
                     "sustained_matrix_rate": {
                         "tflops": SUSTAINED_FP16_TFLOPS, "frac": round(achieved / SUSTAINED_FP16_TFLOPS, 4),
                         "what": "what the chip holds with every SIMD issuing nothing but independent fp16 MFMAs on normally "
                                 "distributed operands (2474 on all-zero ones): power management, not the kernel, sets it; "
                                 "context only, frac above stays on the data-sheet peak",
                         "source": "profiles/simd_probe_mfma_valu_lds.txt (python -m tnn_amd.bench_ops --simd-probe), typed into "
                                   "bench.py, not measured by this run"},
                     "all_gemms_us_per_launch": {k: round(v * 1e3, 2) for k, v in sorted(gemm_ms.items())},
                     "all_gemms_tflops": {k: round(gemm_flops[k] / (v * 1e-3) / 1e12, 1) for k, v in sorted(gemm_ms.items())}},
        "roofline_int8": roof_i8,
        "layer_breakdown_ms_per_step": {k: round(v, 4) for k, v in sorted(breakdown.items())},
    }
    inst.close()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, weights, ids, seg, mask, args.cpu_seqs)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
