"""Timing of the benchmark configurations other than the headline one (which bench.py at the repository root covers):

  c1  one self-attention layer, fp32, S=128, hidden 768, 12 heads (InnerProduct projections, no mask)
  c3  the fused attention kernel alone, fp16, B32 h12 d64 S512, valid lengths U[16,512]
  c4  12-layer BERT-base encoder with int8 projections (per-channel weights), B16 S256, activations fp16
  c5  24-layer BERT-large encoder, fp16, B16 S512, valid lengths U[384,512]

    python -m tnn_amd.bench_configs --config c5 [--steps 20] [--layers N]

  stores  the headline forward (12-layer BERT-base fp16, B8 S384) with the results of the GEMM / attention / LayerNorm
          kernels stored through the L2 at device scope (the default) against ordinary write-back stores: one instance,
          one recorded graph, the switch (tnn_rocm_debug_set_store_through) flipped between timing rounds

Every configuration runs Instance::Forward on DEVICE_ROCM from .tnnproto/.tnnmodel bytes built in memory (synthetic
weights and inputs, seeded), prints one JSON line and needs the built libraries; nothing falls back to the CPU."""
import argparse
import json
import time

import numpy as np

from . import host, quant, tnnmodel
from .encoder import EncoderConfig, make_inputs, make_weights


def _time_forward(inst, steps, warmup=6):
    for _ in range(max(warmup, 3)):
        inst.forward()
    inst.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        inst.forward()
    inst.sync()
    return (time.perf_counter() - t0) / steps


def _layer_table(inst):
    agg = {}
    for t, name, ms in inst.profile(3):
        key = t
        if t == "RocmFusedLinear":
            key = "ffn1" if "_ffn1_" in name else "ffn2" if "_ffn2_" in name else "out"
        agg[key] = round(agg.get(key, 0.0) + ms, 4)
    return agg


def c1(args):
    cfg = EncoderConfig(1, 768, 12, 3072)
    lw = make_weights(cfg, seed=20240601, with_embeddings=False)["layers"][0]
    x = np.random.default_rng(20240602).standard_normal((128, 768)).astype(np.float32)
    inst = host.RocmInstance.from_graph(tnnmodel.attention_layer_graph(lw, 128, 768, 12), "fp32")
    inst.set_input("x", x)
    dt = _time_forward(inst, args.steps)
    flops = 8 * 128 * 768 * 768 + 4 * 128 * 128 * 768
    out = {"config": "c1", "workload": "attention layer fp32, S128 H768 h12", "ms_per_forward": dt * 1e3,
           "tflops": flops / dt / 1e12, "layers": [t for t, _ in inst.layers()]}
    inst.close()
    return out


def c3(args):
    import torch
    from . import ops
    # --batch / --seq move the kernel away from the configuration's own shape (e.g. B4 S4096: its steady state)
    B, h, S = args.batch or 32, 12, args.seq or 512
    H = h * 64
    rng = np.random.default_rng(20240603)
    lens = rng.integers(min(16, S), S + 1, B).astype(np.int32)
    qk = torch.randn(B * S, 2 * H, device="cuda").half()
    vt = torch.randn(B, h, 64, S, device="cuda").half()
    out = torch.empty(B * S, H, device="cuda", dtype=torch.half)
    kv = torch.from_numpy(lens).cuda()
    res = {}
    for name, kvl in (("varlen", kv), ("full", None)):
        # launches recorded into one graph, so the host's launch rate is not what is measured
        def call():
            ops.attention_qk_vt(qk, vt, B, S, h, 0.125, kv_len=kvl, out=out, vt_key_order=1 if S % 16 == 0 else 0)
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        graph, n = torch.cuda.CUDAGraph(), 50
        with torch.cuda.graph(graph):
            for _ in range(n):
                call()
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        res[name] = e0.elapsed_time(e1) / (args.steps * n) * 1e3
    eff, pad = 4 * H * S * int(lens.sum()), 4 * B * S * S * H
    return {"config": "c3", "workload": "attention kernel fp16, B%d h12 d64 S%d, lengths U[%d,%d]" % (B, S, min(16, S), S),
            "us_per_launch": res["varlen"], "tflops_effective": eff / res["varlen"] / 1e6,
            "tflops_padded": pad / res["varlen"] / 1e6, "us_per_launch_full_lengths": res["full"],
            "tflops_full_lengths": pad / res["full"] / 1e6}


def c4(args):
    cfg = EncoderConfig.bert_base(args.layers or 12)
    w = make_weights(cfg, seed=20240604)
    B, S = 16, 256
    ids, seg, lens, mask = make_inputs(cfg, B, S, S, S, seed=20240605)
    feed = {"input_ids": ids, "token_type_ids": seg, "attention_bias": mask.reshape(B, 1, 1, S)}
    # per-tensor activation scales from one fp32 forward of the float model on the device
    names = quant.calibration_outputs(cfg)
    inst = host.RocmInstance.from_graph(tnnmodel.encoder_graph(cfg, w, B, S, extra_outputs=names), "fp32")
    for k, v in feed.items():
        inst.set_input(k, v)
    inst.forward()
    scales = {n: quant.activation_scale(inst.output(n, max_elems=1 << 26)) for n in names}
    ref = inst.output("last_hidden")
    inst.close()
    inst = host.RocmInstance.from_graph(quant.int8_encoder_graph(cfg, w, scales, B, S), "fp16")
    for k, v in feed.items():
        inst.set_input(k, v)
    dt = _time_forward(inst, args.steps)
    got = inst.output("last_hidden")
    T, H, F = B * S, cfg.hidden, cfg.ffn
    int8_ops = cfg.layers * (8 * T * H * H + 4 * T * H * F)
    out = {"config": "c4", "workload": "%d-layer BERT-base int8 projections, B16 S256" % cfg.layers,
           "ms_per_forward": dt * 1e3, "sequences_per_s": B / dt, "int8_tops_projections": int8_ops / dt / 1e12,
           "rel_diff_to_float_model": float(np.abs(got - ref).max() / np.abs(ref).max()),
           "layer_ms": _layer_table(inst)}
    inst.close()
    return out


def c5(args):
    cfg = EncoderConfig.bert_large(args.layers or 24)
    B, S = 16, 512
    w = make_weights(cfg, seed=20240606)
    ids, seg, lens, mask = make_inputs(cfg, B, S, 384, 512, seed=20240607)
    inst = host.RocmInstance.from_graph(tnnmodel.encoder_graph(cfg, w, B, S), "fp16")
    inst.set_input("input_ids", ids)
    inst.set_input("token_type_ids", seg)
    inst.set_input("attention_bias", mask.reshape(B, 1, 1, S))
    dt = _time_forward(inst, args.steps)
    out = {"config": "c5", "workload": "%d-layer BERT-large fp16, B16 S512, lengths U[384,512]" % cfg.layers,
           "ms_per_forward": dt * 1e3, "sequences_per_s": B / dt,
           "model_tflops": cfg.flops_per_sequence(S) * B / dt / 1e12, "layer_ms": _layer_table(inst)}
    inst.close()
    return out


def stores(args):
    from . import capi
    lib = capi.load()
    cfg = EncoderConfig.bert_base(args.layers or 12)
    B, S = 8, 384
    w = make_weights(cfg, seed=20240601)
    ids, seg, lens, mask = make_inputs(cfg, B, S, 200, S, seed=20240602)
    inst = host.RocmInstance.from_graph(tnnmodel.encoder_graph(cfg, w, B, S), "fp16")
    inst.set_input("input_ids", ids)
    inst.set_input("token_type_ids", seg)
    inst.set_input("attention_bias", mask.reshape(B, 1, 1, S))
    for _ in range(6):
        inst.forward()
    ms, outs = {1: [], 0: []}, {}
    try:
        for _ in range(10):
            for through in (1, 0):
                inst.sync()
                lib.tnn_rocm_debug_set_store_through(through)
                ms[through].append(_time_forward(inst, args.steps, warmup=3) * 1e3)
                outs[through] = inst.output("last_hidden")
    finally:
        lib.tnn_rocm_debug_set_store_through(1)
    inst.close()
    med = {k: sorted(v)[len(v) // 2] for k, v in ms.items()}
    return {"config": "stores", "workload": "%d-layer BERT-base fp16, B8 S384, one instance, ten rounds each" % cfg.layers,
            "ms_per_forward_store_through": round(med[1], 4), "ms_per_forward_write_back": round(med[0], 4),
            "min_max_store_through": [round(min(ms[1]), 4), round(max(ms[1]), 4)],
            "min_max_write_back": [round(min(ms[0]), 4), round(max(ms[0]), 4)],
            "outputs_identical": bool(np.array_equal(outs[0], outs[1]))}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--config", choices=["c1", "c3", "c4", "c5", "stores"], required=True)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration names (c4, c5)")
    ap.add_argument("--batch", type=int, default=0, help="c3: batch instead of 32")
    ap.add_argument("--seq", type=int, default=0, help="c3: sequence length instead of 512")
    args = ap.parse_args()
    print(json.dumps({"c1": c1, "c3": c3, "c4": c4, "c5": c5, "stores": stores}[args.config](args)))


if __name__ == "__main__":
    main()
