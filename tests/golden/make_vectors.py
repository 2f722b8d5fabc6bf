#!/usr/bin/env python3
"""Writes the committed fixtures of tests/golden/ by running the reference engine itself.

The reference ships no golden vectors for the encoder path (its tests are differential against DEVICE_NAIVE on rand()
data), so these are produced by the reference's own code: oracle/_ref (the reference sources compiled in this
container by oracle/Makefile.ref) runs small seeded graphs on DEVICE_NAIVE (fp32 oracle) and DEVICE_X86 (the int8
"product" semantics), and inputs + outputs are stored.  The fixtures let the CPU checker and the HIP path be compared
with the reference's results where the reference tree (and hence oracle/_ref) is absent.

Run from the repository root after `make -C oracle`:   python tests/golden/make_vectors.py [fixture name ...]
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import ref_driver  # noqa: E402
from tnn_amd import tnnmodel  # noqa: E402
from tnn_amd.encoder import EncoderConfig, make_weights, make_inputs  # noqa: E402


def run(g, inputs, outs, dev):
    s = ref_driver.RefSession(g, dev, 1)
    for k, v in inputs.items():
        s.set_input(k, v)
    s.forward()
    r = [s.output(o) for o in outs]
    s.close()
    return r


def single_ops():
    rng = np.random.default_rng(100)
    out = {}
    x = (rng.standard_normal((3, 257)) * 3).astype(np.float32)
    x[0, :4] = [-2.281006575, 0.0, 8.5, -8.5]
    g = tnnmodel.Graph()
    g.add_input("x", list(x.shape))
    g.add_layer("GELU", "g", ["x"], ["y"])
    g.add_output("y")
    out["gelu_x"], out["gelu_y"] = x, run(g, {"x": x}, ["y"], "NAIVE")[0]

    x = (rng.standard_normal((5, 96)) * 2 + 0.3).astype(np.float32)
    x[4] += 1000.0  # large mean: exercises the double-precision sums
    ga, be = rng.standard_normal(96).astype(np.float32), rng.standard_normal(96).astype(np.float32)
    g = tnnmodel.Graph()
    g.add_input("x", list(x.shape))
    g.add_constant("ga", ga)
    g.add_constant("be", be)
    g.add_layer("LayerNorm", "ln", ["x", "ga", "be"], ["y"], [1, "1e-12"])
    g.add_output("y")
    out["ln_x"], out["ln_g"], out["ln_b"] = x, ga, be
    out["ln_y"] = run(g, {"x": x}, ["y"], "NAIVE")[0]

    x = (rng.standard_normal((2, 3, 8, 40)) * 4).astype(np.float32)
    x[0, 0, 0, 20:] = -10000.0  # masked keys: exact zeros on the reference
    for axis in (1, 3):
        g = tnnmodel.Graph()
        g.add_input("x", list(x.shape))
        g.add_layer("Softmax", "s", ["x"], ["y"], [axis])
        g.add_output("y")
        out["softmax_y_axis%d" % axis] = run(g, {"x": x}, ["y"], "NAIVE")[0]
    out["softmax_x"] = x

    a = rng.standard_normal((2, 3, 8, 16)).astype(np.float32)
    b = rng.standard_normal((3, 16, 9)).astype(np.float32)
    g = tnnmodel.Graph()
    g.add_input("a", list(a.shape))
    g.add_input("b", list(b.shape))
    g.add_layer("MatMul", "mm", ["a", "b"], ["y"], [-1])
    g.add_output("y")
    out["matmul_a"], out["matmul_b"] = a, b
    out["matmul_y"] = run(g, {"a": a, "b": b}, ["y"], "NAIVE")[0]
    np.savez_compressed(os.path.join(HERE, "single_ops_naive.npz"), **out)


def tiny_encoder():
    # one post-LN encoder layer with embeddings and a padding mask: hidden 64, one head of 64, FFN 128
    cfg = EncoderConfig(1, 64, 1, 128, vocab=50, max_pos=32)
    w = make_weights(cfg, seed=11, bias_std=0.02)
    rng = np.random.default_rng(12)
    lw = w["layers"][0]
    lw["ln1_g"] = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    lw["ln1_b"] = (0.1 * rng.standard_normal(64)).astype(np.float32)
    lw["ln2_g"] = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    lw["ln2_b"] = (0.1 * rng.standard_normal(64)).astype(np.float32)
    B, S = 2, 24
    ids, seg, lens, mask = make_inputs(cfg, B, S, 5, 24, seed=13)
    g = tnnmodel.encoder_graph(cfg, w, B, S, extra_outputs=["x0", "l0_probs", "l0_x1"])
    inputs = {"input_ids": ids, "token_type_ids": seg, "attention_bias": mask.reshape(B, 1, 1, S)}
    names = ["x0", "l0_probs", "l0_x1", "last_hidden"]
    naive = run(g, inputs, names, "NAIVE")
    x86 = run(g, inputs, ["last_hidden"], "X86")
    out = {"ids": ids, "seg": seg, "lens": lens, "mask": mask, "x86_last_hidden": x86[0]}
    for n, v in zip(names, naive):
        out["naive_" + n] = v
    for k, v in w.items():
        if k != "layers":
            out["w_" + k] = v
    for k, v in lw.items():
        out["l0_" + k] = v
    np.savez_compressed(os.path.join(HERE, "tiny_encoder.npz"), **out)


def config1_summary():
    # BASELINE config 1 (B1 S128 H768 h12 fp32): inputs are regenerated from seeds, so only digests and one slice
    cfg = EncoderConfig(1, 768, 12, 3072)
    lw = make_weights(cfg, seed=1, with_embeddings=False)["layers"][0]
    x = np.random.default_rng(2).standard_normal((128, 768)).astype(np.float32)
    g = tnnmodel.attention_layer_graph(lw, 128, 768, 12)
    y = run(g, {"x": x}, ["y"], "NAIVE")[0]
    np.savez_compressed(os.path.join(HERE, "config1_attention_naive.npz"),
                        x_sum=np.float64(x.astype(np.float64).sum()), x_abs_sum=np.float64(np.abs(x).astype(np.float64).sum()),
                        wq_sum=np.float64(lw["wq"].astype(np.float64).sum()), wo_sum=np.float64(lw["wo"].astype(np.float64).sum()),
                        y_sum=np.float64(y.astype(np.float64).sum()), y_abs_sum=np.float64(np.abs(y).astype(np.float64).sum()),
                        y_rows_0_8=y[:8].copy(), y_rows_120_128=y[120:].copy())


def int8_ffn():
    rng = np.random.default_rng(0)
    T, K, F = 32, 64, 128
    x = rng.standard_normal((T, K)).astype(np.float32)
    w1 = rng.integers(-127, 128, (F, K), dtype=np.int8)
    w2 = rng.integers(-127, 128, (K, F), dtype=np.int8)
    b1 = rng.integers(-500, 500, F).astype(np.int32)
    b2 = rng.integers(-500, 500, K).astype(np.int32)
    ws1 = (rng.uniform(0.5, 1.5, F) * 2e-4).astype(np.float32)
    ws2 = (rng.uniform(0.5, 1.5, K) * 2e-4).astype(np.float32)
    scales = np.array([0.031, 0.045, 0.027, 0.052], np.float32)
    g = tnnmodel.int8_ffn_graph(T, K, F, w1, b1, ws1, w2, b2, ws2, *scales)
    y_x86 = run(g, {"x": x}, ["y"], "X86")[0]
    y_naive = run(g, {"x": x}, ["y"], "NAIVE")[0]
    np.savez_compressed(os.path.join(HERE, "int8_ffn.npz"), x=x, w1=w1, w2=w2, b1=b1, b2=b2, ws1=ws1, ws2=ws2,
                        scales=scales, y_x86=y_x86, y_naive=y_naive)


def int8_encoder():
    """One-layer int8 encoder (hidden 128, 2 heads, FFN 256, B2 S16): calibrated on the fp32 NAIVE forward, run on
    DEVICE_X86; weights are regenerated from the seed (digest stored), scales and every int8 blob are stored."""
    from tnn_amd import quant
    cfg = EncoderConfig(1, 128, 2, 256, vocab=1000, max_pos=64)
    w = make_weights(cfg, seed=21, bias_std=0.02)
    B, S = 2, 16
    ids, seg, lens, mask = make_inputs(cfg, B, S, 5, 16, seed=22)
    inputs = {"input_ids": ids, "token_type_ids": seg, "attention_bias": mask.reshape(B, 1, 1, S)}
    names = quant.calibration_outputs(cfg)
    acts = dict(zip(names, run(tnnmodel.encoder_graph(cfg, w, B, S, extra_outputs=names), inputs, names, "NAIVE")))
    scales = quant.scales_from_activations(acts)
    blobs = ["x0"] + ["l0_" + b for b in quant.CALIBRATION_BLOBS]
    g = quant.int8_encoder_graph(cfg, w, scales, B, S, extra_outputs=blobs)
    outs = run(g, inputs, ["last_hidden"] + blobs, "X86")
    out = {"ids": ids, "seg": seg, "mask": mask, "x86_last_hidden": outs[0],
           "w_digest": np.float64(sum(float(np.abs(v).astype(np.float64).sum()) for v in w["layers"][0].values()))}
    for n, v in zip(blobs, outs[1:]):
        out["x86_" + n] = v
    for n in names:
        out["scale_" + n] = scales[n]
    np.savez_compressed(os.path.join(HERE, "int8_encoder_x86.npz"), **out)


def int8_add():
    """QuantizedAdd over all 65536 (a, b) int8 pairs for the scale triples of golden_util.INT8_ADD_SCALES, on both
    devices; the int8 results are stored (the graph's fp32 output divided by the output scale)."""
    import golden_util
    out = {}
    for k in range(len(golden_util.INT8_ADD_SCALES)):
        qa, qb, x, z, sa, sb, so = golden_util.int8_add_case(k)
        g = tnnmodel.int8_add_graph(golden_util.INT8_ADD_DIMS, sa, sb, so)
        for dev in ("NAIVE", "X86"):
            y = run(g, {"x": x, "z": z}, ["y"], dev)[0] / so
            assert np.abs(y - np.rint(y)).max() < 1e-3
            out["y%d_%s" % (k, dev.lower())] = np.rint(y).astype(np.int8)
    np.savez_compressed(os.path.join(HERE, "int8_add.npz"), **out)


ALL = {"single_ops": single_ops, "tiny_encoder": tiny_encoder, "config1_summary": config1_summary,
       "int8_ffn": int8_ffn, "int8_encoder": int8_encoder, "int8_add": int8_add}

if __name__ == "__main__":
    assert ref_driver.available(), "oracle/_ref is not built: run `make -C oracle` where the reference tree is present"
    for name in (sys.argv[1:] or list(ALL)):  # no argument: every fixture; else only the named ones
        ALL[name]()
    for f in sorted(os.listdir(HERE)):
        print("%8d  %s" % (os.path.getsize(os.path.join(HERE, f)), f))
