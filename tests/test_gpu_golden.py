"""The HIP path against the committed fixtures of tests/golden/ (outputs of the reference engine's own DEVICE_NAIVE /
DEVICE_X86 runs).  Everything goes through the host C ABI or the kernel C ABI; no checker is involved."""
import numpy as np
import pytest

import golden_util
from test_gpu_ops import rel_err, say, FP16_TOL, FP32_TOL, FP32_ASSERT

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def test_single_ops_against_reference_naive():
    from tnn_amd import ops
    f = golden_util.load("single_ops_naive.npz")
    say("golden: GELU / LayerNorm / Softmax / MatMul kernels vs reference NAIVE fixtures")
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    got = ops.gelu(d(f["gelu_x"])).cpu().numpy()
    assert rel_err(got, f["gelu_y"]) <= 1e-6  # device erff vs the CPU's double erf
    got = ops.layernorm(d(f["ln_x"]), d(f["ln_g"]), d(f["ln_b"]), 1e-12).cpu().numpy()
    assert rel_err(got, f["ln_y"]) <= 1e-5
    for axis in (1, 3):
        got = ops.softmax(d(f["softmax_x"]), axis).cpu().numpy()
        assert np.abs(got - f["softmax_y_axis%d" % axis]).max() <= 1e-6
        if axis == 3:
            assert np.all(got[0, 0, 0, 20:] == 0.0)
    got = ops.gemm(d(f["matmul_a"]), d(f["matmul_b"]), b_is_nk=False).cpu().numpy()
    assert rel_err(got, f["matmul_y"]) <= 1e-5 <= FP32_TOL


@pytest.mark.parametrize("precision", ["fp32", "fp16"])
def test_tiny_encoder_from_model_files(precision):
    from tnn_amd import host, tnnmodel
    cfg, w, B, S, f = golden_util.tiny_encoder()
    say("golden: tiny encoder (embeddings + mask) on the host, " + precision)
    g = tnnmodel.encoder_graph(cfg, w, B, S, extra_outputs=["x0"])
    inst = host.RocmInstance.from_graph(g, precision)
    inst.set_input("input_ids", f["ids"])
    inst.set_input("token_type_ids", f["seg"])
    inst.set_input("attention_bias", f["mask"].reshape(B, 1, 1, S))
    inst.forward()
    got = inst.output("last_hidden")
    err = rel_err(got, f["naive_last_hidden"].reshape(got.shape))
    say("  max rel err %.3g" % err)
    assert err <= (FP32_ASSERT if precision == "fp32" else FP16_TOL)
    if precision == "fp32":
        assert err <= 1e-4
        assert rel_err(inst.output("x0"), f["naive_x0"].reshape(inst.output("x0").shape)) <= 1e-5
    inst.close()


def test_config1_attention_layer_fp32():
    from tnn_amd import host, tnnmodel
    lw, x, f = golden_util.config1_inputs()
    say("golden: config-1 attention layer, fp32, vs reference NAIVE digest + slices")
    inst = host.RocmInstance.from_graph(tnnmodel.attention_layer_graph(lw, 128, 768, 12), "fp32")
    inst.set_input("x", x)
    inst.forward()
    y = inst.output("y")
    inst.close()
    scale = float(np.abs(f["y_rows_0_8"]).max())
    assert np.abs(y[:8] - f["y_rows_0_8"]).max() / scale <= 1e-5
    assert np.abs(y[120:] - f["y_rows_120_128"]).max() / scale <= 1e-5
    assert abs(float(np.abs(y).astype(np.float64).sum()) - float(f["y_abs_sum"])) / float(f["y_abs_sum"]) <= 1e-6


def test_int8_ffn_bit_exact_against_reference_x86():
    from tnn_amd import host, tnnmodel
    f = golden_util.load("int8_ffn.npz")
    say("golden: int8 FFN on the host vs reference X86 fixture")
    T, K = f["x"].shape
    F = f["w1"].shape[0]
    g = tnnmodel.int8_ffn_graph(T, K, F, f["w1"], f["b1"], f["ws1"], f["w2"], f["b2"], f["ws2"],
                                *(np.float32(v) for v in f["scales"]))
    inst = host.RocmInstance.from_graph(g, "fp32")
    inst.set_input("x", f["x"])
    inst.forward()
    got = inst.output("y")
    inst.close()
    s_y = np.float32(f["scales"][3])
    diff = np.abs(np.rint(got / s_y) - np.rint(f["y_x86"] / s_y))
    say("  mismatching int8 outputs: %d of %d" % (int((diff != 0).sum()), diff.size))
    assert diff.max() == 0  # int8 GEMMs, quantisers and the GELU between them (double erf) are all bit-exact


@pytest.mark.parametrize("case", [0, 1])
def test_int8_add_graph_bit_exact_against_reference_x86(case):
    """QuantizedAdd through the host (Reformat layers inserted by the optimizer, RocmBinaryLayerAcc<Add> on int8
    blobs) over all 65536 (a, b) pairs against the reference's DEVICE_X86 run."""
    from tnn_amd import host, tnnmodel
    qa, qb, x, z, sa, sb, so = golden_util.int8_add_case(case)
    say("golden: QuantizedAdd graph on the host vs reference X86 fixture, scales %d" % case)
    inst = host.RocmInstance.from_graph(tnnmodel.int8_add_graph(golden_util.INT8_ADD_DIMS, sa, sb, so), "fp32")
    types = [t for t, _ in inst.layers()]
    assert types.count("Reformat") == 3 and types.count("QuantizedAdd") == 1, types
    inst.set_input("x", x)
    inst.set_input("z", z)
    inst.forward()
    got = inst.output("y") / so
    inst.close()
    assert np.abs(got - np.rint(got)).max() < 1e-3
    assert np.array_equal(np.rint(got).astype(np.int8), golden_util.load("int8_add.npz")["y%d_x86" % case])


@pytest.mark.parametrize("precision", ["fp32", "fp16"])
def test_int8_encoder_against_reference_x86(precision):
    """Int8 encoder (QuantizedInnerProduct projections, float attention core / LayerNorm / GELU) on the host:
    each projection is bit-exact given its own input blob; the network output stays within the float bar of the
    reference's DEVICE_X86 run."""
    import orc
    from tnn_amd import host, quant
    cfg, w, B, S, scales, f = golden_util.int8_encoder()
    say("golden: int8 encoder on the host vs reference X86 fixture, " + precision)
    blobs = ["x0"] + ["l0_" + b for b in quant.CALIBRATION_BLOBS]
    g = quant.int8_encoder_graph(cfg, w, scales, B, S, extra_outputs=blobs)
    inst = host.RocmInstance.from_graph(g, precision)
    types = [t for t, _ in inst.layers()]
    say("  layers: " + " ".join(sorted(set(types))))
    assert types.count("QuantizedInnerProduct") == 6
    inst.set_input("input_ids", f["ids"])
    inst.set_input("token_type_ids", f["seg"])
    inst.set_input("attention_bias", f["mask"].reshape(B, 1, 1, S))
    inst.forward()
    got = inst.output("last_hidden")
    mine = {n: inst.output(n) for n in blobs}
    inst.close()
    # float blobs that feed a projection are quantised by the Reformat kernel with the reciprocal scale, as on x86;
    # in fp16 mode those blobs are fp16 values, which the read-back reproduces exactly
    assert golden_util.check_projections_bit_exact(cfg, w, scales, mine, B * S, orc.quantize_x86) == 6
    ref = f["x86_last_hidden"].reshape(got.shape)
    err = rel_err(got, ref)
    say("  max rel err vs X86 %.3g" % err)
    # one int8 step of a projection output is ~1/127 of its range, so a float difference upstream that flips a
    # rounding moves the result by more than the float bar; the bound below is two such steps on the final LayerNorm
    assert err <= (2e-2 if precision == "fp16" else 1e-2)


@pytest.mark.parametrize("precision", ["fp32", "fp16"])
def test_int8_encoder_with_folded_reformat_layers(precision, monkeypatch):
    """The same int8 encoder without extra outputs, so that the ROCm int8 pass may fold every Reformat layer into its
    neighbour (projection + dequantise + residual, LayerNorm + quantise, int8 GELU, quantised attention block):
    in fp32 the result is bit-identical to the explicit chain, in fp16 it stays within the bar of the X86 fixture."""
    from tnn_amd import host, quant
    cfg, w, B, S, scales, f = golden_util.int8_encoder()
    say("golden: int8 encoder, Reformat layers folded, " + precision)
    g = quant.int8_encoder_graph(cfg, w, scales, B, S)
    outs, types = {}, {}
    for fuse in ("0", "1"):
        monkeypatch.setenv("TNN_ROCM_FUSE_INT8", fuse)
        inst = host.RocmInstance.from_graph(g, precision)
        types[fuse] = [t for t, _ in inst.layers()]
        inst.set_input("input_ids", f["ids"])
        inst.set_input("token_type_ids", f["seg"])
        inst.set_input("attention_bias", f["mask"].reshape(B, 1, 1, S))
        inst.forward()
        outs[fuse] = inst.output("last_hidden")
        inst.close()
    say("  explicit: " + " ".join("%s x%d" % (t, types["0"].count(t)) for t in sorted(set(types["0"]))))
    say("  folded:   " + " ".join("%s x%d" % (t, types["1"].count(t)) for t in sorted(set(types["1"]))))
    assert types["0"].count("Reformat") == 10 and types["0"].count("QuantizedInnerProduct") == 6
    # FFN1 and its int8 GELU are one layer (the GELU chain as a table in the projection's epilogue)
    assert types["1"].count("RocmQuantLinearGelu") == 1 and types["1"].count("QuantizedInnerProduct") == 0
    if precision == "fp16":
        # only the encoder input is still quantised by a layer of its own: the attention kernel writes its quantised
        # context itself
        assert types["1"].count("Reformat") == 1
        assert types["1"].count("RocmFusedAttention") == 1 and types["1"].count("RocmFusedLinearInt8") == 2
    else:  # fp32 keeps the decomposed attention core; the q, k, v projections still fold their Reformat layers
        assert types["1"].count("Reformat") == 2 and types["1"].count("RocmFusedLinearInt8") == 5
        assert np.array_equal(outs["0"], outs["1"])
    ref = f["x86_last_hidden"].reshape(outs["1"].shape)
    err = rel_err(outs["1"], ref)
    say("  max rel err vs X86 %.3g (explicit chain %.3g)" % (err, rel_err(outs["0"], ref)))
    assert err <= (2e-2 if precision == "fp16" else 1e-2)
