"""The CPU checker against the committed fixtures (outputs of the reference engine itself, see
tests/golden/make_vectors.py).  Runs without the reference tree and without a GPU."""
import numpy as np

import encoder_ref
import golden_util
import orc


def test_single_ops_bit_identical_to_reference_naive():
    f = golden_util.load("single_ops_naive.npz")
    assert np.array_equal(orc.gelu(f["gelu_x"]), f["gelu_y"])
    assert np.array_equal(orc.layernorm(f["ln_x"], f["ln_g"], f["ln_b"], 1e-12), f["ln_y"])
    for axis in (1, 3):
        assert np.array_equal(orc.softmax(f["softmax_x"], axis), f["softmax_y_axis%d" % axis])
    assert np.all(f["softmax_y_axis3"][0, 0, 0, 20:] == 0.0)  # masked keys: exact zeros
    assert np.array_equal(orc.matmul(f["matmul_a"], f["matmul_b"]), f["matmul_y"])
    # the fixtures also satisfy what the mathematics fixes (guards against a fixture written from a broken build)
    assert np.allclose(f["softmax_y_axis3"].sum(-1), 1.0, atol=1e-6)
    x = f["gelu_x"].astype(np.float64)
    from scipy.special import erf
    assert np.allclose(f["gelu_y"], 0.5 * x * (1 + erf(x / np.sqrt(2))), rtol=0, atol=2e-6)
    a, b = f["matmul_a"].astype(np.float64), f["matmul_b"].astype(np.float64)
    assert np.allclose(f["matmul_y"], a @ b, atol=1e-5)


def test_tiny_encoder_bit_identical_to_reference_naive():
    cfg, w, B, S, f = golden_util.tiny_encoder()
    x0 = encoder_ref.embed(w, f["ids"], f["seg"], cfg.eps)
    assert np.array_equal(x0, f["naive_x0"].reshape(B * S, -1))
    out = encoder_ref.encoder(w, cfg, x0, B, S, f["mask"])
    assert np.array_equal(out, f["naive_last_hidden"].reshape(B * S, -1))
    # second witness inside the fixture: the reference's DEVICE_X86 path agrees within the fp32 bar
    ref = f["naive_last_hidden"]
    assert np.abs(f["x86_last_hidden"] - ref).max() / np.abs(ref).max() <= 2e-3
    for b in range(B):  # padded keys carry exactly zero probability
        assert np.all(f["naive_l0_probs"][b, :, :, f["lens"][b]:] == 0.0)


def test_config1_attention_layer_bit_identical_to_reference_naive():
    lw, x, f = golden_util.config1_inputs()
    # the config-1 graph uses InnerProduct (fp32 accumulation, reference utils/naive_compute.cc NaiveFC), not MatMul
    q, k, v = (orc.permute(orc.inner_product(x, lw["w" + n], lw["b" + n]).reshape(1, 128, 12, 64), (0, 2, 1, 3))
               for n in "qkv")
    ctx = orc.permute(orc.attention_core(q, k, v, np.float32(0.125)), (0, 2, 1, 3)).reshape(128, 768)
    y = orc.inner_product(ctx, lw["wo"], lw["bo"])
    assert np.array_equal(y[:8], f["y_rows_0_8"]) and np.array_equal(y[120:], f["y_rows_120_128"])
    assert float(y.astype(np.float64).sum()) == float(f["y_sum"])
    assert float(np.abs(y).astype(np.float64).sum()) == float(f["y_abs_sum"])


def test_int8_ffn_bit_identical_to_reference_x86_and_naive():
    f = golden_util.load("int8_ffn.npz")
    s_a, s_h, s_g, s_y = (np.float32(v) for v in f["scales"])
    F, K = f["w1"].shape
    qa = orc.quantize_x86(f["x"], s_a)
    h, acc = orc.fc_int8(qa, f["w1"], f["b1"], orc.fc_int8_scale(f["ws1"], s_h, F))
    # int32 accumulators are exact integers: numpy pins them independently of either implementation
    assert np.array_equal(acc, qa.astype(np.int32) @ f["w1"].astype(np.int32).T + f["b1"])
    gq = orc.quantize_x86(orc.gelu(orc.dequantize(h, s_h)), s_g)
    yq, _ = orc.fc_int8(gq, f["w2"], f["b2"], orc.fc_int8_scale(f["ws2"], s_y, K))
    assert np.array_equal(orc.dequantize(yq, s_y), f["y_x86"])
    assert np.array_equal(f["y_naive"], f["y_x86"])


def test_fc_quantisation_convention():
    """tnn_amd.quant against what the convention fixes: per-channel scale max|w*s_in|/127, weights reach +-127
    exactly on the extreme element, std::round ties, truncated bias, zero rows."""
    from tnn_amd import quant
    w = np.array([[0.5, -1.0, 0.25, 0.0], [0.0, 0.0, 0.0, 0.0], [3.0, 1.5, -0.75, 0.0]], np.float32)
    b = np.array([0.1, 5.0, -0.2], np.float32)
    wq, bq, ws = quant.quantize_fc_params(w, b, np.float32(2.0))
    assert np.allclose(ws, [2.0 / 127, 0.0, 6.0 / 127], rtol=1e-7)
    assert wq[0].tolist() == [64, -127, 32, 0]       # 63.5 -> 64 (half away from zero), 31.75 -> 32
    assert wq[1].tolist() == [0, 0, 0, 0] and bq[1] == 0
    assert wq[2].tolist() == [127, 64, -32, 0]       # 63.5 -> 64, -31.75 -> -32
    assert bq[0] == int(np.float32(0.1) / ws[0]) and bq[2] == int(np.float32(-0.2) / ws[2])  # truncation toward zero
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((64, 96)) * 0.02).astype(np.float32)
    wq, bq, ws = quant.quantize_fc_params(w, np.zeros(64, np.float32), np.float32(0.03))
    assert np.abs(wq).max(axis=1).tolist() == [127] * 64
    assert np.abs(wq.astype(np.float32) * ws[:, None] - w * np.float32(0.03)).max() <= ws.max() * 0.5 * (1 + 1e-6)


def test_int8_encoder_fixture_projections_bit_exact_and_output_close():
    """The committed DEVICE_X86 run of the int8 encoder: the checker reproduces each projection's int8 output exactly
    from the run's own inputs, and the whole network within the fp32 bar."""
    cfg, w, B, S, scales, f = golden_util.int8_encoder()
    blobs = {k[4:]: v for k, v in f.items() if k.startswith("x86_") and k != "x86_last_hidden"}
    assert golden_util.check_projections_bit_exact(cfg, w, scales, blobs, B * S, orc.quantize_x86) == 6
    x0 = encoder_ref.embed(w, f["ids"], f["seg"], cfg.eps)
    mine, _ = encoder_ref.int8_encoder(w, cfg, scales, x0, B, S, f["mask"], orc.quantize_x86)
    ref = f["x86_last_hidden"].reshape(B * S, -1)
    assert np.abs(mine - ref).max() / np.abs(ref).max() <= 2e-3
