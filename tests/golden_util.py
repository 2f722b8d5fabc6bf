"""Loads the committed fixtures of tests/golden/ (written by tests/golden/make_vectors.py from the reference engine's
own DEVICE_NAIVE / DEVICE_X86 runs) and rebuilds the graphs they belong to."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLDEN, name), allow_pickle=False))


def tiny_encoder():
    """-> (cfg, weights, B, S, fixture dict) of tiny_encoder.npz"""
    from tnn_amd.encoder import EncoderConfig
    f = load("tiny_encoder.npz")
    cfg = EncoderConfig(1, 64, 1, 128, vocab=50, max_pos=32)
    w = {k[2:]: v for k, v in f.items() if k.startswith("w_")}
    w["layers"] = [{k[3:]: v for k, v in f.items() if k.startswith("l0_") and k not in ("l0_probs", "l0_x1")}]
    B, S = f["ids"].shape
    return cfg, w, B, S, f


def config1_inputs():
    """Regenerates the seeded config-1 inputs and checks their digests against the fixture (so a change of the
    generator cannot silently turn the comparison into a different problem)."""
    from tnn_amd.encoder import EncoderConfig, make_weights
    f = load("config1_attention_naive.npz")
    cfg = EncoderConfig(1, 768, 12, 3072)
    lw = make_weights(cfg, seed=1, with_embeddings=False)["layers"][0]
    x = np.random.default_rng(2).standard_normal((128, 768)).astype(np.float32)
    assert float(x.astype(np.float64).sum()) == float(f["x_sum"])
    assert float(np.abs(x).astype(np.float64).sum()) == float(f["x_abs_sum"])
    assert float(lw["wq"].astype(np.float64).sum()) == float(f["wq_sum"])
    assert float(lw["wo"].astype(np.float64).sum()) == float(f["wo_sum"])
    return lw, x, f


def int8_encoder():
    """-> (cfg, weights, B, S, scales, fixture) of int8_encoder_x86.npz; weights are regenerated from the seed and
    checked against the stored digest."""
    from tnn_amd.encoder import EncoderConfig, make_weights
    f = load("int8_encoder_x86.npz")
    cfg = EncoderConfig(1, 128, 2, 256, vocab=1000, max_pos=64)
    w = make_weights(cfg, seed=21, bias_std=0.02)
    digest = sum(float(np.abs(v).astype(np.float64).sum()) for v in w["layers"][0].values())
    assert digest == float(f["w_digest"])
    B, S = f["ids"].shape
    scales = {k[len("scale_"):]: np.float32(v) for k, v in f.items() if k.startswith("scale_")}
    return cfg, w, B, S, scales, f


INT8_ADD_DIMS = [1, 256, 256, 1]
# (scale a, scale b, scale out): a generic triple, and a tie-heavy one (equal input scales, output scale twice that:
# every odd a+b lands on a half-integer, where the x86 form's multiply by float(1/so) and the naive form's division
# round differently for thousands of pairs)
INT8_ADD_SCALES = ((0.031, 0.017, 0.027), (0.031004460528492928, 0.031004460528492928, 0.062008921056985855))


def int8_add_case(k):
    """All 65536 (a, b) int8 pairs as a [1, 256, 256, 1] blob pair: -> (qa, qb, x, z, sa, sb, so); x = qa*sa and
    z = qb*sb are the float inputs whose quantisation gives qa and qb back exactly."""
    sa, sb, so = (np.float32(v) for v in INT8_ADD_SCALES[k])
    qa = np.repeat(np.arange(-128, 128, dtype=np.int8), 256).reshape(INT8_ADD_DIMS)
    qb = np.tile(np.arange(-128, 128, dtype=np.int8), 256).reshape(INT8_ADD_DIMS)
    return qa, qb, qa.astype(np.float32) * sa, qb.astype(np.float32) * sb, sa, sb, so


def int8_projections(cfg, w, li=0):
    """(input blob, output blob, weight [N,K], bias) of the six projections of layer li in the int8 encoder graph"""
    lw, p = w["layers"][li], "l%d_" % li
    xin = "x0" if li == 0 else "l%d_x2" % (li - 1)
    return [(xin, p + "q_o", lw["wq"], lw["bq"]), (xin, p + "k_o", lw["wk"], lw["bk"]), (xin, p + "v_o", lw["wv"], lw["bv"]),
            (p + "ctx", p + "attn_o", lw["wo"], lw["bo"]), (p + "x1", p + "ffn1_o", lw["w1"], lw["b1"]),
            (p + "act", p + "ffn2_o", lw["w2"], lw["b2"])]


def check_projections_bit_exact(cfg, w, scales, blobs, T, quantize, layers=None, rows=None):
    """Teacher forcing: every projection, fed with the float blob the run itself produced (quantised as its Reformat
    layer does), must reproduce the run's own int8 output exactly.  `blobs` maps blob name -> dequantised array."""
    import orc
    from tnn_amd import quant
    n = 0
    for li in (range(cfg.layers) if layers is None else layers):
        for src, dst, wt, bias in int8_projections(cfg, w, li):
            if src not in blobs or dst not in blobs:
                continue
            w_q, b_q, w_s = quant.quantize_fc_params(wt, bias, scales[src])
            sel = slice(None) if rows is None else slice(0, rows)  # a row subset keeps full-size cases fast
            src_q = quantize(np.ascontiguousarray(blobs[src], np.float32).reshape(T, -1)[sel], scales[src])
            y, acc = orc.fc_int8(src_q, w_q, b_q, orc.fc_int8_scale(w_s, scales[dst], w_q.shape[0]))
            got = blobs[dst].reshape(T, -1)[sel] / scales[dst]
            assert np.abs(got - np.rint(got)).max() < 1e-3, dst
            bad = int((np.rint(got).astype(np.int8) != y).sum())
            assert bad == 0, "%s: %d of %d int8 outputs differ" % (dst, bad, y.size)
            n += 1
    return n
