"""Offline int8 preparation of the encoder's projections, following the reference's calibration tool
(reference tools/quantization/calibration.cc:600-675 QuantizeFcParams, :677-701 CalQuantizedWeights MIN_MAX):

    w'        = w * s_in                                 (fp32; s_in = per-tensor scale of the layer's input blob)
    w_scale   = max|w'[oc, :]| / 127                     (fp32, per output channel)
    w_q       = clamp(round(w' * (1 / w_scale)), -127, 127)      (std::round: halves away from zero)
    bias_q    = (int32)(bias / w_scale)                  (C truncation; 0 where w_scale == 0)

Activation scales are per tensor, max|x| / 127 over the calibration run.  This is model preparation, not part of
the forward path: the quantised tensors are written into the .tnnmodel like any other weights."""
import numpy as np

from . import tnnmodel


def activation_scale(x):
    return np.float32(np.float32(np.abs(np.asarray(x, np.float32)).max()) / np.float32(127.0))


def quantize_fc_params(w_nk, bias, s_in):
    """w_nk [N,K] fp32, bias [N] fp32, s_in scalar -> (w_q int8 [N,K], bias_q int32 [N], w_scale fp32 [N])"""
    w = np.asarray(w_nk, np.float32) * np.float32(s_in)
    max_abs = np.maximum(np.abs(w.min(axis=1)), np.abs(w.max(axis=1))).astype(np.float32)
    w_scale = (max_abs / np.float32(127.0)).astype(np.float32)
    inv = np.where(max_abs != 0, np.float32(1.0) / np.where(w_scale != 0, w_scale, np.float32(1.0)), np.float32(1.0))
    t = (w * inv.astype(np.float32)[:, None]).astype(np.float32).astype(np.float64)
    r = np.sign(t) * np.floor(np.abs(t) + 0.5)  # exact in double: std::round of an fp32 value
    w_q = np.clip(r, -127, 127).astype(np.int8)
    b = np.asarray(bias, np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        bq = np.where(w_scale != 0, np.trunc((b / np.where(w_scale != 0, w_scale, np.float32(1.0))).astype(np.float32)), 0.0)
    return w_q, bq.astype(np.int32), w_scale


# blobs of tnnmodel.encoder_graph whose ranges calibrate the int8 encoder (per layer prefix "l<i>_"; the layer
# input is x0 or the previous layer's output)
CALIBRATION_BLOBS = ("q_o", "k_o", "v_o", "ctx", "attn_o", "x1", "ffn1_o", "act", "ffn2_o")


def calibration_outputs(cfg):
    """names to request as extra outputs of tnnmodel.encoder_graph for a calibration forward"""
    names = ["x0"]
    for li in range(cfg.layers):
        names += ["l%d_%s" % (li, b) for b in CALIBRATION_BLOBS]
        if li + 1 < cfg.layers:
            names.append("l%d_x2" % li)
    return names


def scales_from_activations(acts):
    return {k: activation_scale(v) for k, v in acts.items()}


def int8_encoder_graph(cfg, weights, scales, B, S, extra_outputs=()):
    """The encoder with every projection as QuantizedInnerProduct (int8 in, int32 accumulate, int8 out) and
    everything else (attention core, residual adds, LayerNorm, GELU) in floating point.  The float<->int8 Reformat
    layers are not written: the engine's optimizer inserts them wherever a quantised layer meets a float one
    (reference source/tnn/optimizer/net_optimizer_insert_int8_reformat.cc:66-181).  Inputs and output as
    tnnmodel.encoder_graph; inside, token tensors are [B*S, H]."""
    g = tnnmodel.Graph()
    H, h, d, T = cfg.hidden, cfg.heads, cfg.head_dim, B * S
    g.add_input("input_ids", [B, S], tnnmodel.DT_INT32)
    g.add_input("token_type_ids", [B, S], tnnmodel.DT_INT32)
    g.add_input("attention_bias", [B, 1, 1, S], tnnmodel.DT_FLOAT)
    g.add_layer("Gather", "emb_word", ["input_ids"], ["emb_word_o"], [0, 1, 0])
    g.res_gather("emb_word", weights["word_emb"])
    g.add_layer("Gather", "emb_type", ["token_type_ids"], ["emb_type_o"], [0, 1, 0])
    g.res_gather("emb_type", weights["type_emb"])
    g.add_layer("Add", "emb_pos", ["emb_word_o"], ["emb_pos_o"], [1])
    g.res_eltwise("emb_pos", "Add", weights["pos_emb"][:S])
    g.add_layer("Add", "emb_sum", ["emb_pos_o", "emb_type_o"], ["emb_sum_o"], [1])
    g.add_constant("emb_ln_gamma", weights["emb_ln_g"])
    g.add_constant("emb_ln_beta", weights["emb_ln_b"])
    g.add_layer("LayerNorm", "emb_ln", ["emb_sum_o", "emb_ln_gamma", "emb_ln_beta"], ["x0_3d"], [1, repr(cfg.eps)])
    g.add_layer("Reshape", "x0_rs", ["x0_3d"], ["x0"], [0, 2, 2, T, H, 0])
    x = "x0"

    scaled_blobs = set()

    def qfc(name, src, dst, w, b, n_out):
        w_q, b_q, w_s = quantize_fc_params(w, b, scales[src])
        g.add_layer("QuantizedInnerProduct", name, [src], [dst], [n_out, 1, 0, 1])
        g.res_inner_product(name, w_q, b_q, quant_scale=w_s)
        for blob in (src, dst):
            if blob not in scaled_blobs:
                g.res_blob_scale(blob, scales[blob])
                scaled_blobs.add(blob)

    for li, lw in enumerate(weights["layers"]):
        p = "l%d_" % li
        for nm in ("q", "k", "v"):
            qfc(p + nm, x, p + nm + "_o", lw["w" + nm], lw["b" + nm], H)
            g.add_layer("Reshape", p + nm + "_rs", [p + nm + "_o"], [p + nm + "_4d"], [0, 4, 4, B, S, h, d, 0])
        g.add_layer("Permute", p + "q_pm", [p + "q_4d"], [p + "qh"], [4, 0, 2, 1, 3])
        g.add_layer("Permute", p + "k_pm", [p + "k_4d"], [p + "kt"], [4, 0, 2, 3, 1])
        g.add_layer("Permute", p + "v_pm", [p + "v_4d"], [p + "vh"], [4, 0, 2, 1, 3])
        g.add_layer("MatMul", p + "qk", [p + "qh", p + "kt"], [p + "scores"], [-1])
        g.add_layer("Mul", p + "scale", [p + "scores"], [p + "scaled"], [1])
        g.res_eltwise(p + "scale", "Mul", np.array([1.0 / np.sqrt(d)], np.float32))
        g.add_layer("Add", p + "mask", [p + "scaled", "attention_bias"], [p + "masked"], [1])
        g.add_layer("Softmax", p + "sm", [p + "masked"], [p + "probs"], [3])
        g.add_layer("MatMul", p + "pv", [p + "probs", p + "vh"], [p + "ctx_h"], [-1])
        g.add_layer("Permute", p + "ctx_pm", [p + "ctx_h"], [p + "ctx_4d"], [4, 0, 2, 1, 3])
        g.add_layer("Reshape", p + "ctx_rs", [p + "ctx_4d"], [p + "ctx"], [0, 2, 2, T, H, 0])
        qfc(p + "o", p + "ctx", p + "attn_o", lw["wo"], lw["bo"], H)
        g.add_layer("Add", p + "res1", [x, p + "attn_o"], [p + "sum1"], [1])
        g.add_constant(p + "ln1_gamma", lw["ln1_g"])
        g.add_constant(p + "ln1_beta", lw["ln1_b"])
        g.add_layer("LayerNorm", p + "ln1", [p + "sum1", p + "ln1_gamma", p + "ln1_beta"], [p + "x1"],
                    [1, repr(cfg.eps)])
        qfc(p + "ffn1", p + "x1", p + "ffn1_o", lw["w1"], lw["b1"], cfg.ffn)
        g.add_layer("GELU", p + "gelu", [p + "ffn1_o"], [p + "act"], [])
        qfc(p + "ffn2", p + "act", p + "ffn2_o", lw["w2"], lw["b2"], H)
        g.add_layer("Add", p + "res2", [p + "x1", p + "ffn2_o"], [p + "sum2"], [1])
        g.add_constant(p + "ln2_gamma", lw["ln2_g"])
        g.add_constant(p + "ln2_beta", lw["ln2_b"])
        g.add_layer("LayerNorm", p + "ln2", [p + "sum2", p + "ln2_gamma", p + "ln2_beta"], [p + "x2"],
                    [1, repr(cfg.eps)])
        x = p + "x2"
    g.add_layer("Reshape", "out_rs", [x], ["last_hidden"], [0, 3, 3, B, S, H, 0])
    g.add_output("last_hidden")
    for e in extra_outputs:
        g.add_output(e)
    return g
