"""The encoder as the reference's decomposed fp32 graph, evaluated with the CPU checker.

Per layer (op list of an ONNX-exported BERT in the reference's op set):
  MatMul(x, Wq^T)+Add(bq), same for k, v; Reshape/Permute to [B,h,S,d]; MatMul(q, k^T); Mul(scale);
  Add(mask); Softmax(-1); MatMul(p, v); Permute/Reshape; MatMul(Wo^T)+Add(bo); Add(residual);
  LayerNorm; MatMul(W1^T)+Add(b1); GELU; MatMul(W2^T)+Add(b2); Add(residual); LayerNorm.
"""
import numpy as np

import orc


def linear(x, w, b):
    """MatMul with the weight stored [K,N] (weight_position=1) followed by Add(bias)."""
    y = orc.matmul(x, np.ascontiguousarray(w.T))
    return orc.binary("add", y, b)


def attention_layer(x, lw, B, S, heads, mask):
    H = x.shape[1]
    d = H // heads
    q = linear(x, lw["wq"], lw["bq"]).reshape(B, S, heads, d)
    k = linear(x, lw["wk"], lw["bk"]).reshape(B, S, heads, d)
    v = linear(x, lw["wv"], lw["bv"]).reshape(B, S, heads, d)
    q, k, v = (orc.permute(t, (0, 2, 1, 3)) for t in (q, k, v))
    ctx = orc.attention_core(q, k, v, np.float32(1.0 / np.sqrt(d)), mask)
    ctx = orc.permute(ctx, (0, 2, 1, 3)).reshape(B * S, H)
    return linear(ctx, lw["wo"], lw["bo"])


def encoder_layer(x, lw, B, S, heads, mask, eps):
    a = attention_layer(x, lw, B, S, heads, mask)
    x1 = orc.layernorm(orc.binary("add", x, a), lw["ln1_g"], lw["ln1_b"], eps)
    h = orc.gelu(linear(x1, lw["w1"], lw["b1"]))
    y = linear(h, lw["w2"], lw["b2"])
    return orc.layernorm(orc.binary("add", x1, y), lw["ln2_g"], lw["ln2_b"], eps)


def embed(w, ids, seg, eps):
    B, S = ids.shape
    H = w["word_emb"].shape[1]
    we = orc.gather(w["word_emb"], ids.reshape(-1))[0].reshape(B, S, H)
    pe = orc.gather(w["pos_emb"], np.arange(S, dtype=np.int32))[0]
    te = orc.gather(w["type_emb"], seg.reshape(-1))[0].reshape(B, S, H)
    x = orc.binary("add", orc.binary("add", we, pe), te)
    return orc.layernorm(x.reshape(B * S, H), w["emb_ln_g"], w["emb_ln_b"], eps)


def encoder(w, cfg, x, B, S, mask):
    for lw in w["layers"]:
        x = encoder_layer(x, lw, B, S, cfg.heads, mask, cfg.eps)
    return x


def int8_encoder(w, cfg, scales, x0, B, S, mask, quantize=None):
    """The graph of tnn_amd.quant.int8_encoder_graph evaluated with the checker: every projection is
    quantise(input) -> int8 FC (int32 accumulate, requantise) -> dequantise; everything else in fp32.
    `quantize` is orc.quantize_x86 (multiply by the reciprocal scale, the x86 Reformat) or orc.quantize_naive (divide).
    Returns (last hidden [T,H] fp32, {blob name: int8 array} of every int8 blob)."""
    from tnn_amd import quant
    quantize = quantize or orc.quantize_x86
    heads, d = cfg.heads, cfg.head_dim
    q8 = {}

    def qfc(src_name, src, dst_name, wt, bias):
        w_q, b_q, w_s = quant.quantize_fc_params(wt, bias, scales[src_name])
        if src_name not in q8:
            q8[src_name] = quantize(src, scales[src_name])
        y, _ = orc.fc_int8(q8[src_name], w_q, b_q, orc.fc_int8_scale(w_s, scales[dst_name], w_q.shape[0]))
        q8[dst_name] = y
        return orc.dequantize(y, scales[dst_name])

    x, xn = x0, "x0"
    for li, lw in enumerate(w["layers"]):
        p = "l%d_" % li
        q, k, v = (qfc(xn, x, p + nm + "_o", lw["w" + nm], lw["b" + nm]).reshape(B, S, heads, d) for nm in "qkv")
        q, k, v = (orc.permute(t, (0, 2, 1, 3)) for t in (q, k, v))
        ctx = orc.attention_core(q, k, v, np.float32(1.0 / np.sqrt(d)), mask)
        ctx = orc.permute(ctx, (0, 2, 1, 3)).reshape(B * S, cfg.hidden)
        a = qfc(p + "ctx", ctx, p + "attn_o", lw["wo"], lw["bo"])
        x1 = orc.layernorm(orc.binary("add", x, a), lw["ln1_g"], lw["ln1_b"], cfg.eps)
        h = orc.gelu(qfc(p + "x1", x1, p + "ffn1_o", lw["w1"], lw["b1"]))
        y = qfc(p + "act", h, p + "ffn2_o", lw["w2"], lw["b2"])
        x = orc.layernorm(orc.binary("add", x1, y), lw["ln2_g"], lw["ln2_b"], cfg.eps)
        xn = p + "x2"
    return x, q8
