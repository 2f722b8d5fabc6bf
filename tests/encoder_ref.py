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


def encoder_blobs(w, cfg, ids, seg, B, S, mask):
    """Every named blob of tnn_amd.tnnmodel.encoder_graph that is a whole tensor of the decomposed graph and may
    survive the device's fusion passes, as the CPU evaluates it: {blob name: array}.  Used as the CPU side of the
    per-blob model check."""
    out = {}
    x = embed(w, ids, seg, cfg.eps)
    out["x0"] = x
    H, heads, d = cfg.hidden, cfg.heads, cfg.head_dim
    for li, lw in enumerate(w["layers"]):
        p = "l%d_" % li
        q, k, v = (linear(x, lw["w" + n], lw["b" + n]) for n in "qkv")
        out[p + "q_o"], out[p + "k_o"], out[p + "v_o"] = q, k, v
        q4, k4, v4 = (orc.permute(t.reshape(B, S, heads, d), (0, 2, 1, 3)) for t in (q, k, v))
        ctx = orc.attention_core(q4, k4, v4, np.float32(1.0 / np.sqrt(d)), mask)
        ctx = orc.permute(ctx, (0, 2, 1, 3)).reshape(B * S, H)
        out[p + "ctx"] = ctx
        a = linear(ctx, lw["wo"], lw["bo"])
        out[p + "attn_o"] = a
        s1 = orc.binary("add", x, a)
        out[p + "sum1"] = s1
        x1 = orc.layernorm(s1, lw["ln1_g"], lw["ln1_b"], cfg.eps)
        out[p + "x1"] = x1
        f1 = linear(x1, lw["w1"], lw["b1"])
        out[p + "ffn1_o"] = f1
        h = orc.gelu(f1)
        out[p + "act"] = h
        f2 = linear(h, lw["w2"], lw["b2"])
        out[p + "ffn2_o"] = f2
        s2 = orc.binary("add", x1, f2)
        out[p + "sum2"] = s2
        x = orc.layernorm(s2, lw["ln2_g"], lw["ln2_b"], cfg.eps)
        out["last_hidden" if li == cfg.layers - 1 else p + "x2"] = x
    return out


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
