"""Synthetic BERT-style encoder on the fused DEVICE_ROCM kernels (driven through the C ABI).

The graph is the post-LN encoder the reference runs as a decomposed op list
(MatMul/Add, Reshape/Permute, MatMul, Mul, Add(mask), Softmax, MatMul, Permute/Reshape, MatMul/Add,
Add, LayerNorm, MatMul/Add, GELU, MatMul/Add, Add, LayerNorm); here each encoder layer is seven
launches: QKV GEMM(+bias) -> fused attention -> out-proj GEMM(+bias+residual) -> LayerNorm ->
FFN1 GEMM(+bias+GELU) -> FFN2 GEMM(+bias+residual) -> LayerNorm.

Weights follow the benchmark description: N(0, 0.02) matrices, zero biases unless asked otherwise,
LayerNorm gamma=1 / beta=0, eps 1e-12, additive padding mask 0 / -10000.
"""
import math

import numpy as np
import torch

from . import ops

MASK_VALUE = -10000.0


class EncoderConfig:
    def __init__(self, layers=12, hidden=768, heads=12, ffn=3072, vocab=30522, max_pos=512, type_vocab=2,
                 eps=1e-12):
        self.layers, self.hidden, self.heads, self.ffn = layers, hidden, heads, ffn
        self.vocab, self.max_pos, self.type_vocab, self.eps = vocab, max_pos, type_vocab, eps
        assert hidden % heads == 0
        self.head_dim = hidden // heads

    @staticmethod
    def bert_base(layers=12):
        return EncoderConfig(layers, 768, 12, 3072)

    @staticmethod
    def bert_large(layers=24):
        return EncoderConfig(layers, 1024, 16, 4096)

    def flops_per_sequence(self, S):
        """Algorithmic FLOPs (2 per MAC) of the padded-dense encoder for one sequence of length S."""
        H, F = self.hidden, self.ffn
        return self.layers * (8 * S * H * H + 4 * S * S * H + 4 * S * H * F)


def make_weights(cfg, seed=20240601, bias_std=0.0, with_embeddings=True):
    """fp32 master weights as numpy arrays (one dict per layer)."""
    rng = np.random.default_rng(seed)
    H, F = cfg.hidden, cfg.ffn

    def mat(n, k):
        return (rng.standard_normal((n, k)) * 0.02).astype(np.float32)

    def vec(n):
        return (rng.standard_normal(n) * bias_std).astype(np.float32) if bias_std else np.zeros(n, np.float32)

    w = {"layers": []}
    if with_embeddings:
        w["word_emb"] = mat(cfg.vocab, H)
        w["pos_emb"] = mat(cfg.max_pos, H)
        w["type_emb"] = mat(cfg.type_vocab, H)
        w["emb_ln_g"], w["emb_ln_b"] = np.ones(H, np.float32), np.zeros(H, np.float32)
    for _ in range(cfg.layers):
        w["layers"].append({
            "wq": mat(H, H), "wk": mat(H, H), "wv": mat(H, H), "wo": mat(H, H),
            "bq": vec(H), "bk": vec(H), "bv": vec(H), "bo": vec(H),
            "ln1_g": np.ones(H, np.float32), "ln1_b": np.zeros(H, np.float32),
            "w1": mat(F, H), "b1": vec(F), "w2": mat(H, F), "b2": vec(H),
            "ln2_g": np.ones(H, np.float32), "ln2_b": np.zeros(H, np.float32),
        })
    return w


def make_inputs(cfg, B, S, len_lo, len_hi, seed=7):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, cfg.vocab, (B, S)).astype(np.int32)
    split = rng.integers(1, S, B)
    seg = (np.arange(S)[None, :] >= split[:, None]).astype(np.int32)
    lens = rng.integers(len_lo, len_hi + 1, B).astype(np.int32)
    mask = np.where(np.arange(S)[None, :] < lens[:, None], 0.0, MASK_VALUE).astype(np.float32)
    return ids, seg, lens, mask


class DeviceEncoder:
    """Weights resident in HBM in the compute dtype; forward() enqueues the whole encoder."""

    def __init__(self, cfg, weights, dtype=torch.float16, device="cuda"):
        self.cfg, self.dtype = cfg, dtype

        def d(a, dt=dtype):
            return torch.from_numpy(np.ascontiguousarray(a)).to(device).to(dt)

        self.emb = None
        if "word_emb" in weights:
            self.emb = {"word": d(weights["word_emb"]), "pos": d(weights["pos_emb"]), "type": d(weights["type_emb"]),
                        "g": d(weights["emb_ln_g"], torch.float32), "b": d(weights["emb_ln_b"], torch.float32)}
        self.layers = []
        for lw in weights["layers"]:
            self.layers.append({
                "wqkv": d(np.concatenate([lw["wq"], lw["wk"], lw["wv"]], 0)),
                "bqkv": d(np.concatenate([lw["bq"], lw["bk"], lw["bv"]]), torch.float32),
                "wo": d(lw["wo"]), "bo": d(lw["bo"], torch.float32),
                "ln1_g": d(lw["ln1_g"], torch.float32), "ln1_b": d(lw["ln1_b"], torch.float32),
                "w1": d(lw["w1"]), "b1": d(lw["b1"], torch.float32),
                "w2": d(lw["w2"]), "b2": d(lw["b2"], torch.float32),
                "ln2_g": d(lw["ln2_g"], torch.float32), "ln2_b": d(lw["ln2_b"], torch.float32),
            })
        self._ws = {}
        self.hook = None  # optional callable(name, fn) used by the bench to time individual launches

    def _buf(self, name, shape, dtype=None):
        key = (name, tuple(shape), dtype or self.dtype)
        t = self._ws.get(key)
        if t is None:
            t = torch.empty(*shape, dtype=dtype or self.dtype, device="cuda")
            self._ws[key] = t
        return t

    def _run(self, name, fn):
        return self.hook(name, fn) if self.hook else fn()

    def embed(self, ids, seg):
        B, S = ids.shape
        H = self.cfg.hidden
        e = self.emb
        pos_ids = self._buf("pos_ids", (S,), torch.int32)
        pos_ids.copy_(torch.arange(S, dtype=torch.int32, device="cuda"))
        we, _ = ops.gather(e["word"], ids.reshape(-1))
        te, _ = ops.gather(e["type"], seg.reshape(-1))
        pe, _ = ops.gather(e["pos"], pos_ids)
        x = ops.binary("add", we.view(B, S, H), pe.view(S, H))
        x = ops.binary("add", x, te.view(B, S, H))
        return ops.layernorm(x.view(B * S, H), e["g"], e["b"], self.cfg.eps)

    def forward_hidden(self, x, B, S, mask=None, kv_len=None):
        """x: [B*S, H] in the compute dtype; returns the last hidden state [B*S, H]."""
        cfg = self.cfg
        T, H, F = B * S, cfg.hidden, cfg.ffn
        scale = 1.0 / math.sqrt(cfg.head_dim)
        qkv = self._buf("qkv", (T, 3 * H))
        ctx = self._buf("ctx", (T, H))
        t1 = self._buf("t1", (T, H))
        x1 = self._buf("x1", (T, H))
        hbuf = self._buf("h", (T, F))
        t2 = self._buf("t2", (T, H))
        xbufs = [self._buf("xa", (T, H)), self._buf("xb", (T, H))]
        if kv_len is None and mask is not None:
            kv_len = ops.mask_to_kv_len(mask)
        for i, L in enumerate(self.layers):
            xo = xbufs[i & 1]
            self._run("gemm_qkv", lambda: ops.gemm(x, L["wqkv"], True, bias=L["bqkv"], out=qkv))
            self._run("attention", lambda: ops.attention_packed(qkv, B, S, cfg.heads, scale, mask=mask, kv_len=kv_len,
                                                                out=ctx))
            self._run("gemm_out", lambda: ops.gemm(ctx, L["wo"], True, bias=L["bo"], residual=x, out=t1))
            self._run("layernorm", lambda: _ln_into(t1, L["ln1_g"], L["ln1_b"], cfg.eps, x1))
            self._run("gemm_ffn1", lambda: ops.gemm(x1, L["w1"], True, bias=L["b1"], gelu=True, out=hbuf))
            self._run("gemm_ffn2", lambda: ops.gemm(hbuf, L["w2"], True, bias=L["b2"], residual=x1, out=t2))
            self._run("layernorm", lambda: _ln_into(t2, L["ln2_g"], L["ln2_b"], cfg.eps, xo))
            x = xo
        return x

    def forward(self, ids, seg, mask=None, kv_len=None):
        B, S = ids.shape
        x = self.embed(ids, seg)
        return self.forward_hidden(x, B, S, mask, kv_len)


def _ln_into(x, g, b, eps, out):
    from . import capi
    capi.call("tnn_rocm_layernorm", torch.cuda.current_stream().cuda_stream, ops.dt(x), x.data_ptr(), None,
              g.data_ptr(), b.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], float(eps), None, 0.0)
    return out
