"""The C++ host (Instance::Forward on DEVICE_ROCM) fed with the same .tnnproto/.tnnmodel files the reference
engine loads: un-fused fp32 path, fused fp16 path, int8 path, error behaviour."""
import numpy as np
import pytest

import encoder_ref
import orc
from test_gpu_ops import rel_err, say, FP16_TOL, FP32_TOL

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _mods():
    from tnn_amd import host, tnnmodel
    from tnn_amd.encoder import EncoderConfig, make_weights, make_inputs
    return host, tnnmodel, EncoderConfig, make_weights, make_inputs


def r16w(w):
    out = {}
    for k, v in w.items():
        if k == "layers":
            out[k] = [{n: (a.astype(np.float16).astype(np.float32) if a.ndim == 2 else a) for n, a in lw.items()}
                      for lw in v]
        else:
            out[k] = v.astype(np.float16).astype(np.float32) if v.ndim == 2 else v
    return out


def test_config1_attention_layer_fp32_from_model_files():
    host, tnnmodel, EncoderConfig, make_weights, _ = _mods()
    say("host: config-1 attention layer proto, fp32")
    cfg = EncoderConfig(1, 768, 12, 3072)
    lw = make_weights(cfg, seed=1, with_embeddings=False)["layers"][0]
    x = np.random.default_rng(2).standard_normal((128, 768)).astype(np.float32)
    g = tnnmodel.attention_layer_graph(lw, 128, 768, 12)
    inst = host.RocmInstance.from_graph(g, "fp32")
    types = [t for t, _ in inst.layers()]
    say("  layers: " + " ".join(types))
    assert "RocmFusedAttention" not in types          # fp32 keeps the decomposed attention core
    assert types.count("RocmFusedLinear") == 4        # the four InnerProduct projections
    inst.set_input("x", x)
    inst.forward()
    got = inst.output("y")
    ref = encoder_ref.attention_layer(x, lw, 1, 128, 12, None)
    err = rel_err(got, ref)
    say("  max rel err %.3g" % err)
    assert got.shape == (128, 768) and err <= 1e-5 <= FP32_TOL
    inst.close()


@pytest.mark.parametrize("precision", ["fp32", "fp16"])
def test_encoder_from_model_files(precision):
    host, tnnmodel, EncoderConfig, make_weights, make_inputs = _mods()
    say("host: 2-layer encoder proto with embeddings + mask, " + precision)
    cfg = EncoderConfig.bert_base(2)
    w = make_weights(cfg, seed=3, bias_std=0.02)
    B, S = 2, 96
    ids, seg, lens, mask = make_inputs(cfg, B, S, 30, 96, seed=4)
    g = tnnmodel.encoder_graph(cfg, w, B, S)
    inst = host.RocmInstance.from_graph(g, precision)
    types = [t for t, _ in inst.layers()]
    if precision == "fp16":
        # per encoder layer: attention, out-proj(+res), LN, ffn1(+gelu), ffn2(+res), LN = 6 host layers (7 launches)
        assert types.count("RocmFusedAttention") == 2 and types.count("RocmFusedLinear") == 6
        assert not any(t in ("Softmax", "Permute", "Reshape", "MatMul", "GELU") for t in types), types
    else:
        assert types.count("RocmFusedLinear") == 12 and types.count("Softmax") == 2
    inst.set_input("input_ids", ids)
    inst.set_input("token_type_ids", seg)
    inst.set_input("attention_bias", mask.reshape(B, 1, 1, S))
    inst.forward()
    got = inst.output("last_hidden").reshape(B * S, -1)
    wr = r16w(w) if precision == "fp16" else w
    ref = encoder_ref.encoder(wr, cfg, encoder_ref.embed(wr, ids, seg, cfg.eps), B, S, mask)
    err = rel_err(got, ref)
    say("  max rel err %.3g" % err)
    assert err <= (FP16_TOL if precision == "fp16" else 1e-4)
    # second forward with other inputs on the same instance (blob memory is reused between layers)
    ids2, seg2, lens2, mask2 = make_inputs(cfg, B, S, 30, 96, seed=9)
    inst.set_input("input_ids", ids2)
    inst.set_input("token_type_ids", seg2)
    inst.set_input("attention_bias", mask2.reshape(B, 1, 1, S))
    inst.forward()
    got2 = inst.output("last_hidden").reshape(B * S, -1)
    ref2 = encoder_ref.encoder(wr, cfg, encoder_ref.embed(wr, ids2, seg2, cfg.eps), B, S, mask2)
    assert rel_err(got2, ref2) <= (FP16_TOL if precision == "fp16" else 1e-4)
    inst.close()


def test_int8_ffn_from_model_files_bit_exact(monkeypatch):
    host, tnnmodel, *_ = _mods()
    say("host: QuantizedInnerProduct -> GELU -> QuantizedInnerProduct, fp32 boundaries")
    rng = np.random.default_rng(0)
    T, K, F = 256, 768, 3072
    x = rng.standard_normal((T, K)).astype(np.float32)
    w1 = rng.integers(-127, 128, (F, K), dtype=np.int8)
    w2 = rng.integers(-127, 128, (K, F), dtype=np.int8)
    b1 = rng.integers(-500, 500, F).astype(np.int32)
    b2 = rng.integers(-500, 500, K).astype(np.int32)
    ws1 = (rng.uniform(0.5, 1.5, F) * 6e-5).astype(np.float32)
    ws2 = (rng.uniform(0.5, 1.5, K) * 3e-5).astype(np.float32)
    s_a, s_h, s_g, s_y = (np.float32(v) for v in (0.031, 0.045, 0.027, 0.052))
    g = tnnmodel.int8_ffn_graph(T, K, F, w1, b1, ws1, w2, b2, ws2, s_a, s_h, s_g, s_y)
    qa = orc.quantize_x86(x, s_a)
    h, _ = orc.fc_int8(qa, w1, b1, orc.fc_int8_scale(ws1, s_h, F))
    ref_act = orc.gelu(orc.dequantize(h, s_h))
    gq = orc.quantize_x86(ref_act, s_g)
    yq, _ = orc.fc_int8(gq, w2, b2, orc.fc_int8_scale(ws2, s_y, K))
    assert np.abs(h).max() > 20  # the requantisation really exercised the int8 range
    outs = {}
    # once as the explicit chain (Reformat layers as the engine inserts them), once with the Reformat layers folded
    # into their neighbours by the ROCm int8 pass
    for fuse, want in (("0", {"Reformat": 4, "QuantizedInnerProduct": 2}),
                       ("1", {"Reformat": 1, "QuantizedInnerProduct": 1, "RocmGeluInt8": 1, "RocmFusedLinearInt8": 1})):
        monkeypatch.setenv("TNN_ROCM_FUSE_INT8", fuse)
        inst = host.RocmInstance.from_graph(g, "fp32")
        types = [t for t, _ in inst.layers()]
        for k, n in want.items():
            assert types.count(k) == n, types
        inst.set_input("x", x)
        inst.forward()
        got = inst.output("y")
        inst.close()
        # the two int8 GEMMs and both quantisers are bit-exact; the fp32 GELU between them uses the device erff
        # (last-ulp differences against the CPU's double erf), which can move a value across a rounding boundary of
        # the second quantiser in rare cases: allow at most 1 LSB on at most 0.1 % of the outputs
        diff = np.abs(np.rint(got / s_y) - yq.astype(np.float64))
        say("  fuse=%s mismatching int8 outputs: %d of %d" % (fuse, int((diff != 0).sum()), diff.size))
        assert diff.max() <= 1 and (diff != 0).mean() <= 1e-3
        outs[fuse] = got
    assert np.array_equal(outs["0"], outs["1"])  # folding the Reformat layers changes no value in fp32


def test_host_error_paths():
    host, tnnmodel, *_ = _mods()
    say("host: error paths")
    g = tnnmodel.Graph()
    g.add_input("x", [4, 8])
    g.add_layer("GELU", "g", ["x"], ["y"])
    g.add_output("y")
    proto, model = g.proto(), g.model()
    with pytest.raises(host.HostError, match="not supported"):
        host.RocmInstance(proto.replace("GELU g", "Convolution g"), model)   # unknown layer type
    with pytest.raises(host.HostError):
        host.RocmInstance(proto, model[: len(model) // 2] if len(model) > 16 else b"")  # truncated / empty model
    inst = host.RocmInstance(proto, model, "fp32")
    with pytest.raises(host.HostError, match="dont have the input"):
        inst.set_input("nope", np.zeros((4, 8), np.float32))
    with pytest.raises(host.HostError):
        inst.set_input("x", np.zeros((4, 9), np.float32))                    # wrong element count
    inst.close()
    # MatMul with inconsistent shapes is rejected at Init like the engine's shape inference does
    g = tnnmodel.Graph()
    g.add_input("a", [4, 8])
    g.add_input("b", [7, 5])
    g.add_layer("MatMul", "mm", ["a", "b"], ["c"], [-1])
    g.add_output("c")
    with pytest.raises(host.HostError, match="wrong shape"):
        host.RocmInstance(g.proto(), g.model(), "fp32")
    # Gather index out of range surfaces as an error from Forward (the engine returns TNNERR_MODEL_ERR)
    g = tnnmodel.Graph()
    g.add_input("ids", [1, 4], tnnmodel.DT_INT32)
    g.add_layer("Gather", "emb", ["ids"], ["e"], [0, 1, 0])
    g.res_gather("emb", np.ones((10, 8), np.float32))
    g.add_output("e")
    inst = host.RocmInstance(g.proto(), g.model(), "fp32")
    inst.set_input("ids", np.array([[0, 3, 9, 2]], np.int32))
    inst.forward()
    assert inst.output("e").shape == (1, 4, 8)
    inst.set_input("ids", np.array([[0, 3, 10, 2]], np.int32))
    with pytest.raises(host.HostError, match="invalid slice_index"):
        inst.forward()
    inst.close()


def test_graph_replay_matches_eager_on_every_replay(monkeypatch):
    """The whole-forward graph (recorded on the third Forward) must reproduce the eager result on every replay, with
    new inputs each time and unrelated eager GPU work and synchronisations between the replays."""
    host, tnnmodel, EncoderConfig, make_weights, make_inputs = _mods()
    say("host: graph replay vs eager")
    cfg = EncoderConfig.bert_base(2)
    w = make_weights(cfg, seed=13, bias_std=0.02)
    B, S = 2, 128
    g = tnnmodel.encoder_graph(cfg, w, B, S)
    monkeypatch.setenv("TNN_ROCM_GRAPH", "0")
    eager = host.RocmInstance.from_graph(g, "fp16")
    monkeypatch.setenv("TNN_ROCM_GRAPH", "1")
    graph = host.RocmInstance.from_graph(g, "fp16")
    scratch = torch.zeros(1 << 20, device="cuda")
    for it in range(7):
        ids, seg, lens, mask = make_inputs(cfg, B, S, 20, 128, seed=100 + it)
        outs = []
        for inst in (eager, graph):
            inst.set_input("input_ids", ids)
            inst.set_input("token_type_ids", seg)
            inst.set_input("attention_bias", mask.reshape(B, 1, 1, S))
            inst.forward()
            outs.append(inst.output("last_hidden"))
        assert np.array_equal(outs[0], outs[1]), "replay %d differs from eager" % it
        # unrelated eager work + a device synchronisation between replays
        scratch.add_(1.0)
        assert float(scratch.sum().item()) == (it + 1) * (1 << 20)
        torch.cuda.synchronize()
    eager.close()
    graph.close()
