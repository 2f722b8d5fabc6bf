"""Host logic without a GPU: model interpretation, the optimizer passes and shape / type inference of the C++ host
(tnn_host_plan: everything Instance::Init does short of creating a device context), plus its error behaviour."""
import collections

import numpy as np
import pytest

from tnn_amd import host, quant, tnnmodel
from tnn_amd.encoder import EncoderConfig, make_weights


def _graph(layers=2, hidden=256, heads=4, ffn=512, B=2, S=32, seed=1, **kw):
    cfg = EncoderConfig(layers, hidden, heads, ffn)
    w = make_weights(cfg, seed=seed)
    if not kw.get("position_ids"):
        w["pos_emb"] = w["pos_emb"][:S]
    return cfg, w, tnnmodel.encoder_graph(cfg, w, B, S, **kw)


def _types(plan):
    return collections.Counter(l["type"] for l in plan)


def test_fp16_encoder_is_rewritten_into_fused_layers():
    cfg, w, g = _graph()
    plan = host.plan(g, precision="fp16")
    # per layer: fused attention (QKV + core), out-projection, FFN1 (+GELU), FFN2; every residual Add folded;
    # every LayerNorm except the one that produces the model output folded into the projection that reads it
    assert _types(plan) == {"RocmFusedEmbedding": 1, "RocmFusedAttention": 2, "RocmFusedLinear": 6, "LayerNorm": 1}
    by_out = {o: l for l in plan for o in l["outputs"]}
    assert by_out["last_hidden"]["output_dims"] == [[2, 32, 256]]
    att = [l for l in plan if l["type"] == "RocmFusedAttention"]
    assert all(l["inputs"][1] == "attention_bias" for l in att)
    assert all(d == [2, 32, 256] for l in att for d in l["output_dims"])
    ffn1 = [l for l in plan if l["name"].endswith("ffn1_mm") or "ffn1" in l["name"]]
    assert any(l["output_dims"][0] == [2, 32, 512] for l in ffn1)
    # layer order stays topological: every input is a model input, a constant or an earlier output
    seen = {"input_ids", "token_type_ids", "attention_bias"}
    for l in plan:
        for i in l["inputs"]:
            assert i in seen or i.endswith(("gamma", "beta")), (l["name"], i)
        seen.update(l["outputs"])


def test_fp32_keeps_the_decomposed_attention_core():
    _, _, g = _graph()
    t = _types(host.plan(g, precision="fp32"))
    assert "RocmFusedAttention" not in t and t["Softmax"] == 2 and t["MatMul"] == 4 and t["Permute"] == 8
    assert t["RocmFusedLinear"] == 12 and t["LayerNorm"] == 4 and t["RocmFusedEmbedding"] == 1


def test_bf16_plans_like_fp16():
    _, _, g = _graph()
    assert _types(host.plan(g, precision="bf16")) == _types(host.plan(g, precision="fp16"))


def test_layernorm_fold_switch(monkeypatch):
    _, _, g = _graph()
    monkeypatch.setenv("TNN_ROCM_FOLD_LN", "0")
    assert _types(host.plan(g, precision="fp16"))["LayerNorm"] == 4
    monkeypatch.setenv("TNN_ROCM_FOLD_LN", "1")
    assert _types(host.plan(g, precision="fp16"))["LayerNorm"] == 1


def test_row_statistics_hand_over_switch(monkeypatch):
    """A folded LayerNorm whose output is read once more, as the residual of a projection: by default the output tensor
    disappears (the folding layer has one output, the residual reader takes the raw tensor); TNN_ROCM_LN_STATS=0 keeps
    the tensor as a second output."""
    _, _, g = _graph()
    for stats, n_out in (("1", 1), ("0", 2)):
        monkeypatch.setenv("TNN_ROCM_LN_STATS", stats)
        plan = host.plan(g, precision="fp16")
        by_out = {o: l for l in plan for o in l["outputs"]}
        ffn1, ffn2 = by_out["l0_act"], by_out["l0_sum2"]
        assert ffn1["inputs"][0] == "l0_sum1" and len(ffn1["outputs"]) == n_out
        assert ffn2["inputs"] == ["l0_act", "l0_sum1" if stats == "1" else "l0_x1"]
        att, out = by_out["l1_ctx"], by_out["l1_sum1"]
        assert att["inputs"][0] == "l0_sum2" and len(att["outputs"]) == n_out
        assert out["inputs"] == ["l1_ctx", "l0_sum2" if stats == "1" else "l0_x2"]
        assert ("l0_x1" in by_out) == (stats == "0")
        # (which layer hands its output's row sums to which folding layer is not part of the blob graph: covered on
        # the device, where every combination of the switches must give the same encoder output)
        # layer 0 reads the embedding output, which is a LayerNorm output of the embedding layer itself: nothing to rebuild
        assert by_out["l0_sum1"]["inputs"] == ["l0_ctx", "x0"]


def test_width_that_cannot_fold_keeps_its_layernorms():
    # hidden 192 is no multiple of 128: the LayerNorms stay launches of their own, everything else still fuses
    _, _, g = _graph(hidden=192, heads=3, ffn=384)
    t = _types(host.plan(g, precision="fp16"))
    assert t["LayerNorm"] == 4 and t["RocmFusedAttention"] == 2 and t["RocmFusedLinear"] == 6


def test_dynamic_head_split_planned_at_other_shapes():
    _, _, g = _graph(B=4, S=32, dynamic=True)
    shapes = {"input_ids": [3, 24], "token_type_ids": [3, 24], "attention_bias": [3, 1, 1, 24]}
    plan = host.plan(g, precision="fp16", input_shapes=shapes)
    assert _types(plan)["RocmFusedAttention"] == 2 and _types(plan)["LayerNorm"] == 1
    assert [l for l in plan if "last_hidden" in l["outputs"]][0]["output_dims"] == [[3, 24, 256]]
    # the static graph names B and S in its Reshape layers: other input shapes fail in the layer that notices (fp32 keeps
    # those layers)
    _, _, gs = _graph(B=4, S=32)
    with pytest.raises(host.HostError, match="reshape"):
        host.plan(gs, precision="fp32", input_shapes=shapes)
    with pytest.raises(host.HostError, match="not an input"):
        host.plan(g, input_shapes={"nope": [1]})
    with pytest.raises(host.HostError, match="number of dimensions"):
        host.plan(g, input_shapes={"input_ids": [3]})


def test_mask_front_end_position_gather_and_pooler_layers():
    cfg, w, _ = _graph()
    rng = np.random.default_rng(3)
    w["pool_w"] = rng.standard_normal((256, 256)).astype(np.float32)
    w["pool_b"] = rng.standard_normal(256).astype(np.float32)
    g = tnnmodel.encoder_graph(cfg, make_weights(cfg, seed=1) | {"pool_w": w["pool_w"], "pool_b": w["pool_b"]}, 2, 32,
                               int_mask=True, position_ids=True)
    plan = host.plan(g, precision="fp16")
    t = _types(plan)
    assert t["Cast"] == 1 and t["Unsqueeze"] == 1 and t["Sub"] == 1 and t["Mul"] == 1
    assert t["RocmFusedEmbedding"] == 1 and t["Gather"] == 1 and t["Squeeze"] == 1 and t["Tanh"] == 1
    emb = [l for l in plan if l["type"] == "RocmFusedEmbedding"][0]
    assert emb["inputs"][-1] == "position_ids" and len(emb["inputs"]) == 5
    by_out = {o: l for l in plan for o in l["outputs"]}
    assert by_out["attention_bias"]["output_dims"] == [[2, 1, 1, 32]]
    assert by_out["mask_4d"]["output_dims"] == [[2, 1, 1, 32]] and by_out["mask_f"]["output_dims"] == [[2, 32]]
    assert by_out["pool_tok3"]["output_dims"] == [[2, 1, 256]] and by_out["pool_tok"]["output_dims"] == [[2, 256]]
    assert by_out["pooled"]["output_dims"] == [[2, 256]]


def test_config1_attention_layer_graph():
    cfg = EncoderConfig(1, 768, 12, 3072)
    lw = make_weights(cfg, seed=1, with_embeddings=False)["layers"][0]
    g = tnnmodel.attention_layer_graph(lw, 128, 768, 12)
    t = _types(host.plan(g, precision="fp32"))
    assert t["RocmFusedLinear"] == 4 and "RocmFusedAttention" not in t      # InnerProduct x4, decomposed core
    t16 = _types(host.plan(g, precision="fp16"))
    assert t16 == {"RocmFusedAttention": 1, "RocmFusedLinear": 1}


def test_error_behaviour_of_interpreter_and_layer_creation():
    _, _, g = _graph(layers=1)
    proto, model = g.proto(), g.model()
    text = proto.decode() if isinstance(proto, bytes) else proto
    # an unknown layer type is TNNERR_PARAM_ERR from layer creation (default_network.cc:246-250)
    bad = text.replace("\"GELU ", "\"Gelu2 ", 1)
    assert bad != text
    with pytest.raises(host.HostError):
        host.plan(bad, model, "fp32")
    # a layer that reads a blob nobody produced
    bad = text.replace("GELU l0_gelu 1 1 l0_ffn1_o", "GELU l0_gelu 1 1 l0_missing", 1)
    assert bad != text
    with pytest.raises(host.HostError):
        host.plan(bad, model, "fp32")
    # truncated model file
    with pytest.raises(host.HostError):
        host.plan(text, model[: len(model) // 2], "fp32")
    # garbage proto
    with pytest.raises(host.HostError):
        host.plan("this is not a proto", model, "fp32")


def _raw_buffer_records(model):
    """offsets of the weight records of a model file: magic 0x0FABC0004, element type, byte length, rank, dims (objseri.h:57-77)"""
    import struct
    magic, out, at = struct.pack("<I", 0x0FABC0004), [], 0
    while True:
        at = model.find(magic, at)
        if at < 0 or at + 16 > len(model):
            return out
        dt, length, rank = struct.unpack("<3i", model[at + 4:at + 16])
        if 0 <= dt <= 6 and 0 < length <= len(model) and 0 <= rank <= 8:
            dims = struct.unpack("<%di" % rank, model[at + 16:at + 16 + 4 * rank])
            out.append((at, dt, length, dims))
        at += 4


def test_malformed_model_files_are_refused_with_a_status():
    """Files that promise more than they hold end in a Status, never in a read beyond a buffer: a count in a layer line
    larger than the line, a layer of the path without blobs, a weight record whose dims or element type do not fit its
    bytes, an input line with an absurd rank.  (The parser and the passes were also run over some thousand randomly
    damaged files under the address sanitizer; these are the kinds of damage that found something.)"""
    import re
    import struct
    _, _, g = _graph(layers=1)
    proto, model = g.proto(), g.model()
    text = proto.decode() if isinstance(proto, bytes) else proto
    host.plan(text, model, "fp16")  # the undamaged pair plans

    def refused(t, m, why):
        with pytest.raises(host.HostError):
            host.plan(t, m, "fp16")
        with pytest.raises(host.HostError):
            host.plan(t, m, "fp32")

    # counts in front of a list larger than the list: Reshape dims, Permute orders, the rank of an input
    refused(text.replace("l0_q_4d 0 4 4 2 32 4 64 0", "l0_q_4d 0 4 2147483647 2 32 4 64 0", 1), model, "reshape count")
    refused(text.replace("l0_qh 4 0 2 1 3", "l0_qh 2147483647 0 2 1 3", 1), model, "permute count")
    refused(text.replace("input_ids 2 2 32 3", "input_ids 2147483647 2 32 3", 1), model, "input rank")
    refused(text.replace("input_ids 2 2 32 3", "input_ids 2 2 32 77", 1), model, "input data type")
    # layers of the path without an input or an output blob
    refused(text.replace("Reshape l0_q_rs 1 1 l0_q_o l0_q_4d", "Reshape l0_q_rs 0 1 l0_q_4d", 1), model, "no input")
    refused(text.replace("Permute l0_q_pm 1 1 l0_q_4d l0_qh", "Permute l0_q_pm 1 0 l0_q_4d", 1), model, "no output")
    refused(text.replace("MatMul l0_q_mm 1 1 x0 l0_q_mm_o", "MatMul l0_q_mm 0 1 l0_q_mm_o", 1), model, "no input")
    # weight records: dims that promise more (or fewer) elements than the record holds, an element type outside the format
    records = [r for r in _raw_buffer_records(model) if len(r[3]) == 2 and r[1] == 0]
    assert len(records) >= 6, len(records)
    for at, dt, length, dims in records[:8]:
        bigger = bytearray(model)
        bigger[at + 16:at + 20] = struct.pack("<i", dims[0] * 2)
        refused(text, bytes(bigger), "dims larger than the data")
        smaller = bytearray(model)
        smaller[at + 20:at + 24] = struct.pack("<i", max(dims[1] // 2, 1))
        refused(text, bytes(smaller), "dims smaller than the data")
    at = records[0][0]
    alien = bytearray(model)
    alien[at + 4:at + 8] = struct.pack("<i", 77)
    refused(text, bytes(alien), "element type")
    negative = bytearray(model)
    negative[at + 16:at + 20] = struct.pack("<i", -records[0][3][0])
    refused(text, bytes(negative), "negative dim")


@pytest.mark.parametrize("precision", ["fp32", "fp16"])
def test_int8_encoder_reformat_layers_are_folded(precision, monkeypatch):
    """The quantised encoder of the X86 fixture: with the int8 pass off the explicit Reformat / QuantizedInnerProduct
    chain stays; with it on every Reformat is folded into its neighbour (the counts the device tests also see)."""
    import golden_util
    cfg, w, B, S, scales, f = golden_util.int8_encoder()
    g = quant.int8_encoder_graph(cfg, w, scales, B, S)
    monkeypatch.setenv("TNN_ROCM_FUSE_INT8", "0")
    t0 = _types(host.plan(g, precision=precision))
    assert t0["Reformat"] == 10 and t0["QuantizedInnerProduct"] == 6
    monkeypatch.setenv("TNN_ROCM_FUSE_INT8", "1")
    plan = host.plan(g, precision=precision)
    t1 = _types(plan)
    assert t1["RocmQuantLinearGelu"] == 1 and t1["QuantizedInnerProduct"] == 0
    if precision == "fp16":
        assert t1["Reformat"] == 1 and t1["RocmFusedAttention"] == 1 and t1["RocmFusedLinearInt8"] == 2
        att = [l for l in plan if l["type"] == "RocmFusedAttention"][0]
        assert len(att["outputs"]) == 2          # the context and its int8 quantisation
    else:
        assert t1["Reformat"] == 2 and t1["RocmFusedLinearInt8"] == 5
    for fold in ("TNN_ROCM_FOLD_GELU_LUT", "TNN_ROCM_FOLD_ATTN_Q8"):
        monkeypatch.setenv(fold, "0")
    t2 = _types(host.plan(g, precision=precision))
    assert t2["RocmQuantLinearGelu"] == 0 and t2["RocmGeluInt8"] == 1


def test_quantized_add_graph_gets_reformat_layers_and_int8_blobs():
    g = tnnmodel.int8_add_graph([1, 256, 256, 1], np.float32(0.031), np.float32(0.017), np.float32(0.027))
    plan = host.plan(g, precision="fp32")
    t = _types(plan)
    assert t["QuantizedAdd"] == 1 and t["Reformat"] == 3 and t["Mul"] == 3, t
    add = [l for l in plan if l["type"] == "QuantizedAdd"][0]
    assert add["inputs"] == ["a_int8_reformat", "b_int8_reformat"]
    assert add["output_dims"] == [[1, 256, 256, 1]]


# ---- the attention rewrite: spellings it must accept, graphs it must leave alone ----------------------------------
def _attention_block(B=2, S=32, H=256, heads=4, **spelling):
    cfg = EncoderConfig(1, H, heads, 2 * H)
    lw = make_weights(cfg, seed=3, bias_std=0.02)["layers"][0]
    return tnnmodel.attention_block_graph(lw, B, S, H, heads, **spelling)


ACCEPTED_SPELLINGS = {
    "mul_scale": dict(),
    "div_scale": dict(scale="div"),
    "scale_on_q": dict(scale="q"),
    "scale_on_q_and_k": dict(scale="qk"),
    "no_scale": dict(scale="none"),
    "mask_operand_first": dict(mask_first=True),
    "mask_first_div": dict(mask_first=True, scale="div"),
    "no_mask": dict(mask=None),
    "one_mask_row_for_all": dict(mask="111s"),
    "inner_product_projections": dict(proj="inner_product"),
    "rank3_single_sequence": dict(B=1, rank3=True, mask="11s"),
    "rank3_inner_product_no_mask": dict(B=1, rank3=True, mask=None, proj="inner_product"),
    "negative_softmax_axis": dict(softmax_axis=-1),
}
REFUSED_SPELLINGS = {
    # (no mask in these two: in fp16 blobs -10000 + score keeps nothing of the score, and a softmax across the queries
    #  or heads of a masked key would then compare the fp16 rounding of the device with the fp32 of the checker)
    "softmax_over_queries": dict(softmax_axis=2, mask=None),
    "softmax_over_heads": dict(softmax_axis=1, mask=None),
    "mask_per_query_and_key": dict(mask="b1ss"),
    "rank3_mask_per_query": dict(B=1, rank3=True, mask="1ss"),
    "scores_read_twice": dict(tap_scores=True),
    "head_dim_32": dict(heads=8),
}


@pytest.mark.parametrize("name", sorted(ACCEPTED_SPELLINGS))
def test_attention_spelling_is_fused(name):
    plan = host.plan(_attention_block(**ACCEPTED_SPELLINGS[name]), precision="fp16")
    t = _types(plan)
    assert t == {"RocmFusedAttention": 1, "RocmFusedLinear": 1}, (name, t)
    att = [l for l in plan if l["type"] == "RocmFusedAttention"][0]
    assert att["inputs"] == (["hidden"] if ACCEPTED_SPELLINGS[name].get("mask", "b11s") is None
                             else ["hidden", "attention_bias"])
    # the fused layer's output is the head-merging Reshape's output, with that layer's dims
    sp = ACCEPTED_SPELLINGS[name]
    B = sp.get("B", 2)
    flat = sp.get("rank3") or sp.get("proj") == "inner_product"
    assert att["output_dims"] == [[B * 32, 256] if flat else [B, 32, 256]], att["output_dims"]


@pytest.mark.parametrize("name", sorted(REFUSED_SPELLINGS))
def test_attention_lookalike_stays_decomposed(name):
    """Graphs that look like the attention core but are not what the fused kernel computes: a softmax over another
    axis, a mask with one value per (query, key), scores somebody else reads, a head size the kernel has no form
    for.  The plan must succeed (Instance::Init would) and keep Softmax and both batched MatMuls as single ops."""
    plan = host.plan(_attention_block(**REFUSED_SPELLINGS[name]), precision="fp16")
    t = _types(plan)
    assert "RocmFusedAttention" not in t and t["Softmax"] == 1 and t["MatMul"] == 2 and t["Permute"] == 4, (name, t)
    assert t["RocmFusedLinear"] == 4


def _input_read_by_both_kinds(T=64, K=128, N=128, seed=5):
    """x feeds a quantised InnerProduct and, as a residual, a float Add: the model-input case of the engine's Reformat
    insertion (net_optimizer_insert_int8_reformat.cc:84-131)"""
    rng = np.random.default_rng(seed)
    g = tnnmodel.Graph()
    one = np.array([1.0], np.float32)
    g.add_input("x", [T, K])
    g.add_layer("QuantizedInnerProduct", "fc", ["x"], ["yq"], [N, 1, 0, 1])
    w = rng.integers(-127, 128, size=(N, K)).astype(np.int8)
    g.res_inner_product("fc", w, rng.integers(-500, 500, size=N).astype(np.int32),
                        quant_scale=rng.uniform(1e-3, 2e-3, size=N).astype(np.float32))
    g.res_blob_scale("x", np.float32(0.03))
    g.res_blob_scale("yq", np.float32(0.05))
    g.add_layer("Mul", "out_copy", ["yq"], ["y"], [1])
    g.res_eltwise("out_copy", "Mul", one)
    g.add_layer("Add", "res", ["y", "x"], ["z"], [1])
    g.add_output("z")
    return g


def test_model_input_read_by_quantised_and_float_layers_gets_a_reformat_at_the_head():
    plan = host.plan(_input_read_by_both_kinds(), precision="fp32")
    assert plan[0]["type"] == "Reformat" and plan[0]["inputs"] == ["x"]
    assert plan[0]["name"] == "x_int8_reformat__from_model_input__"
    by_name = {l["name"]: l for l in plan}
    fc = [l for l in plan if "fc" in l["name"]][0]
    assert fc["inputs"][0] == "x_int8_reformat"            # the quantised reader takes the int8 copy ...
    assert "x" in by_name["res"]["inputs"]                 # ... the float reader the model input itself


@pytest.mark.parametrize("blob", ["q_o", "qh", "kt", "scores", "scaled", "masked", "probs", "ctx_h", "ctx_s", "ctx"])
def test_intermediate_blob_named_as_model_output_survives_the_rewrites(blob):
    """TNN::AddOutput / an output line in the model file can name any blob of the attention block.  Whatever the
    rewrites fold, a blob the caller asked for must still be written by some layer of the plan, with the dims the
    un-rewritten graph gives it."""
    g = _attention_block()
    names = {b for l in host.plan(g, precision="fp32") for b in l["outputs"]}
    if blob not in names:
        pytest.skip("the block's writer does not name a blob %r" % blob)
    want = {b: d for l in host.plan(g, precision="fp32") for b, d in zip(l["outputs"], l["output_dims"])}[blob]
    g.add_output(blob)
    plan = host.plan(g, precision="fp16")
    got = {b: d for l in plan for b, d in zip(l["outputs"], l["output_dims"])}
    assert blob in got, (blob, _types(plan))
    assert got[blob] == want


def test_every_encoder_blob_named_as_model_output_survives_the_rewrites():
    """The same for the whole encoder graph, one blob at a time: embeddings, every LayerNorm output that the rewrites
    would otherwise leave un-materialised, the FFN's GELU input and output, the residual sums."""
    base = _graph(layers=2)[2]
    first = host.plan(base, precision="fp32")
    dims = {b: d for l in first for b, d in zip(l["outputs"], l["output_dims"])}
    kept_anyway = {b for l in host.plan(base, precision="fp16") for b in l["outputs"]}
    asked = 0
    for blob in sorted(dims):
        if blob in kept_anyway:
            continue
        g = _graph(layers=2, extra_outputs=(blob,))[2]
        got = {b: d for l in host.plan(g, precision="fp16") for b, d in zip(l["outputs"], l["output_dims"])}
        assert blob in got and got[blob] == dims[blob], blob
        asked += 1
    assert asked > 20


def test_weight_only_int8_model_plans_like_its_float_form():
    """A model whose MatMul weights and embedding tables were stored as int8 + scale (the engine's dynamic range
    quantisation: DynamicRangeQuantizedMatMul / Gather layers, net_optimizer_dynamic_range_dequant.cc) is dequantised
    before the device's passes see it, so it is rewritten into the same fused layers as the float model; a weight record
    whose scale is missing is refused."""
    cfg, w, g = _graph()
    plain = _types(host.plan(g, precision="fp16"))
    _, _, g8 = _graph()
    deq = g8.weight_only_int8()
    assert len(deq) == 2 + 6 * cfg.layers            # two tables, six projections per layer
    text = g8.proto()
    assert text.count("DynamicRangeQuantizedMatMul") == 6 * cfg.layers and text.count("DynamicRangeQuantizedGather") == 2
    assert len(g8.model()) < len(g.model()) // 3
    assert _types(host.plan(g8, precision="fp16")) == plain
    assert _types(host.plan(g8, precision="fp32")) == _types(host.plan(g, precision="fp32"))
    # the scale record of the first MatMul taken out of the file: the int8 weight is left without a float scale
    model = g8.model()
    first = [r for r in _raw_buffer_records(model) if r[1] == 2 and len(r[3]) == 2 and r[3][0] == cfg.hidden][0]
    at = first[0] + 16 + 4 * len(first[3]) + first[2]     # the record behind the int8 weight: its scale
    damaged = bytearray(model)
    damaged[at + 4:at + 8] = (2).to_bytes(4, "little")     # typed int8 instead of float
    with pytest.raises(host.HostError):
        host.plan(text, bytes(damaged), "fp16")


def test_half_precision_weight_file_plans_like_its_float_form():
    """a model file with its weights stored as IEEE half (the converter's option for files of half the size) is widened
    ahead of the rewrites and ends as the same fused layers"""
    cfg, w, g = _graph()
    plain16, plain32 = _types(host.plan(g, precision="fp16")), _types(host.plan(g, precision="fp32"))
    _, _, gh = _graph()
    gh.half_weights()
    assert len(gh.model()) < len(g.model()) * 0.55
    assert _types(host.plan(gh, precision="fp16")) == plain16
    assert _types(host.plan(gh, precision="fp32")) == plain32


def test_first_version_of_the_file_format_plans_like_the_current_one():
    """files of the first format version (proto magic 0x0FABC0002: input lines without rank and type, weight records
    without dims; model_interpreter.cc:262-272, objseri.h:57-77) are read as the current ones are"""
    cfg = EncoderConfig(1, 256, 4, 512)
    lw = make_weights(cfg, seed=5)["layers"][0]
    current = tnnmodel.attention_block_graph(lw, 2, 40, 256, 4, proj="inner_product")
    with tnnmodel.legacy_format():
        old = tnnmodel.attention_block_graph(lw, 2, 40, 256, 4, proj="inner_product")
        proto, model = old.proto(), old.model()
    assert "4206624770" in proto.split("\n")[0] and "hidden 80 256 :" in proto
    assert len(model) < len(current.model())                      # no dims in the records
    for precision in ("fp16", "fp32"):
        a, b = host.plan(proto, model, precision), host.plan(current, precision=precision)
        assert [(l["type"], l["output_dims"]) for l in a] == [(l["type"], l["output_dims"]) for l in b]
