"""Writer for the engine's on-disk model formats: the .tnnproto text graph and the .tnnmodel weight blob.

Format facts (reference tree):
  proto  : source/tnn/interpreter/tnn/model_interpreter.cc:174-398, model_packer.cc:70-184
           line0 "1 <nblobs> 1 <magic> ," ; line1 inputs (v2: "name rank d0.. dtype" joined by ':') ;
           line2 blob names ; line3 outputs ; line4 layer count ; then one line per layer
           "Type name n_in n_out inputs.. outputs.. params.. ,"
  model  : model_packer.cc:186-248 / model_interpreter.cc:400-476
           u32 magic ; i32 resource count ; per resource {i32 type, str type_str, str name, payload} ;
           then {u32 magic, i32 n, (str key, raw buffer)*n} for the constant map.
  raw    : objseri.h:57-77   {u32 0x0FABC0004, i32 dtype, i32 nbytes, [i32 ndims, dims.., bytes]}
  strings: i32 byte length + bytes.

`Graph` collects layers, resources and constants; `encoder_graph()` emits the decomposed BERT encoder the
way an ONNX export looks after conversion (MatMul+Add projections, Reshape/Permute head split, MatMul,
Mul, Add(mask), Softmax, MatMul, LayerNorm, GELU), and `int8_ffn_graph()` the QuantizedInnerProduct variant.
"""
import struct

import numpy as np

MAGIC_V2 = 0x0FABC0004
MAGIC_V1 = 0x0FABC0002
_version = 2  # file version written: 2, or 1 inside `with legacy_format():`
DT_FLOAT, DT_HALF, DT_INT8, DT_INT32 = 0, 1, 2, 3
_NP2DT = {np.dtype(np.float32): DT_FLOAT, np.dtype(np.float16): DT_HALF, np.dtype(np.int8): DT_INT8,
          np.dtype(np.int32): DT_INT32}

# LayerType numbers (source/tnn/core/layer_type.h) for the resource headers; the reader re-derives the type
# from the type string, the number only has to be in range.
_LAYER_TYPE_NUM = {"InnerProduct": 19, "QuantizedInnerProduct": 19, "Add": 38, "Mul": 42, "Sub": 39, "Div": 43,
                   "Gather": 104, "MatMul": 105, "BlobScale": 600, "DynamicRangeQuantizedMatMul": 105,
                   "DynamicRangeQuantizedGather": 104, "DynamicRangeQuantizedInnerProduct": 19}
BLOB_SCALE_SUFFIX = "_scale_data_"


def _i32(v):
    return struct.pack("<i", int(v))


def _u32(v):
    return struct.pack("<I", int(v))


def _str(s):
    b = s.encode("utf-8")
    return _i32(len(b)) + b


class legacy_format:
    """`with legacy_format():` -- graphs built AND serialised inside write the first version of the file format (proto
    magic 0x0FABC0002: input lines are a name and its dims, every input is float; weight records carry no dims:
    model_interpreter.cc:262-272, objseri.h:57-77), which old model files still have."""
    def __enter__(self):
        global _version
        self._saved, _version = _version, 1

    def __exit__(self, *exc):
        global _version
        _version = self._saved


def raw_buffer(arr, dims=None):
    """Serialise one RawBuffer record.  `arr` None or empty gives the zero-length form."""
    magic = MAGIC_V2 if _version == 2 else MAGIC_V1
    if arr is None or arr.size == 0:
        return _u32(magic) + _i32(DT_FLOAT) + _i32(0)
    a = np.ascontiguousarray(arr)
    dt = _NP2DT[a.dtype]
    out = _u32(magic) + _i32(dt) + _i32(a.nbytes)
    if _version == 2:
        dims = list(a.shape if dims is None else dims)
        out += _i32(len(dims)) + b"".join(_i32(d) for d in dims)
    return out + a.tobytes()


class Graph:
    def __init__(self):
        self.inputs = []      # (name, dims, dtype)
        self.outputs = []
        self.layers = []      # (type, name, inputs, outputs, params)
        self.resources = []   # (name, type_str, payload bytes) in layer order
        self.constants = {}   # blob name -> ndarray
        self.blobs = []
        self._float_weights = {}  # layer name -> ("MatMul" | "Gather" | "InnerProduct", fp32 array[, bias]): what
        #                           weight_only_int8() and half_weights() rewrite
        self._float_operands = {}  # layer name -> (type string, fp32 operand of an Add / Sub / Mul / Div resource)

    def _blob(self, name):
        if name not in self.blobs:
            self.blobs.append(name)

    def add_input(self, name, dims, dtype=DT_FLOAT):
        self.inputs.append((name, list(dims), dtype))
        self._blob(name)

    def add_output(self, name):
        self.outputs.append(name)

    def add_constant(self, name, arr):
        self.constants[name] = np.ascontiguousarray(arr)
        self._blob(name)

    def add_layer(self, type_str, name, inputs, outputs, params=()):
        for b in list(inputs) + list(outputs):
            self._blob(b)
        self.layers.append((type_str, name, list(inputs), list(outputs), [str(p) for p in params]))

    # ---- resources ------------------------------------------------------------------------------
    def _res(self, name, type_str, payload):
        self.resources.append((name, type_str, payload))

    def res_matmul(self, name, weight_kn):
        self._res(name, "MatMul", raw_buffer(weight_kn))
        self._float_weights[name] = ("MatMul", np.ascontiguousarray(weight_kn, np.float32))

    def res_eltwise(self, name, type_str, element):
        self._res(name, type_str, raw_buffer(element))
        if element is not None and np.asarray(element).dtype == np.float32:
            self._float_operands[name] = (type_str, np.ascontiguousarray(element, np.float32))

    def res_gather(self, name, data, indices=None):
        p = (_i32(1) + raw_buffer(data)) if data is not None else _i32(0)
        p += (_i32(1) + raw_buffer(indices)) if indices is not None else _i32(0)
        self._res(name, "Gather", p)
        if data is not None and indices is None and np.asarray(data).dtype == np.float32 and np.asarray(data).ndim == 2:
            self._float_weights[name] = ("Gather", np.ascontiguousarray(data, np.float32))

    def res_inner_product(self, name, weight_nk, bias=None, quant_scale=None):
        """fp32: weight [N,K] + bias [N].  int8: int8 weight, int32 bias, zero points (int8 zeros), fp32 scale."""
        p = _str(name) + raw_buffer(weight_nk) + raw_buffer(bias)
        type_str = "InnerProduct"
        if quant_scale is not None:
            type_str = "QuantizedInnerProduct"
            zp = np.zeros(quant_scale.shape, np.int8)
            p += raw_buffer(zp) + raw_buffer(np.asarray(quant_scale, np.float32))
        elif np.asarray(weight_nk).dtype == np.float32:
            self._float_weights[name] = ("InnerProduct", np.ascontiguousarray(weight_nk, np.float32), bias)
        self._res(name, type_str, p)

    def res_blob_scale(self, blob_name, scale):
        scale = np.atleast_1d(np.asarray(scale, np.float32))
        zp = np.zeros(scale.shape, np.int8)
        bias = np.zeros(scale.shape, np.int32)
        self._res(blob_name + BLOB_SCALE_SUFFIX, "BlobScale", raw_buffer(zp) + raw_buffer(scale) + raw_buffer(bias))

    def weight_only_int8(self):
        """The model as the engine's weight-only quantiser leaves it (tools/dynamic_range_quantization; the file format of
        model_packer.cc:148-153 and mat_mul / gather_layer_interpreter.cc): every MatMul weight resource becomes int8 with
        one fp32 scale (max|w| / 127, symmetric), every fp32 Gather table int8 with one scale per row, and the layers are
        typed DynamicRangeQuantized*.  Returns {layer name: the fp32 weights scale * int8 the engine will compute with}."""
        dequantised = {}
        for name, entry in self._float_weights.items():
            kind, w = entry[0], entry[1]
            if kind == "InnerProduct":   # weight, bias, then the scale alone (inner_product_layer_interpreter.cc:111-114)
                scale = np.float32(np.abs(w).max() / 127.0) if w.size and np.abs(w).max() > 0 else np.float32(1.0)
                q = np.clip(np.rint(w / scale), -127, 127).astype(np.int8)
                payload = _str(name) + raw_buffer(q) + raw_buffer(entry[2]) + raw_buffer(np.array([scale], np.float32))
                dequantised[name] = (scale * q.astype(np.float32)).astype(np.float32)
            elif kind == "MatMul":
                scale = np.float32(np.abs(w).max() / 127.0) if w.size and np.abs(w).max() > 0 else np.float32(1.0)
                q = np.clip(np.rint(w / scale), -127, 127).astype(np.int8)
                payload = raw_buffer(q) + raw_buffer(np.array([scale], np.float32))
                dequantised[name] = (scale * q.astype(np.float32)).astype(np.float32)
            else:
                amax = np.abs(w).max(axis=1)
                scale = np.where(amax > 0, amax / 127.0, 1.0).astype(np.float32)
                q = np.clip(np.rint(w / scale[:, None]), -127, 127).astype(np.int8)
                payload = _i32(1) + raw_buffer(q) + _i32(0) + raw_buffer(scale)
                dequantised[name] = (scale[:, None] * q.astype(np.float32)).astype(np.float32)
            new_type = "DynamicRangeQuantized" + kind
            self.resources = [(n, new_type, payload) if n == name else (n, t, pl) for n, t, pl in self.resources]
            self.layers = [(new_type, n, i, o, pr) if n == name else (t, n, i, o, pr) for t, n, i, o, pr in self.layers]
        self._float_weights = {}
        return dequantised

    def half_weights(self, tables=True, constants=True):
        """The model as the converter's half-precision option stores it: every fp32 weight record (MatMul and InnerProduct
        weights and biases, embedding tables, the operands of Add / Sub / Mul / Div resources, the constants) as IEEE half.
        Layer types are unchanged; the devices widen the records when they load them (ConvertHalfResource,
        source/tnn/interpreter/layer_resource_generator.cc:52-58).  tables / constants False leave the embedding tables
        and the constant map in fp32 (the engine's CPU devices take half records for layer resources only)."""
        def h(a):
            return None if a is None else np.ascontiguousarray(a, np.float32).astype(np.float16)
        new = {}
        for name, entry in self._float_weights.items():
            kind, w = entry[0], entry[1]
            if kind == "MatMul":
                new[name] = raw_buffer(h(w))
            elif kind == "InnerProduct":
                new[name] = _str(name) + raw_buffer(h(w)) + raw_buffer(h(entry[2]))
            elif tables:
                new[name] = _i32(1) + raw_buffer(h(w)) + _i32(0)
        for name, (type_str, element) in self._float_operands.items():
            new[name] = raw_buffer(h(element))
        self.resources = [(n, t, new.get(n, pl)) for n, t, pl in self.resources]
        if constants:
            self.constants = {k: (h(v) if v.dtype == np.float32 else v) for k, v in self.constants.items()}
        self._float_weights, self._float_operands = {}, {}

    # ---- serialisation ------------------------------------------------------------------------------
    def proto(self):
        lines = ['"1 %d 1 %d ,"' % (len(self.blobs), MAGIC_V2 if _version == 2 else MAGIC_V1)]
        ins = []
        for name, dims, dt in self.inputs:
            if _version == 1:
                assert dt == DT_FLOAT, "the first file version has float inputs only"
                ins.append("%s %s" % (name, " ".join(str(d) for d in dims)))
                continue
            ins.append("%s %d %s %d" % (name, len(dims), " ".join(str(d) for d in dims), dt))
        lines.append('"%s ,"' % " : ".join(ins))
        lines.append('" %s ,"' % " ".join(self.blobs))
        lines.append('"%s ,"' % " ".join(self.outputs))
        lines.append('" %d ,"' % len(self.layers))
        for t, n, i, o, p in self.layers:
            lines.append('"%s ,"' % " ".join([t, n, str(len(i)), str(len(o))] + i + o + p))
        return "\n".join(lines) + "\n"

    def model(self):
        magic = MAGIC_V2 if _version == 2 else MAGIC_V1
        out = _u32(magic) + _i32(len(self.resources))
        for name, type_str, payload in self.resources:
            out += _i32(_LAYER_TYPE_NUM.get(type_str, 0)) + _str(type_str) + _str(name) + payload
        if self.constants:
            out += _u32(magic) + _i32(len(self.constants))
            for key in sorted(self.constants):
                out += _str(key) + raw_buffer(self.constants[key])
        return out


# ---------------------------------------------------------------------------------------------------
def _linear(g, name, x, out, w_nk, bias):
    """y = x W^T + b as the ONNX-exported pair MatMul(weight [K,N] in the resource) + Add(bias resource)."""
    g.add_layer("MatMul", name + "_mm", [x], [name + "_mm_o"], [1])
    g.res_matmul(name + "_mm", np.ascontiguousarray(w_nk.T))
    g.add_layer("Add", name + "_add", [name + "_mm_o"], [out], [1])
    g.res_eltwise(name + "_add", "Add", bias)


def encoder_graph(cfg, weights, B, S, with_embeddings=True, extra_outputs=(), dynamic=False, int_mask=False,
                  position_ids=False):
    """The decomposed encoder graph.  Inputs: input_ids, token_type_ids [B,S] int32 (or `hidden` [B,S,H] fp32
    without embeddings) and `attention_bias` [B,1,1,S] fp32 additive mask.  Output: `last_hidden` [B,S,H].
    dynamic: the head split / merge Reshape layers copy batch and sequence length from their input (shape entries
    0, as an export with dynamic axes has them) instead of naming B and S, so the graph can be reshaped.
    int_mask: the third input is `input_mask` [B,S] int32 (1 = token, 0 = padding), as the tokenizer hands it over
    (examples/base/bert_tokenizer.cc:351-355), and the additive mask is built in the graph the way exported BERT
    models do: Cast(float) -> Unsqueeze(1,2) -> Sub(1 - m) -> Mul(-10000).
    position_ids: positions come in as a fourth int32 input `position_ids` [B,S] and are looked up with a third
    Gather (exports that keep the position ids an input) instead of adding the first S rows of the table."""
    g = Graph()
    H, h, d = cfg.hidden, cfg.heads, cfg.head_dim
    split_shape = [0, 4, 4, 0, 0, h, d, 0] if dynamic else [0, 4, 4, B, S, h, d, 0]
    merge_shape = [0, 3, 3, 0, 0, H, 0] if dynamic else [0, 3, 3, B, S, H, 0]
    if with_embeddings:
        g.add_input("input_ids", [B, S], DT_INT32)
        g.add_input("token_type_ids", [B, S], DT_INT32)
    else:
        g.add_input("hidden", [B, S, H], DT_FLOAT)
    if int_mask:
        g.add_input("input_mask", [B, S], DT_INT32)
        g.add_layer("Cast", "mask_cast", ["input_mask"], ["mask_f"], [DT_FLOAT])
        g.add_layer("Unsqueeze", "mask_unsq", ["mask_f"], ["mask_4d"], [2, 1, 2])
        g.add_layer("Sub", "mask_inv", ["mask_4d"], ["mask_pad"], [0])      # constant first: 1 - m
        g.res_eltwise("mask_inv", "Sub", np.array([1.0], np.float32))
        g.add_layer("Mul", "mask_scale", ["mask_pad"], ["attention_bias"], [1])
        g.res_eltwise("mask_scale", "Mul", np.array([-10000.0], np.float32))
    else:
        g.add_input("attention_bias", [B, 1, 1, S], DT_FLOAT)
    if with_embeddings:
        g.add_layer("Gather", "emb_word", ["input_ids"], ["emb_word_o"], [0, 1, 0])
        g.res_gather("emb_word", weights["word_emb"])
        g.add_layer("Gather", "emb_type", ["token_type_ids"], ["emb_type_o"], [0, 1, 0])
        g.res_gather("emb_type", weights["type_emb"])
        if position_ids:
            g.add_input("position_ids", [B, S], DT_INT32)
            g.add_layer("Gather", "emb_posg", ["position_ids"], ["emb_posg_o"], [0, 1, 0])
            g.res_gather("emb_posg", weights["pos_emb"])
            g.add_layer("Add", "emb_pos", ["emb_word_o", "emb_posg_o"], ["emb_pos_o"], [1])
        else:
            g.add_layer("Add", "emb_pos", ["emb_word_o"], ["emb_pos_o"], [1])
            g.res_eltwise("emb_pos", "Add", weights["pos_emb"][:S])
        g.add_layer("Add", "emb_sum", ["emb_pos_o", "emb_type_o"], ["emb_sum_o"], [1])
        g.add_constant("emb_ln_gamma", weights["emb_ln_g"])
        g.add_constant("emb_ln_beta", weights["emb_ln_b"])
        g.add_layer("LayerNorm", "emb_ln", ["emb_sum_o", "emb_ln_gamma", "emb_ln_beta"], ["x0"], [1, repr(cfg.eps)])
        x = "x0"
    else:
        x = "hidden"
    for li, lw in enumerate(weights["layers"]):
        p = "l%d_" % li
        for nm in ("q", "k", "v"):
            _linear(g, p + nm, x, p + nm + "_o", lw["w" + nm], lw["b" + nm])
            g.add_layer("Reshape", p + nm + "_rs", [p + nm + "_o"], [p + nm + "_4d"], split_shape)
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
        g.add_layer("Reshape", p + "ctx_rs", [p + "ctx_4d"], [p + "ctx"], merge_shape)
        _linear(g, p + "o", p + "ctx", p + "attn_o", lw["wo"], lw["bo"])
        g.add_layer("Add", p + "res1", [x, p + "attn_o"], [p + "sum1"], [1])
        g.add_constant(p + "ln1_gamma", lw["ln1_g"])
        g.add_constant(p + "ln1_beta", lw["ln1_b"])
        g.add_layer("LayerNorm", p + "ln1", [p + "sum1", p + "ln1_gamma", p + "ln1_beta"], [p + "x1"],
                    [1, repr(cfg.eps)])
        _linear(g, p + "ffn1", p + "x1", p + "ffn1_o", lw["w1"], lw["b1"])
        g.add_layer("GELU", p + "gelu", [p + "ffn1_o"], [p + "act"], [])
        _linear(g, p + "ffn2", p + "act", p + "ffn2_o", lw["w2"], lw["b2"])
        g.add_layer("Add", p + "res2", [p + "x1", p + "ffn2_o"], [p + "sum2"], [1])
        g.add_constant(p + "ln2_gamma", lw["ln2_g"])
        g.add_constant(p + "ln2_beta", lw["ln2_b"])
        out = "last_hidden" if li == len(weights["layers"]) - 1 else p + "x2"
        g.add_layer("LayerNorm", p + "ln2", [p + "sum2", p + "ln2_gamma", p + "ln2_beta"], [out], [1, repr(cfg.eps)])
        x = out
    g.add_output("last_hidden")
    if "pool_w" in weights:
        # pooler: the first token's hidden state -> dense -> tanh, the way an exported BERT spells it
        # (Gather with a constant index on the sequence axis, Squeeze, MatMul + Add, Tanh)
        g.add_layer("Gather", "pool_first", ["last_hidden"], ["pool_tok3"], [1, 0, 1])
        g.res_gather("pool_first", None, np.array([0], np.int32))
        g.add_layer("Squeeze", "pool_sq", ["pool_tok3"], ["pool_tok"], [1, 1])
        _linear(g, "pool_fc", "pool_tok", "pool_fc_o", weights["pool_w"], weights["pool_b"])
        g.add_layer("Tanh", "pool_act", ["pool_fc_o"], ["pooled"], [])
        g.add_output("pooled")
    for e in extra_outputs:
        g.add_output(e)
    return g


def attention_block_graph(lw, B, S, H, heads, scale="mul", mask="b11s", mask_first=False, proj="matmul", rank3=False,
                          softmax_axis=None, tap_scores=False):
    """One self-attention block (three projections, attention core, output projection) in the spellings exporters
    produce for the same arithmetic -- what a graph rewrite that recognises the core has to cope with:
    scale     "mul" scores * (1/sqrt d) | "div" scores / sqrt d | "q" q * (1/sqrt d) ahead of the score product |
              "qk" q and k^T each scaled by d^-1/4 | "none"
    mask      None | "b11s" [B,1,1,S] | "111s" one row for every sequence | "b1ss" one value per query and key
              [B,1,S,S] (rank3: "11s" [1,1,S] | "1ss" [1,S,S]); the model input is `attention_bias`
    mask_first  Add(mask, scores) instead of Add(scores, mask)
    proj      "matmul" MatMul + Add on `hidden` [B,S,H] | "inner_product" InnerProduct on `hidden` [B*S,H]
    rank3     a single sequence (B == 1) split as [S,heads,d] with three-axis Permutes, scores [heads,S,S]
    softmax_axis  default: the last axis of the scores
    tap_scores    the scaled scores get a second reader (`scores_tap`, a model output)
    Output `y` has the shape of `hidden`."""
    assert H % heads == 0 and (not rank3 or B == 1)
    d = H // heads
    g = Graph()
    flat = proj == "inner_product"
    g.add_input("hidden", [B * S, H] if flat else [B, S, H])
    if mask is not None:
        g.add_input("attention_bias", {"b11s": [B, 1, 1, S], "111s": [1, 1, 1, S], "b1ss": [B, 1, S, S],
                                       "11s": [1, 1, S], "1ss": [1, S, S]}[mask])
    for nm in ("q", "k", "v"):
        if flat:
            g.add_layer("InnerProduct", "fc_" + nm, ["hidden"], [nm + "_o"], [H, 1, 0, 1])
            g.res_inner_product("fc_" + nm, lw["w" + nm], lw["b" + nm])
        else:
            _linear(g, nm, "hidden", nm + "_o", lw["w" + nm], lw["b" + nm])
        split = [0, 3, 3, S, heads, d, 0] if rank3 else [0, 4, 4, B, S, heads, d, 0]
        g.add_layer("Reshape", nm + "_rs", [nm + "_o"], [nm + "_s"], split)
    po, pt = ([3, 1, 0, 2], [3, 1, 2, 0]) if rank3 else ([4, 0, 2, 1, 3], [4, 0, 2, 3, 1])
    g.add_layer("Permute", "q_pm", ["q_s"], ["qh"], po)
    g.add_layer("Permute", "k_pm", ["k_s"], ["kt"], pt)
    g.add_layer("Permute", "v_pm", ["v_s"], ["vh"], po)
    qb, kb = "qh", "kt"
    if scale in ("q", "qk"):
        f = np.array([d ** -0.5 if scale == "q" else d ** -0.25], np.float32)
        g.add_layer("Mul", "q_scale", ["qh"], ["qh_scaled"], [1])
        g.res_eltwise("q_scale", "Mul", f)
        qb = "qh_scaled"
        if scale == "qk":
            g.add_layer("Mul", "k_scale", ["kt"], ["kt_scaled"], [1])
            g.res_eltwise("k_scale", "Mul", f)
            kb = "kt_scaled"
    g.add_layer("MatMul", "qk", [qb, kb], ["scores"], [-1])
    cur = "scores"
    if scale == "mul":
        g.add_layer("Mul", "scale", [cur], ["scaled"], [1])
        g.res_eltwise("scale", "Mul", np.array([1.0 / np.sqrt(d)], np.float32))
        cur = "scaled"
    elif scale == "div":
        g.add_layer("Div", "scale", [cur], ["scaled"], [1])
        g.res_eltwise("scale", "Div", np.array([np.sqrt(d)], np.float32))
        cur = "scaled"
    if tap_scores:
        g.add_layer("Mul", "tap", [cur], ["scores_tap"], [1])
        g.res_eltwise("tap", "Mul", np.array([1.0], np.float32))
    if mask is not None:
        g.add_layer("Add", "mask", ["attention_bias", cur] if mask_first else [cur, "attention_bias"], ["masked"], [1])
        cur = "masked"
    rank = 3 if rank3 else 4
    g.add_layer("Softmax", "sm", [cur], ["probs"], [rank - 1 if softmax_axis is None else softmax_axis])
    g.add_layer("MatMul", "pv", ["probs", "vh"], ["ctx_h"], [-1])
    g.add_layer("Permute", "ctx_pm", ["ctx_h"], ["ctx_s"], po)
    merge = [0, 2, 2, B * S, H, 0] if (flat or rank3) else [0, 3, 3, B, S, H, 0]
    g.add_layer("Reshape", "ctx_rs", ["ctx_s"], ["ctx"], merge)
    if flat:
        g.add_layer("InnerProduct", "fc_o", ["ctx"], ["y"], [H, 1, 0, 1])
        g.res_inner_product("fc_o", lw["wo"], lw["bo"])
    else:
        _linear(g, "o", "ctx", "y", lw["wo"], lw["bo"])
    g.add_output("y")
    if tap_scores:
        g.add_output("scores_tap")
    return g


def attention_layer_graph(lw, S, H, heads):
    """Benchmark config 1: one self-attention layer on a [S,H] fp32 input with InnerProduct projections
    (mask all ones, so no Add(mask); scale applied by a Mul)."""
    g = Graph()
    d = H // heads
    g.add_input("x", [S, H], DT_FLOAT)
    for nm in ("q", "k", "v"):
        g.add_layer("InnerProduct", "fc_" + nm, ["x"], [nm], [H, 1, 0, 1])
        g.res_inner_product("fc_" + nm, lw["w" + nm], lw["b" + nm])
        g.add_layer("Reshape", "rs_" + nm, [nm], [nm + "3"], [0, 3, 3, S, heads, d, 0])
    g.add_layer("Permute", "pm_q", ["q3"], ["qh"], [3, 1, 0, 2])
    g.add_layer("Permute", "pm_k", ["k3"], ["kh"], [3, 1, 2, 0])
    g.add_layer("Permute", "pm_v", ["v3"], ["vh"], [3, 1, 0, 2])
    g.add_layer("MatMul", "mm_qk", ["qh", "kh"], ["s"], [-1])
    g.add_layer("Mul", "scale", ["s"], ["ss"], [1])
    g.res_eltwise("scale", "Mul", np.array([1.0 / np.sqrt(d)], np.float32))
    g.add_layer("Softmax", "sm", ["ss"], ["p"], [2])
    g.add_layer("MatMul", "mm_pv", ["p", "vh"], ["c"], [-1])
    g.add_layer("Permute", "pm_c", ["c"], ["ch"], [3, 1, 0, 2])
    g.add_layer("Reshape", "rs_c", ["ch"], ["c2"], [0, 2, 2, S, H, 0])
    g.add_layer("InnerProduct", "fc_o", ["c2"], ["y"], [H, 1, 0, 1])
    g.res_inner_product("fc_o", lw["wo"], lw["bo"])
    g.add_output("y")
    return g


def int8_ffn_graph(T, K, F, w1_q, b1_q, w1_scale, w2_q, b2_q, w2_scale, s_in, s_h, s_act, s_out):
    """fp32 [T,K] -> quantize -> QuantizedInnerProduct K->F -> dequantize -> GELU -> quantize ->
    QuantizedInnerProduct F->K -> dequantize -> fp32 [T,K].  The float<->int8 Reformat layers are not written:
    the engine's optimizer inserts them wherever a quantized layer meets a float one
    (source/tnn/optimizer/net_optimizer_insert_int8_reformat.cc:66-181); the two Mul-by-one layers keep the
    model input and output in fp32.  Blob scales are BlobScale resources named <blob>_scale_data_."""
    g = Graph()
    one = np.array([1.0], np.float32)
    g.add_input("x", [T, K])
    g.add_layer("Mul", "in_copy", ["x"], ["a"], [1])
    g.res_eltwise("in_copy", "Mul", one)
    g.add_layer("QuantizedInnerProduct", "fc1", ["a"], ["h"], [F, 1, 0, 1])
    g.res_blob_scale("a", s_in)
    g.res_inner_product("fc1", w1_q, b1_q, quant_scale=w1_scale)
    g.res_blob_scale("h", s_h)
    g.add_layer("GELU", "act", ["h"], ["g"])
    g.add_layer("QuantizedInnerProduct", "fc2", ["g"], ["yq"], [K, 1, 0, 1])
    g.res_blob_scale("g", s_act)
    g.res_inner_product("fc2", w2_q, b2_q, quant_scale=w2_scale)
    g.res_blob_scale("yq", s_out)
    g.add_layer("Mul", "out_copy", ["yq"], ["y"], [1])
    g.res_eltwise("out_copy", "Mul", one)
    g.add_output("y")
    return g


def int8_add_graph(dims, s_a, s_b, s_out):
    """Two fp32 inputs `x`, `z` of shape `dims` -> quantize each -> QuantizedAdd -> dequantize -> fp32 `y`.  As in
    int8_ffn_graph the Reformat layers are left to the engine's optimizer and the Mul-by-one layers keep the model
    inputs and the output in fp32; the three int8 blobs carry per-tensor BlobScale resources.  The x86 int8 Add
    (source/tnn/device/x86/acc/x86_add_layer_acc.cc:77-86) walks dims[1] channels x count(dims[2:]) positions of
    the first batch entry only, so `dims` should be [1, C, H, W] for the engine's DEVICE_X86 to cover every value."""
    g = Graph()
    one = np.array([1.0], np.float32)
    g.add_input("x", dims)
    g.add_input("z", dims)
    g.add_layer("Mul", "in_copy_a", ["x"], ["a"], [1])
    g.res_eltwise("in_copy_a", "Mul", one)
    g.add_layer("Mul", "in_copy_b", ["z"], ["b"], [1])
    g.res_eltwise("in_copy_b", "Mul", one)
    g.add_layer("QuantizedAdd", "sum", ["a", "b"], ["c"], [1])
    g.res_blob_scale("a", s_a)
    g.res_blob_scale("b", s_b)
    g.res_blob_scale("c", s_out)
    g.add_layer("Mul", "out_copy", ["c"], ["y"], [1])
    g.res_eltwise("out_copy", "Mul", one)
    g.add_output("y")
    return g
