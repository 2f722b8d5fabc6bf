// What DEVICE_ROCM adds to the engine's own vocabulary: the device / network type constants, the layer types the
// ROCm optimizer passes produce, and their params and resources.
//
// Included after the engine's headers (include/tnn/core/common.h, source/tnn/core/layer_type.h,
// source/tnn/interpreter/layer_param.h, layer_resource.h) inside the engine tree, and after this repository's own
// restatement of them otherwise, so the backend sources read the same in both builds.  The engine's enums are closed
// (include/tnn/core/common.h:88-116, source/tnn/core/layer_type.h:25-260), so the new values are typed constants that
// no enumerator of the engine uses and that lie inside each enum's range of values (a cast to a value outside it is
// undefined, and clang rejects it in a constant expression): LayerType ends at 1001, so its range is [0, 1023];
// NetworkType spans -1 ... 0x8000 (range up to 0xFFFF), DeviceType 0 ... 0x1070 (range up to 0x1FFF).  A maintainer who prefers enumerators moves them into the
// enums and deletes the constants here, nothing else changes.
#ifndef TNN_AMD_HOST_ROCM_ENGINE_ADDITIONS_H_
#define TNN_AMD_HOST_ROCM_ENGINE_ADDITIONS_H_

namespace TNN_NS {

// include/tnn/core/common.h:103-115 (DeviceType), :90-100 (NetworkType)
constexpr DeviceType DEVICE_ROCM        = static_cast<DeviceType>(0x1080);
constexpr NetworkType NETWORK_TYPE_ROCM = static_cast<NetworkType>(0x9000);

// produced only by the ROCm optimizer passes (no proto spelling, so no layer interpreter)
constexpr LayerType LAYER_ROCM_FUSED_LINEAR      = static_cast<LayerType>(901);
constexpr LayerType LAYER_ROCM_FUSED_ATTENTION   = static_cast<LayerType>(902);
constexpr LayerType LAYER_ROCM_FUSED_LINEAR_INT8 = static_cast<LayerType>(903);
constexpr LayerType LAYER_ROCM_GELU_INT8         = static_cast<LayerType>(904);
constexpr LayerType LAYER_ROCM_FUSED_EMBEDDING   = static_cast<LayerType>(905);
constexpr LayerType LAYER_ROCM_QUANT_LINEAR_GELU = static_cast<LayerType>(906);
// LayerNorm (LayerNormLayerParam, inputs x, scale, bias) with a second, int8 output: the quantised copy of the first
constexpr LayerType LAYER_ROCM_LAYER_NORM_QUANT  = static_cast<LayerType>(907);

struct RocmFusedLinearResource : public LayerResource {
    RawBuffer weight_nk;  // [N, K] fp32
    RawBuffer bias;       // [N] fp32 (may be empty)
    // scale / shift ([K] fp32) of a LayerNorm folded into this layer (the one whose output was the A operand)
    RawBuffer ln_gamma, ln_beta;
    // scale / shift ([N] fp32) of the LayerNorm whose output is this layer's residual operand (residual_ln)
    RawBuffer residual_gamma, residual_beta;
};

struct RocmFusedLinearParam : public LayerParam {
    int num_output   = 0;
    int has_bias     = 0;
    int gelu         = 0;  // erf GELU applied to (x W^T + b)
    int has_residual = 0;  // second input added after the activation
    int axis         = -1; // -1: contract the last dimension; >= 0: InnerProduct form, contract dims[axis:]
    // LayerNorm folded into this projection (RocmFusionPass::FoldLayerNorm): input 0 is the tensor the LayerNorm
    // read, the layer computes act(LayerNorm(x) W^T + b); with ln_y a second output blob receives LayerNorm(x)
    // itself for the other readers of that tensor.
    int ln_fold = 0, ln_y = 0;
    float ln_eps = 0.f;
    // ln_stats: instead of LayerNorm(x) the layer leaves every row's {rstd, mean} in the context's side buffer named
    // ln_stats_key, for the one other reader of that tensor, which is a RocmFusedLinear with residual_ln: its second
    // input is then the tensor the LayerNorm read, and it adds LayerNorm(that tensor), rebuilt from the statistics
    // under residual_ln_key and its resource's residual_gamma / residual_beta (RocmFusionPass::HandOverRowStatistics).
    int ln_stats = 0, residual_ln = 0;
    std::string ln_stats_key, residual_ln_key;
    // Row sums: a residual_ln layer whose output feeds a folding layer also leaves every row's sum and sum of squares
    // per tile column in the side buffer row_sums_key; the folding layer (ln_sums_key, the same name) adds those up
    // instead of taking the LayerNorm statistics from its A tiles (RocmFusionPass::HandOverRowSums).
    std::string row_sums_key, ln_sums_key;
};
struct RocmFusedAttentionParam : public LayerParam {
    int heads    = 0;
    int head_dim = 0;
    float scale  = 1.0f;
    int has_mask = 0;  // second input: additive mask broadcastable to [B,1,1,S]
    int seq_len  = 0;  // S of the matched head split ([B,S,h,d]); 0 = take it from the input blob's shape
    // The fused layer's output is the output of the head-merging Reshape it replaced and must have that layer's dims:
    // split_rank is the rank of the head split (4: [B,S,h,d], 3: [S,h,d]), merge_shape the Reshape's shape parameter
    // (0 copies the dim of the split tensor, -1 is inferred; source/tnn/layer/reshape_layer.cc:41-63).  Empty = the
    // dims of input 0.
    int split_rank = 0;
    std::vector<int> merge_shape;
    // quantised form: the first input is the int8 blob the three QuantizedInnerProduct projections read, the
    // resource is a RocmFusedQkvInt8Resource and qkv_out_scale are the scales of their three int8 output blobs
    int quant = 0;
    float qkv_out_scale[3] = {0.f, 0.f, 0.f};
    // LayerNorm folded into the QKV projection, as in RocmFusedLinearParam
    int ln_fold = 0, ln_y = 0, ln_stats = 0;
    float ln_eps = 0.f;
    std::string ln_stats_key, ln_sums_key;
    // the last output blob is int8: the context quantised as the Reformat layer that followed would (ROCm int8 pass)
    int out_quant = 0;
};
// Gather(word ids) + Add(position constant) + Gather(type ids) + Add + LayerNorm of a BERT-style front end.
// Inputs: word ids, type ids (int32), gamma, beta (constant blobs); resource: RocmFusedEmbeddingResource.
struct RocmFusedEmbeddingParam : public LayerParam {
    float eps = 1e-5f;
};
struct RocmFusedEmbeddingResource : public LayerResource {
    RawBuffer word;  // [vocab, H]
    RawBuffer type;  // [types, H]
    RawBuffer pos;   // [S, H]: the constant added to the word rows, one row per position
};
// QuantizedInnerProduct whose int8 result is consumed as float: y = q * out_scale (+ residual), q never stored.
// Input 0 is the int8 blob, input 1 (has_residual) a float blob of the output's shape; the output is float.
struct RocmFusedLinearInt8Param : public InnerProductLayerParam {
    float out_scale  = 0.f;  // scale of the int8 blob the original layer produced
    int has_residual = 0;
};
// QuantizedInnerProduct whose int8 result went through Reformat -> GELU -> Reformat: the projection applies that
// int8 -> int8 map as a 256-entry table in its epilogue.  mid_scale is the scale of the int8 blob the projection used
// to write; the output blob is the one the second Reformat wrote.
struct RocmQuantLinearGeluParam : public InnerProductLayerParam {
    float mid_scale = 0.f;
};
// Which blobs of a layer are int8 blobs (BlobInt8 with a scale resource) in a quantised net on this device: the engine's
// rule (default_network.cc:362-440: all blobs of a layer whose param is quantized; a Reformat's by its src / dst type)
// plus the layers of the ROCm int8 pass that read one kind of blob and write the other.
inline bool RocmBlobIsInt8(LayerType type, LayerParam *param, bool is_input, size_t index, size_t n_outputs) {
    if (type == LAYER_REFORMAT) {
        auto rp = dynamic_cast<ReformatLayerParam *>(param);
        return rp && (is_input ? rp->src_type == DATA_TYPE_INT8 : rp->dst_type == DATA_TYPE_INT8);
    }
    if (type == LAYER_ROCM_FUSED_LINEAR_INT8)  // int8 in, dequantised (+ residual) out
        return is_input && index == 0;
    if (type == LAYER_ROCM_FUSED_ATTENTION) {  // int8 in when the projections are quantised; last output the int8 context
        auto ap = dynamic_cast<RocmFusedAttentionParam *>(param);
        return ap && (is_input ? (index == 0 && ap->quant) : (ap->out_quant && index + 1 == n_outputs));
    }
    if (type == LAYER_ROCM_LAYER_NORM_QUANT)  // float in, float out, and the quantised copy of the output
        return !is_input && index == 1;
    return param && param->quantized;
}

struct RocmFusedQkvInt8Resource : public LayerResource {
    RawBuffer weight;   // int8 [3H, K]
    RawBuffer bias;     // int32 [3H] (may be empty)
    RawBuffer w_scale;  // fp32 [3H] per-output-channel weight scales
};

}  // namespace TNN_NS
#endif
