// Shape and data-type inference for the layer types the ROCm optimizer passes create (rocm_fused.cc), as BaseLayer
// classes registered with the engine's layer registry (source/tnn/layer/base_layer.h:108-170: TypeLayerCreator,
// TypeLayerRegister, the map CreateLayer() consults).  They are produced only by those passes, so no model interpreter
// knows them and none needs to.
#include "rocm_device.h"
#ifdef TNN_ROCM_ENGINE_TREE
#include "tnn/layer/base_layer.h"
#endif

namespace TNN_NS {
namespace {

// Every blob's data type is settled by the network before the layers are created (int8 blobs by their scale resources,
// float blobs by the network precision, integer inputs as the model declares them), and several of these layers read
// one kind of blob and write another.  The default rule "outputs take the type of the first non-constant input"
// (base_layer.cc:119-164) therefore runs for its bookkeeping of the blobs' change flags only: the types are put back.
class RocmFusedLayerBase : public BaseLayer {
public:
    explicit RocmFusedLayerBase(LayerType type) : BaseLayer(type) {}

protected:
    Status InferOutputDataType() override {
        std::vector<DataType> keep;
        for (auto b : output_blobs_)
            keep.push_back(b->GetBlobDesc().data_type);
        Status st = BaseLayer::InferOutputDataType();
        for (size_t i = 0; i < output_blobs_.size(); ++i)
            output_blobs_[i]->GetBlobDesc().data_type = keep[i];
        return st;
    }
    // every output has the dims of input 0 unless a subclass says otherwise
    Status InferOutputShape(bool ignore_error = false) override {
        Status st = BaseLayer::InferOutputShape(ignore_error);
        if (st != TNN_OK)
            return st;
        if (input_blobs_.empty())
            return Status(TNNERR_PARAM_ERR, "fused layer without an input blob");
        for (auto b : output_blobs_)
            b->GetBlobDesc().dims = input_blobs_[0]->GetBlobDesc().dims;
        return TNN_OK;
    }
    // x[.., K] -> [.., N] contracting the last dimension, or dims[axis:] in the InnerProduct form
    // (layer/inner_product_layer.cc:27-46)
    Status LinearDims(int axis, int num_output) {
        DimsVector out = input_blobs_[0]->GetBlobDesc().dims;
        if (out.empty())
            return Status(TNNERR_PARAM_ERR, "fused linear on a rank-0 blob");
        if (axis >= 0) {
            if (axis > (int)out.size())
                return Status(TNNERR_PARAM_ERR, "fused linear axis out of range");
            out.resize(axis);
            out.push_back(num_output);
        } else {
            out.back() = num_output;
        }
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

// RocmFusedLinear: act(x W^T + b) (+ residual); with ln_y a second output holds LayerNorm(x), dims of x
class RocmFusedLinearLayer : public RocmFusedLayerBase {
public:
    explicit RocmFusedLinearLayer(LayerType type) : RocmFusedLayerBase(type) {}

protected:
    // a float layer throughout: the engine's own rule applies (the outputs take the input's float type)
    Status InferOutputDataType() override { return BaseLayer::InferOutputDataType(); }
    Status InferOutputShape(bool ignore_error = false) override {
        Status st = RocmFusedLayerBase::InferOutputShape(ignore_error);
        if (st != TNN_OK)
            return st;
        auto p = dynamic_cast<RocmFusedLinearParam *>(param_);
        if (!p)
            return Status(TNNERR_NULL_PARAM, "fused linear: param is nil");
        st = LinearDims(p->axis, p->num_output);
        if (st != TNN_OK)
            return st;
        if (p->ln_y && output_blobs_.size() != 2)
            return Status(TNNERR_PARAM_ERR, "fused linear: the LayerNorm output needs a second output blob");
        return TNN_OK;
    }
};

// RocmFusedAttention: context [B,S,H] (+ LayerNorm output, + quantised context), all with the dims of input 0;
// input and outputs may be of different kinds (int8 in, float out; float out plus an int8 copy)
class RocmFusedAttentionLayer : public RocmFusedLayerBase {
public:
    explicit RocmFusedAttentionLayer(LayerType type) : RocmFusedLayerBase(type) {}

protected:
    // The context (output 0, and its quantised copy when there is one) gets the dims the head-merging Reshape of the
    // replaced chain would have given it; a LayerNorm output keeps the dims of input 0.
    Status InferOutputShape(bool ignore_error = false) override {
        Status st = RocmFusedLayerBase::InferOutputShape(ignore_error);
        if (st != TNN_OK)
            return st;
        auto p = dynamic_cast<RocmFusedAttentionParam *>(param_);
        if (!p)
            return Status(TNNERR_NULL_PARAM, "fused attention: param is nil");
        if (p->merge_shape.empty() || p->heads <= 0 || p->head_dim <= 0)
            return TNN_OK;
        const DimsVector in = input_blobs_[0]->GetBlobDesc().dims;
        const int hidden    = p->heads * p->head_dim;
        if (in.empty() || in.back() <= 0)
            return TNN_OK;
        const int tokens = DimsVectorUtils::Count(in) / in.back();
        const int seq    = p->seq_len > 0 ? p->seq_len : (in.size() >= 3 ? in[in.size() - 2] : tokens);
        if (seq <= 0 || tokens % seq != 0)
            return Status(TNNERR_PARAM_ERR, "fused attention: token count is not a multiple of the sequence length");
        DimsVector split = p->split_rank == 3 ? DimsVector({seq, p->heads, p->head_dim})
                                              : DimsVector({tokens / seq, seq, p->heads, p->head_dim});
        if (p->split_rank == 3 && tokens != seq)
            return Status(TNNERR_PARAM_ERR, "fused attention: a three-axis head split holds one sequence");
        DimsVector out;
        int infer = -1, known = 1;
        for (size_t i = 0; i < p->merge_shape.size(); ++i) {
            int v = p->merge_shape[i];
            if (v == 0) {
                if (i >= split.size())
                    return Status(TNNERR_PARAM_ERR, "fused attention: head-merge shape copies a dim that does not exist");
                v = split[i];
            }
            if (v == -1) {
                if (infer >= 0)
                    return Status(TNNERR_PARAM_ERR, "fused attention: head-merge shape infers two dims");
                infer = (int)i;
                v     = 1;
            }
            known *= v;
            out.push_back(v);
        }
        if (infer >= 0 && known > 0)
            out[infer] = tokens * hidden / known;
        if (DimsVectorUtils::Count(out) != tokens * hidden)
            return Status(TNNERR_PARAM_ERR, "fused attention: head-merge shape does not hold the context");
        output_blobs_[0]->GetBlobDesc().dims = out;
        if (p->out_quant && output_blobs_.size() >= 2)
            output_blobs_.back()->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

// RocmFusedEmbedding: ids [..] int32 -> [.., H] in the network's float type
class RocmFusedEmbeddingLayer : public RocmFusedLayerBase {
public:
    explicit RocmFusedEmbeddingLayer(LayerType type) : RocmFusedLayerBase(type) {}

protected:
    Status InferOutputShape(bool ignore_error = false) override {
        Status st = BaseLayer::InferOutputShape(ignore_error);
        if (st != TNN_OK)
            return st;
        auto r = dynamic_cast<RocmFusedEmbeddingResource *>(resource_);
        if (!r)
            return Status(TNNERR_NULL_PARAM, "fused embedding: resource is nil");
        DimsVector out = input_blobs_[0]->GetBlobDesc().dims;
        out.push_back(r->word.GetBufferDims().back());
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

// RocmFusedLinearInt8 (int8 in, float out) and RocmQuantLinearGelu (int8 in, int8 out): InnerProduct shapes
class RocmInt8LinearLayer : public RocmFusedLayerBase {
public:
    explicit RocmInt8LinearLayer(LayerType type) : RocmFusedLayerBase(type) {}

protected:
    Status InferOutputShape(bool ignore_error = false) override {
        Status st = BaseLayer::InferOutputShape(ignore_error);
        if (st != TNN_OK)
            return st;
        auto p = dynamic_cast<InnerProductLayerParam *>(param_);
        if (!p)
            return Status(TNNERR_NULL_PARAM, "quantised linear: param is nil");
        if (p->axis < 0 || p->axis > (int)input_blobs_[0]->GetBlobDesc().dims.size())
            return Status(TNNERR_PARAM_ERR, "InnerProduct axis out of range");
        return LinearDims(p->axis, p->num_output);
    }
};

// RocmLayerNormQuant: LayerNorm(x) and its quantised copy, both with the dims of x (float and int8)
class RocmLayerNormQuantLayer : public RocmFusedLayerBase {
public:
    explicit RocmLayerNormQuantLayer(LayerType type) : RocmFusedLayerBase(type) {}

protected:
    Status InferOutputShape(bool ignore_error = false) override {
        if (input_blobs_.size() < 3 || output_blobs_.size() != 2)
            return Status(TNNERR_PARAM_ERR, "RocmLayerNormQuant needs x, scale, bias and two outputs");
        return RocmFusedLayerBase::InferOutputShape(ignore_error);
    }
};

// RocmGeluInt8: element-wise on an int8 blob
class RocmGeluInt8Layer : public RocmFusedLayerBase {
public:
    explicit RocmGeluInt8Layer(LayerType type) : RocmFusedLayerBase(type) {}
};

TypeLayerRegister<TypeLayerCreator<RocmFusedLinearLayer>> g_rocm_fused_linear_layer(LAYER_ROCM_FUSED_LINEAR);
TypeLayerRegister<TypeLayerCreator<RocmFusedAttentionLayer>> g_rocm_fused_attention_layer(LAYER_ROCM_FUSED_ATTENTION);
TypeLayerRegister<TypeLayerCreator<RocmFusedEmbeddingLayer>> g_rocm_fused_embedding_layer(LAYER_ROCM_FUSED_EMBEDDING);
TypeLayerRegister<TypeLayerCreator<RocmInt8LinearLayer>> g_rocm_fused_linear_int8_layer(LAYER_ROCM_FUSED_LINEAR_INT8);
TypeLayerRegister<TypeLayerCreator<RocmInt8LinearLayer>> g_rocm_quant_linear_gelu_layer(LAYER_ROCM_QUANT_LINEAR_GELU);
TypeLayerRegister<TypeLayerCreator<RocmGeluInt8Layer>> g_rocm_gelu_int8_layer(LAYER_ROCM_GELU_INT8);
TypeLayerRegister<TypeLayerCreator<RocmLayerNormQuantLayer>> g_rocm_layer_norm_quant_layer(LAYER_ROCM_LAYER_NORM_QUANT);

}  // namespace
}  // namespace TNN_NS
