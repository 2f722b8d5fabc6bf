// One AbstractLayerAcc per op of the decomposed encoder graph, so unchanged protos run on DEVICE_ROCM
// before (or without) the fusion pass: MatMul, InnerProduct (fp and int8), Add/Sub/Mul/Div, Softmax,
// LayerNorm, GELU, Permute, Reshape, Reformat, Gather, Cast.
//
// Each Forward only enqueues kernels on the context's stream (DefaultNetwork::Forward synchronises once
// at the end, source/tnn/core/default_network.cc:632-633).  dtype-dependent preparation (weight upload in
// the activation dtype) happens in Reshape(), when every blob's data type is final.
#include <cfloat>
#include <cmath>

#include "rocm_device.h"

namespace TNN_NS {

namespace {
bool IsFloatType(DataType t) { return t == DATA_TYPE_FLOAT || t == DATA_TYPE_HALF || t == DATA_TYPE_BFP16; }
Status Unsupported(const std::string &who, DataType t) {
    return Status(TNNERR_LAYER_ERR, who + " dont support data type: " + std::to_string((int)t));
}
}  // namespace

// ---- MatMul (cpu_mat_mul_layer_acc.cc:64-117, x86_mat_mul_layer_acc.cc:49-114) ---------------------
class RocmMatMulLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        if (inputs.size() == 2 || weight_)
            return TNN_OK;
        auto res = dynamic_cast<MatMulLayerResource *>(resource_);
        CHECK_PARAM_NULL(res);
        DataType wt = res->weight.GetDataType();
        if (wt != DATA_TYPE_FLOAT && wt != DATA_TYPE_HALF)  // cpu_mat_mul_layer_acc.cc:45-56
            return Status(TNNERR_PARAM_ERR, "MatMul has invalid direction param");
        return UploadConverted(res->weight.force_to<void *>(), (size_t)res->weight.GetDataCount(), wt,
                               inputs[0]->GetBlobDesc().data_type, &weight_);
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<MatMulLayerParam *>(param_);
        CHECK_PARAM_NULL(param);
        DataType dt = inputs[0]->GetBlobDesc().data_type;
        if (!IsFloatType(dt))
            return Unsupported("RocmMatMulLayerAcc", dt);
        DimsVector a_dims = param->matrix_a_dims, b_dims = param->matrix_b_dims;
        if (a_dims.size() == 1)
            a_dims.insert(a_dims.begin(), 1);
        if (b_dims.size() == 1)
            b_dims.push_back(1);
        const void *a, *b;
        if (inputs.size() == 2) {
            a = Ptr(In(inputs[0]));
            b = Ptr(In(inputs[1]));
        } else {
            a = param->weight_position == 0 ? weight_ : Ptr(inputs[0]);
            b = param->weight_position == 1 ? weight_ : Ptr(inputs[0]);
        }
        auto c_dims = outputs[0]->GetBlobDesc().dims;
        int M = a_dims[a_dims.size() - 2], K = a_dims.back(), N = b_dims.back();
        if (M * K == 0 || K * N == 0 || M * N == 0)
            return TNN_OK;
        int batch_a = DimsVectorUtils::Count(a_dims) / (M * K);
        int batch_b = DimsVectorUtils::Count(b_dims) / (K * N);
        int batch_c = DimsVectorUtils::Count(c_dims) / (M * N);
        if (batch_a == batch_c && batch_b == 1 && batch_c > 1) {
            // weight / shared right operand: fold the batch into the rows, one large GEMM
            ROCM_CALL(tnn_rocm_gemm(Stream(), (int)dt, 0, a, b, Ptr(outputs[0]), M * batch_c, N, K, K, N, N, 1, 1, 1, 0,
                                    nullptr, nullptr, 0));
            return TNN_OK;
        }
        if (batch_a > batch_c || batch_b > batch_c)
            return Status(TNNERR_PARAM_ERR, "MatMul batch broadcast not representable");
        ROCM_CALL(tnn_rocm_gemm(Stream(), (int)dt, 0, a, b, Ptr(outputs[0]), M, N, K, K, N, N, batch_c, batch_a, batch_b,
                                0, nullptr, nullptr, 0));
        return TNN_OK;
    }

private:
    void *weight_ = nullptr;
};
REGISTER_ROCM_ACC(RocmMatMulLayerAcc, LAYER_MATMUL);

// ---- InnerProduct (fp: naive_compute.cc:271-288 ; int8: naive_compute.cc:316-347, x86_compute_int8.cc:833-914) ----
class RocmInnerProductLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        if (weight_)
            return TNN_OK;
        auto param = dynamic_cast<InnerProductLayerParam *>(param_);
        auto res   = dynamic_cast<InnerProductLayerResource *>(resource_);
        if (!param)
            return Status(TNNERR_MODEL_ERR, "Error: InnerProductLayerParam is nil");
        if (!res)
            return Status(TNNERR_MODEL_ERR, "Error: InnerProductLayerResource is nil");
        DataType dt  = outputs[0]->GetBlobDesc().data_type;
        const int N  = param->num_output;
        auto in_dims = inputs[0]->GetBlobDesc().dims;
        const int K  = DimsVectorUtils::Count(in_dims, param->axis);
        if ((long)res->weight_handle.GetDataCount() != (long)N * K)
            return Status(TNNERR_MODEL_ERR, "InnerProduct weight size does not match num_output x K");
        if (dt == DATA_TYPE_INT8) {
            if (res->weight_handle.GetDataType() != DATA_TYPE_INT8)
                return Status(TNNERR_MODEL_ERR, "quantized InnerProduct needs int8 weights");
            RETURN_ON_NEQ(UploadConverted(res->weight_handle.force_to<void *>(), (size_t)N * K, DATA_TYPE_INT8,
                                          DATA_TYPE_INT8, &weight_), TNN_OK);
            // requantisation factor = w_scale / o_scale as one fp32 division on the host, 0 when o_scale < FLT_MIN
            // (cpu_inner_product_layer_acc.cc:50-76, x86_inner_product_layer_acc.cc:197-222)
            auto out8 = dynamic_cast<BlobInt8 *>(outputs[0]);
            if (!out8 || !out8->GetIntResource())
                return Status(TNNERR_NULL_PARAM, "int8 output blob without scale resource");
            const float *w_scale = res->scale_handle.force_to<float *>();
            CHECK_PARAM_NULL(w_scale);
            const float *o_scale = out8->GetIntResource()->scale_handle.force_to<float *>();
            int n_w = res->scale_handle.GetDataCount(), n_o = out8->GetIntResource()->scale_handle.GetDataCount();
            std::vector<float> scale(N);
            for (int i = 0; i < N; ++i) {
                float os = o_scale[n_o == 1 ? 0 : i];
                scale[i] = os >= FLT_MIN ? w_scale[n_w == 1 ? 0 : i] / os : 0.0f;
            }
            RETURN_ON_NEQ(UploadConverted(scale.data(), (size_t)N, DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &scale_), TNN_OK);
            if (param->has_bias && res->bias_handle.GetDataCount() == N)
                RETURN_ON_NEQ(UploadConverted(res->bias_handle.force_to<void *>(), (size_t)N, DATA_TYPE_INT32,
                                              DATA_TYPE_INT32, &bias_), TNN_OK);
            return TNN_OK;
        }
        if (!IsFloatType(dt))
            return Unsupported("RocmInnerProductLayerAcc", dt);
        DataType wt = res->weight_handle.GetDataType();
        if (!IsFloatType(wt))
            return Status(TNNERR_MODEL_ERR, "float InnerProduct needs float weights");
        RETURN_ON_NEQ(UploadConverted(res->weight_handle.force_to<void *>(), (size_t)N * K, wt, dt, &weight_), TNN_OK);
        if (param->has_bias && res->bias_handle.GetDataCount() == N)
            RETURN_ON_NEQ(UploadConverted(res->bias_handle.force_to<void *>(), (size_t)N, res->bias_handle.GetDataType(),
                                          DATA_TYPE_FLOAT, &bias_), TNN_OK);
        return TNN_OK;
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param   = dynamic_cast<InnerProductLayerParam *>(param_);
        auto in_dims = inputs[0]->GetBlobDesc().dims;
        const int N = param->num_output, K = DimsVectorUtils::Count(in_dims, param->axis);
        const int rows = DimsVectorUtils::Count(in_dims, 0, param->axis);
        DataType dt    = outputs[0]->GetBlobDesc().data_type;
        if (dt == DATA_TYPE_INT8) {
            ROCM_CALL(tnn_rocm_gemm_i8(Stream(), (const int8_t *)Ptr(inputs[0]), (const int8_t *)weight_,
                                       (const int32_t *)bias_, (const float *)scale_, (int8_t *)Ptr(outputs[0]), nullptr,
                                       rows, N, K, K, K, N, nullptr, 0, 0.f));
            return TNN_OK;
        }
        ROCM_CALL(tnn_rocm_gemm(Stream(), (int)dt, 1, Ptr(inputs[0]), weight_, Ptr(outputs[0]), rows, N, K, K, K, N, 1, 1, 1,
                                bias_ ? TNN_ROCM_EPI_BIAS : 0, (const float *)bias_, nullptr, 0));
        return TNN_OK;
    }

private:
    void *weight_ = nullptr, *bias_ = nullptr, *scale_ = nullptr;
};
REGISTER_ROCM_ACC(RocmInnerProductLayerAcc, LAYER_INNER_PRODUCT);

// ---- Add / Sub / Mul / Div (compute_elewise.cc:37-65 ; int8 add x86_compute_int8.cc:795-831) ----------
template <int OP> class RocmBinaryLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto res = dynamic_cast<EltwiseLayerResource *>(resource_);
        if (!res || weight_ || res->element_handle.GetBytesSize() == 0)
            return TNN_OK;
        DataType dt = inputs[0]->GetBlobDesc().data_type;
        if (!IsFloatType(dt))
            return Unsupported("RocmBinaryLayerAcc", dt);
        return UploadConverted(res->element_handle.force_to<void *>(), (size_t)res->element_handle.GetDataCount(),
                               res->element_handle.GetDataType(), dt, &weight_);
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<MultidirBroadcastLayerParam *>(param_);
        auto res   = dynamic_cast<EltwiseLayerResource *>(resource_);
        DataType dt = outputs[0]->GetBlobDesc().data_type;
        auto out_dims = outputs[0]->GetBlobDesc().dims;
        if (dt == DATA_TYPE_INT8) {
            if (OP != 0 || inputs.size() != 2)
                return Status(TNNERR_LAYER_ERR, "int8 element-wise op other than a 2-input Add");
            float s[3];
            Blob *bl[3] = {inputs[0], inputs[1], outputs[0]};
            const int channels = out_dims.size() > 1 ? out_dims[1] : 1;
            const size_t inner = out_dims.size() > 2 ? (size_t)DimsVectorUtils::Count(out_dims, 2) : 1;
            bool per_channel = false;
            const float *hs[3];
            int ns[3];
            for (int i = 0; i < 3; ++i) {
                auto b8 = dynamic_cast<BlobInt8 *>(bl[i]);
                if (!b8 || !b8->GetIntResource())
                    return Status(TNNERR_LAYER_ERR, "int8 Add needs blob scales");
                ns[i] = b8->GetIntResource()->scale_handle.GetDataCount();
                hs[i] = b8->GetIntResource()->scale_handle.force_to<float *>();
                if (ns[i] != 1 && ns[i] < channels)
                    return Status(TNNERR_LAYER_ERR, "int8 Add: a blob has fewer scales than channels");
                per_channel |= ns[i] != 1;
                s[i] = hs[i][0];
            }
            if (per_channel) {
                // one scale per channel (dims[1]): the three arrays x86_add_layer_acc.cc:33-66 prepares, kept on the device
                if (!chan_scale_ || chan_count_ != channels) {
                    std::vector<float> host(3 * (size_t)channels);
                    for (int c = 0; c < channels; ++c) {
                        host[c]                = hs[0][ns[0] == 1 ? 0 : c];
                        host[channels + c]     = hs[1][ns[1] == 1 ? 0 : c];
                        host[2 * channels + c] = (float)(1.0 / hs[2][ns[2] == 1 ? 0 : c]);
                    }
                    chan_scale_ = nullptr;
                    RETURN_ON_NEQ(UploadConverted(host.data(), host.size(), DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &chan_scale_), TNN_OK);
                    chan_count_ = channels;
                }
                const float *d = (const float *)chan_scale_;
                ROCM_CALL(tnn_rocm_add_i8_per_channel(Stream(), (const int8_t *)Ptr(inputs[0]), d, (const int8_t *)Ptr(inputs[1]),
                                                      d + channels, d + 2 * channels, (int8_t *)Ptr(outputs[0]),
                                                      (size_t)DimsVectorUtils::Count(out_dims), channels > 0 ? channels : 1,
                                                      inner > 0 ? inner : 1));
                return TNN_OK;
            }
            float inv_so = (float)(1.0 / s[2]);  // x86_add_layer_acc.cc:54-58
            ROCM_CALL(tnn_rocm_add_i8(Stream(), (const int8_t *)Ptr(inputs[0]), s[0], (const int8_t *)Ptr(inputs[1]), s[1],
                                      inv_so, (int8_t *)Ptr(outputs[0]), (size_t)DimsVectorUtils::Count(out_dims),
                                      channels > 0 ? channels : 1, inner > 0 ? inner : 1));
            return TNN_OK;
        }
        if (!IsFloatType(dt))
            return Unsupported("RocmBinaryLayerAcc", dt);
        // operand list in evaluation order: inputs, with the resource weight spliced in at weight_input_index
        struct Operand {
            const void *ptr;
            DimsVector dims;
        };
        std::vector<Operand> ops;
        for (auto b : inputs)
            ops.push_back({Ptr(In(b)), In(b)->GetBlobDesc().dims});
        if (weight_ && res) {
            // the shape the layer derived for the resource operand must be the shape of what was uploaded
            if ((long)DimsVectorUtils::Count(res->element_shape) != (long)res->element_handle.GetDataCount())
                return Status(TNNERR_MODEL_ERR, "binary op: the resource operand's shape does not match its data");
            Operand w{weight_, res->element_shape};
            if (param && param->weight_input_index == 0)
                ops.insert(ops.begin(), w);
            else
                ops.push_back(w);
        }
        if (ops.size() < 2)
            return Status(TNNERR_LAYER_ERR, "binary op needs two operands");
        if (out_dims.size() > 6)
            return Status(TNNERR_LAYER_ERR, "binary op rank above 6");
        const void *acc_ptr = ops[0].ptr;
        DimsVector acc_dims = ops[0].dims;
        for (size_t i = 1; i < ops.size(); ++i) {
            bool last = i + 1 == ops.size();
            // intermediate results of >2-operand chains take the output buffer as well (same shape from i=1 on)
            DimsVector cur_out = out_dims;
            ROCM_CALL(tnn_rocm_binary(Stream(), (int)dt, OP, acc_ptr, acc_dims.data(), (int)acc_dims.size(), ops[i].ptr,
                                      ops[i].dims.data(), (int)ops[i].dims.size(), Ptr(outputs[0]), cur_out.data(),
                                      (int)cur_out.size()));
            acc_ptr  = Ptr(outputs[0]);
            acc_dims = cur_out;
            (void)last;
        }
        return TNN_OK;
    }

private:
    void *weight_ = nullptr;
    void *chan_scale_ = nullptr;  // int8 Add with per-channel blob scales: a, b scales and reciprocal output scales
    int chan_count_   = 0;
};
typedef RocmBinaryLayerAcc<0> RocmAddLayerAcc;
typedef RocmBinaryLayerAcc<1> RocmSubLayerAcc;
typedef RocmBinaryLayerAcc<2> RocmMulLayerAcc;
typedef RocmBinaryLayerAcc<3> RocmDivLayerAcc;
REGISTER_ROCM_ACC(RocmAddLayerAcc, LAYER_ADD);
REGISTER_ROCM_ACC(RocmSubLayerAcc, LAYER_SUB);
REGISTER_ROCM_ACC(RocmMulLayerAcc, LAYER_MUL);
REGISTER_ROCM_ACC(RocmDivLayerAcc, LAYER_DIV);

// ---- Softmax (cpu_softmax_layer_acc.cc:30-97) -----------------------------------------------------------
class RocmSoftmaxLayerAcc : public RocmLayerAcc {
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<SoftmaxLayerParam *>(param_);
        if (!param)
            return Status(TNNERR_MODEL_ERR, "Error: SoftmaxLayerParam is unsupported");
        auto dims   = inputs[0]->GetBlobDesc().dims;
        DataType dt = inputs[0]->GetBlobDesc().data_type;
        if (!IsFloatType(dt))
            return Unsupported("RocmSoftmaxLayerAcc", dt);
        if (dims.empty())
            return Status(TNNERR_PARAM_ERR, "softmax on a rank-0 blob");
        int axis = (int)((param->axis + (int)dims.size()) % (int)dims.size());
        ROCM_CALL(tnn_rocm_softmax(Stream(), (int)dt, Ptr(inputs[0]), Ptr(outputs[0]), DimsVectorUtils::Count(dims, 0, axis),
                                   dims[axis], DimsVectorUtils::Count(dims, axis + 1)));
        return TNN_OK;
    }
};
REGISTER_ROCM_ACC(RocmSoftmaxLayerAcc, LAYER_SOFTMAX);

// ---- LayerNorm (cpu_layer_norm_layer_acc.cc:30-140) ------------------------------------------------------
class RocmLayerNormLayerAcc : public RocmLayerAcc {
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<LayerNormLayerParam *>(param_);
        CHECK_PARAM_NULL(param);
        if (inputs.size() < 3)
            return Status(TNNERR_PARAM_ERR, "LayerNormLayer has no input blob of scale or bias");
        Blob *scale = In(inputs[1]), *bias = In(inputs[2]);
        auto dims_in = inputs[0]->GetBlobDesc().dims, dims_s = scale->GetBlobDesc().dims;
        if (!DimsVectorUtils::Equal(dims_s, bias->GetBlobDesc().dims))
            return Status(TNNERR_PARAM_ERR, "LayerNormLayer has invalid dims for input blob of scale or bias");
        int offset = (int)dims_in.size() - (int)dims_s.size();
        for (int i = 0; i < (int)dims_s.size(); ++i)
            if (offset < 0 || dims_in[i + offset] != dims_s[i])
                return Status(TNNERR_PARAM_ERR, "LayerNormLayer has invalid dims for input blob");
        param->reduce_dims_size = (int)dims_s.size();  // InferRuntimeOutputShape, cpu_layer_norm_layer_acc.cc:30-61
        DataType dt = outputs[0]->GetBlobDesc().data_type;
        if (!IsFloatType(dt))
            return Unsupported("RocmLayerNormLayerAcc", dt);
        int rows = DimsVectorUtils::Count(dims_in, 0, offset), cols = DimsVectorUtils::Count(dims_in, offset);
        if (rows == 0 || cols == 0)
            return Status(TNNERR_COMMON_ERROR, "Error: blob count is zero");
        // Scale and bias are constants of the model as a rule (kept in fp32, ConstantBlobDataType below).  When they are
        // ordinary input blobs (the reference's layer test feeds them so, test_layer_norm_layer.cc:70) they carry the
        // network's float type and are widened into a side buffer of the context first.
        const float *gamma = (const float *)Ptr(scale), *beta = (const float *)Ptr(bias);
        const DataType st = scale->GetBlobDesc().data_type, bt = bias->GetBlobDesc().data_type;
        if (!IsFloatType(st) || !IsFloatType(bt))
            return Unsupported("RocmLayerNormLayerAcc scale/bias", IsFloatType(st) ? bt : st);
        if (st != DATA_TYPE_FLOAT || bt != DATA_TYPE_FLOAT) {
            void *wide = nullptr;
            RETURN_ON_NEQ(context_->SideBuffer(param_->name + "/layernorm_scale_bias_f32", (size_t)cols * 2 * sizeof(float), &wide),
                          TNN_OK);
            float *w = (float *)wide;
            ROCM_CALL(tnn_rocm_cast(Stream(), (int)st, Ptr(scale), (int)DATA_TYPE_FLOAT, w, (size_t)cols));
            ROCM_CALL(tnn_rocm_cast(Stream(), (int)bt, Ptr(bias), (int)DATA_TYPE_FLOAT, w + cols, (size_t)cols));
            gamma = w;
            beta  = w + cols;
        }
        // a second output (added by the ROCm int8 pass in place of a following Reformat layer) receives the
        // quantised copy of the first: float2int8(y * float(1.0 / scale)) on the value as stored in the float blob
        // (x86_reformat_layer_acc.cc:66-75, x86_compute_int8.cc:1254-1318)
        int8_t *out_q = nullptr;
        float q_inv   = 0.f;
        if (outputs.size() >= 2) {
            auto b8 = dynamic_cast<BlobInt8 *>(outputs[1]);
            if (!b8 || !b8->GetIntResource() || b8->GetIntResource()->scale_handle.GetDataCount() != 1)
                return Status(TNNERR_LAYER_ERR, "LayerNorm quantised output needs a per-tensor blob scale");
            q_inv = (float)(1.0 / b8->GetIntResource()->scale_handle.force_to<float *>()[0]);
            out_q = (int8_t *)Ptr(outputs[1]);
        }
        ROCM_CALL(tnn_rocm_layernorm(Stream(), (int)dt, Ptr(inputs[0]), nullptr, gamma, beta, Ptr(outputs[0]), rows, cols,
                                     param->eps, out_q, q_inv));
        return TNN_OK;
    }

protected:
    DataType ConstantBlobDataType(const std::vector<Blob *> &, int) override { return DATA_TYPE_FLOAT; }
};
REGISTER_ROCM_ACC(RocmLayerNormLayerAcc, LAYER_LAYER_NORM);
// the same kernel with its second, quantised output (the layer the ROCm int8 pass makes of LayerNorm -> Reformat)
class RocmLayerNormQuantLayerAcc : public RocmLayerNormLayerAcc {};
REGISTER_ROCM_ACC(RocmLayerNormQuantLayerAcc, LAYER_ROCM_LAYER_NORM_QUANT);

// ---- GELU (cpu_gelu_layer_acc.cc:31-51) --------------------------------------------------------------------
class RocmGeluLayerAcc : public RocmLayerAcc {
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        DataType dt = outputs[0]->GetBlobDesc().data_type;
        if (!IsFloatType(dt))
            return Status(TNNERR_NO_RESULT, "RocmGeluLayerAcc dont support data type");
        ROCM_CALL(tnn_rocm_gelu(Stream(), (int)dt, Ptr(inputs[0]), Ptr(outputs[0]),
                                (size_t)DimsVectorUtils::Count(outputs[0]->GetBlobDesc().dims)));
        return TNN_OK;
    }
};
REGISTER_ROCM_ACC(RocmGeluLayerAcc, LAYER_GELU);

class RocmTanhLayerAcc : public RocmLayerAcc {  // cpu_tanh_layer_acc.cc:23-31
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        DataType dt = outputs[0]->GetBlobDesc().data_type;
        if (!IsFloatType(dt))
            return Status(TNNERR_LAYER_ERR, "RocmTanhLayerAcc dont support data type");
        ROCM_CALL(tnn_rocm_tanh(Stream(), (int)dt, Ptr(inputs[0]), Ptr(outputs[0]),
                                (size_t)DimsVectorUtils::Count(outputs[0]->GetBlobDesc().dims)));
        return TNN_OK;
    }
};
REGISTER_ROCM_ACC(RocmTanhLayerAcc, LAYER_TANH);

// ---- Permute / Reshape (naive_compute.cc:943-956 ; reshape is a copy) ----------------------------------------
class RocmPermuteLayerAcc : public RocmLayerAcc {
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<PermuteLayerParam *>(param_);
        CHECK_PARAM_NULL(param);
        auto dims = inputs[0]->GetBlobDesc().dims;
        if (dims.size() > 6 || param->orders.size() != dims.size())
            return Status(TNNERR_PARAM_ERR, "Permute rank unsupported or order size mismatch");
        int es = DataTypeUtils::GetBytesSize(inputs[0]->GetBlobDesc().data_type);
        ROCM_CALL(tnn_rocm_permute(Stream(), es, Ptr(inputs[0]), Ptr(outputs[0]), dims.data(), param->orders.data(),
                                   (int)dims.size()));
        return TNN_OK;
    }
};
REGISTER_ROCM_ACC(RocmPermuteLayerAcc, LAYER_PERMUTE);

class RocmReshapeLayerAcc : public RocmLayerAcc {
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<ReshapeLayerParam *>(param_);
        size_t bytes = (size_t)DimsVectorUtils::Count(outputs[0]->GetBlobDesc().dims) *
                       DataTypeUtils::GetBytesSize(outputs[0]->GetBlobDesc().data_type);
        if (param && param->reshape_type == 1) {
            // The "TensorFlow" reshape (cpu_reshape_layer_acc.cc:101-131): the input, taken as [N,C,H,W], is laid out
            // channels-last, and that sequence of values, taken as channels-last data of the OUTPUT's [N,C,H,W], is
            // brought back to channels-first.  Two permutes through the context workspace.
            auto nchw = [](const DimsVector &d) {
                return std::vector<int>{d.size() > 0 ? d[0] : 1, d.size() > 1 ? d[1] : 1, d.size() > 2 ? d[2] : 1,
                                        d.size() > 3 ? d[3] : 1};
            };
            const DimsVector od = outputs[0]->GetBlobDesc().dims, id = inputs[0]->GetBlobDesc().dims;
            if (od.size() > 4 || id.size() > 4)
                return Status(TNNERR_MODEL_ERR, "Error: RocmReshapeLayerAcc: reshape type 1 does not support dims > 4");
            if (bytes == 0)
                return TNN_OK;
            const int es = DataTypeUtils::GetBytesSize(outputs[0]->GetBlobDesc().data_type);
            void *tmp    = nullptr;
            RETURN_ON_NEQ(context_->Workspace(bytes, &tmp), TNN_OK);
            std::vector<int> in4 = nchw(id), out4 = nchw(od);
            const int to_last[4]  = {0, 2, 3, 1};
            ROCM_CALL(tnn_rocm_permute(Stream(), es, Ptr(inputs[0]), tmp, in4.data(), to_last, 4));
            const int nhwc[4]     = {out4[0], out4[2], out4[3], out4[1]};
            const int to_first[4] = {0, 3, 1, 2};
            ROCM_CALL(tnn_rocm_permute(Stream(), es, tmp, Ptr(outputs[0]), nhwc, to_first, 4));
            return TNN_OK;
        }
        if (param && param->reshape_type != 0)
            return Status(TNNERR_MODEL_ERR, "Error: RocmReshapeLayerAcc: unsupported reshape type");
        if (Ptr(outputs[0]) == Ptr(inputs[0]))
            return TNN_OK;  // the memory planner let the output share the input's buffer: nothing to move
        ROCM_CALL(tnn_rocm_memcpy_d2d(Ptr(outputs[0]), Ptr(inputs[0]), bytes, Stream()));
        return TNN_OK;
    }
};
REGISTER_ROCM_ACC(RocmReshapeLayerAcc, LAYER_RESHAPE);
// Squeeze / Unsqueeze only rename dimensions (cpu_squeeze_layer_acc.cc, cpu_unsqueeze_layer_acc.cc: one copy)
class RocmSqueezeLayerAcc : public RocmReshapeLayerAcc {};
class RocmUnsqueezeLayerAcc : public RocmReshapeLayerAcc {};
REGISTER_ROCM_ACC(RocmSqueezeLayerAcc, LAYER_SQUEEZE);
REGISTER_ROCM_ACC(RocmUnsqueezeLayerAcc, LAYER_UNSQUEEZE);

// ---- Reformat: float <-> int8 (x86_reformat_layer_acc.cc:50-80, x86_compute_int8.cc:1193-1318) -------------------
class RocmReformatLayerAcc : public RocmLayerAcc {
public:
    // the direction follows from the two data types, and the acc records it in the param like the engine's own
    // Reformat accs do (x86_reformat_layer_acc.cc:29-44)
    Status Init(Context *context, LayerParam *param, LayerResource *resource, const std::vector<Blob *> &inputs,
                const std::vector<Blob *> &outputs) override {
        RETURN_ON_NEQ(RocmLayerAcc::Init(context, param, resource, inputs, outputs), TNN_OK);
        auto p = dynamic_cast<ReformatLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        if (p->src_type == DATA_TYPE_INT8 && IsFloatType(p->dst_type)) {
            p->type = DEQUANT_ONLY;
            mode_   = kDequant;
        } else if (IsFloatType(p->src_type) && p->dst_type == DATA_TYPE_INT8) {
            p->type = QUANT_ONLY;
            mode_   = kQuant;
        } else if (IsFloatType(p->src_type) && IsFloatType(p->dst_type)) {
            mode_ = kCast;
        } else {
            return Status(TNNERR_MODEL_ERR, "unsupport precision mode");
        }
        return TNN_OK;
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        for (size_t i = 0; i < inputs.size(); ++i) {
            size_t count = (size_t)DimsVectorUtils::Count(outputs[i]->GetBlobDesc().dims);
            DataType st = inputs[i]->GetBlobDesc().data_type, dt = outputs[i]->GetBlobDesc().data_type;
            if (mode_ == kQuant || mode_ == kDequant) {
                // the int8 side's blob scale: one value, or one per channel (dims[1]) as x86_reformat_layer_acc.cc:50-80
                // prepares them (reciprocals for the quantiser: a double division stored as float)
                auto b8 = dynamic_cast<BlobInt8 *>(mode_ == kQuant ? outputs[i] : inputs[i]);
                if (!b8 || !b8->GetIntResource() || !IsFloatType(mode_ == kQuant ? st : dt))
                    return Status(TNNERR_LAYER_ERR, "Reformat needs a float blob on one side and an int8 blob with a scale on the other");
                const auto &dims   = outputs[i]->GetBlobDesc().dims;
                const int channels = dims.size() > 1 ? dims[1] : 1;
                const size_t inner = dims.size() > 2 ? (size_t)DimsVectorUtils::Count(dims, 2) : 1;
                const int ns       = b8->GetIntResource()->scale_handle.GetDataCount();
                const float *hs    = b8->GetIntResource()->scale_handle.force_to<float *>();
                if (ns != 1 && ns < channels)
                    return Status(TNNERR_LAYER_ERR, "Reformat: the int8 blob has fewer scales than channels");
                if (ns != 1) {
                    if (i >= chan_scale_.size())
                        chan_scale_.resize(i + 1, nullptr), chan_count_.resize(i + 1, 0);
                    if (!chan_scale_[i] || chan_count_[i] != channels) {
                        std::vector<float> host((size_t)channels);
                        for (int c = 0; c < channels; ++c)
                            host[c] = mode_ == kQuant ? (float)(1.0 / hs[c]) : hs[c];
                        chan_scale_[i] = nullptr;
                        RETURN_ON_NEQ(UploadConverted(host.data(), host.size(), DATA_TYPE_FLOAT, DATA_TYPE_FLOAT, &chan_scale_[i]), TNN_OK);
                        chan_count_[i] = channels;
                    }
                    if (mode_ == kQuant)
                        ROCM_CALL(tnn_rocm_quantize_per_channel(Stream(), (int)st, Ptr(inputs[i]), (const float *)chan_scale_[i],
                                                                (int8_t *)Ptr(outputs[i]), count, channels, inner > 0 ? inner : 1));
                    else
                        ROCM_CALL(tnn_rocm_dequantize_per_channel(Stream(), (const int8_t *)Ptr(inputs[i]), (const float *)chan_scale_[i],
                                                                  (int)dt, Ptr(outputs[i]), count, channels, inner > 0 ? inner : 1));
                } else if (mode_ == kQuant) {
                    float inv = (float)(1.0 / hs[0]);  // x86_reformat_layer_acc.cc:70 : double division, stored as float
                    ROCM_CALL(tnn_rocm_quantize(Stream(), (int)st, Ptr(inputs[i]), inv, (int8_t *)Ptr(outputs[i]), count));
                } else {
                    ROCM_CALL(tnn_rocm_dequantize(Stream(), (const int8_t *)Ptr(inputs[i]), hs[0], (int)dt, Ptr(outputs[i]), count));
                }
            } else if (IsFloatType(st) && IsFloatType(dt)) {
                ROCM_CALL(tnn_rocm_cast(Stream(), (int)st, Ptr(inputs[i]), (int)dt, Ptr(outputs[i]), count));
            } else {
                return Status(TNNERR_MODEL_ERR, "unsupport precision mode");
            }
        }
        return TNN_OK;
    }

private:
    enum { kQuant, kDequant, kCast } mode_ = kCast;
    std::vector<void *> chan_scale_;  // per blob pair: the per-channel scales (reciprocals for the quantiser) on the device
    std::vector<int> chan_count_;
};
REGISTER_ROCM_ACC(RocmReformatLayerAcc, LAYER_REFORMAT);

// ---- Gather (cpu_gather_layer_acc.cc:27-86) -----------------------------------------------------------------------
class RocmGatherLayerAcc : public RocmLayerAcc {
public:
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<GatherLayerParam *>(param_);
        auto res   = dynamic_cast<GatherLayerResource *>(resource_);
        CHECK_PARAM_NULL(param);
        if ((param->data_in_resource || param->indices_in_resource) && !res)
            return Status(TNNERR_MODEL_ERR, "Gather resource is invalid");
        if (param->data_in_resource && !data_) {
            DataType st = res->data.GetDataType(), dt = outputs[0]->GetBlobDesc().data_type;
            RETURN_ON_NEQ(UploadConverted(res->data.force_to<void *>(), (size_t)res->data.GetDataCount(), st,
                                          IsFloatType(st) ? dt : st, &data_), TNN_OK);
        }
        if (param->indices_in_resource && !indices_) {
            if (res->indices.GetDataType() != DATA_TYPE_INT32)
                return Status(TNNERR_MODEL_ERR, "Gather indices must be int32");
            RETURN_ON_NEQ(UploadConverted(res->indices.force_to<void *>(), (size_t)res->indices.GetDataCount(),
                                          DATA_TYPE_INT32, DATA_TYPE_INT32, &indices_), TNN_OK);
        }
        return TNN_OK;
    }
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        auto param = dynamic_cast<GatherLayerParam *>(param_);
        auto res   = dynamic_cast<GatherLayerResource *>(resource_);
        CHECK_PARAM_NULL(param);
        if ((param->data_in_resource || param->indices_in_resource) && !res)
            return Status(TNNERR_MODEL_ERR, "Gather resource is invalid");
        if (inputs.size() < (size_t)(!param->data_in_resource) + (size_t)(!param->indices_in_resource))
            return Status(TNNERR_MODEL_ERR, "Gather with fewer input blobs than operands outside its resource");
        DimsVector data_dims = param->data_in_resource ? res->data.GetBufferDims() : inputs.front()->GetBlobDesc().dims;
        DimsVector idx_dims  = param->indices_in_resource ? res->indices.GetBufferDims() : inputs.back()->GetBlobDesc().dims;
        if (param->axis < 0 || param->axis >= (int)data_dims.size())
            return Status(TNNERR_PARAM_ERR, "Gather axis out of range");
        if ((param->data_in_resource && (long)DimsVectorUtils::Count(data_dims) != (long)res->data.GetDataCount()) ||
            (param->indices_in_resource && (long)DimsVectorUtils::Count(idx_dims) != (long)res->indices.GetDataCount()))
            return Status(TNNERR_MODEL_ERR, "Gather: the dims of a resource operand do not match its data");
        const void *data = param->data_in_resource ? data_ : Ptr(In(inputs.front()));
        const void *idx  = param->indices_in_resource ? indices_ : Ptr(In(inputs.back()));
        if (!param->indices_in_resource && inputs.back()->GetBlobDesc().data_type != DATA_TYPE_INT32)
            return Status(TNNERR_MODEL_ERR, "Gather indices blob must be int32");
        int axis  = param->axis;
        int es    = DataTypeUtils::GetBytesSize(outputs[0]->GetBlobDesc().data_type);
        int batch = DimsVectorUtils::Count(data_dims, 0, axis), slices = data_dims[axis];
        size_t slice_bytes = (size_t)DimsVectorUtils::Count(data_dims, axis + 1) * es;
        ROCM_CALL(tnn_rocm_gather(Stream(), data, (const int32_t *)idx, Ptr(outputs[0]), batch, slices, slice_bytes,
                                  DimsVectorUtils::Count(idx_dims), context_->ErrorFlag()));
        return TNN_OK;
    }

private:
    void *data_ = nullptr, *indices_ = nullptr;
};
REGISTER_ROCM_ACC(RocmGatherLayerAcc, LAYER_GATHER);

// ---- Cast ----------------------------------------------------------------------------------------------------------
class RocmCastLayerAcc : public RocmLayerAcc {
public:
    Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override {
        DataType st = inputs[0]->GetBlobDesc().data_type, dt = outputs[0]->GetBlobDesc().data_type;
        size_t count = (size_t)DimsVectorUtils::Count(outputs[0]->GetBlobDesc().dims);
        if (IsFloatType(st) && IsFloatType(dt)) {
            ROCM_CALL(tnn_rocm_cast(Stream(), (int)st, Ptr(inputs[0]), (int)dt, Ptr(outputs[0]), count));
            return TNN_OK;
        }
        if (st == dt) {
            ROCM_CALL(tnn_rocm_memcpy_d2d(Ptr(outputs[0]), Ptr(inputs[0]), count * DataTypeUtils::GetBytesSize(st), Stream()));
            return TNN_OK;
        }
        if ((st == DATA_TYPE_INT32 && IsFloatType(dt)) || (IsFloatType(st) && dt == DATA_TYPE_INT32)) {
            // cpu_cast_layer_acc.cc:41-53; a float output follows the network precision like every float blob
            ROCM_CALL(tnn_rocm_cast(Stream(), (int)st, Ptr(inputs[0]), (int)dt, Ptr(outputs[0]), count));
            return TNN_OK;
        }
        return Status(TNNERR_LAYER_ERR, "Cast between these data types is not implemented on DEVICE_ROCM");
    }
};
REGISTER_ROCM_ACC(RocmCastLayerAcc, LAYER_CAST);

}  // namespace TNN_NS
