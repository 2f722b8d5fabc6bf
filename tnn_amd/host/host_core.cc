// Device-independent host: status/utilities, registries, model interpreter, layers with shape
// inference, optimizer manager, network and instance.  Mirrors the behaviour of the engine files
// cited next to each part; nothing here touches the GPU except through AbstractDevice / Context /
// AbstractLayerAcc / BlobConverterAcc.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <sstream>

#include "tnn_host.h"
#include "tnn_rocm.h"

namespace TNN_NS {

// ---- Status / utils (include/tnn/core/status.h, source/tnn/utils/dims_vector_utils.cc) ----------
std::string Status::description() const {
    char buf[64];
    snprintf(buf, sizeof(buf), "code: 0x%X msg: ", code_);
    return std::string(buf) + (message_.empty() ? (code_ == TNN_OK ? "OK" : "error") : message_);
}

int DimsVectorUtils::Count(const DimsVector &dims, int start, int end) {
    if (end < 0 || end > (int)dims.size())
        end = (int)dims.size();
    if (start < 0)
        start = 0;
    long r = 1;
    for (int i = start; i < end; ++i)
        r *= dims[i];
    return (int)r;
}
bool DimsVectorUtils::Equal(const DimsVector &a, const DimsVector &b) { return a == b; }

int DataTypeUtils::GetBytesSize(DataType dt) {
    switch (dt) {
        case DATA_TYPE_FLOAT: return 4;
        case DATA_TYPE_HALF: return 2;
        case DATA_TYPE_BFP16: return 2;
        case DATA_TYPE_INT8: return 1;
        case DATA_TYPE_INT32: return 4;
        case DATA_TYPE_INT64: return 8;
        case DATA_TYPE_UINT32: return 4;
        default: return 0;
    }
}

// the engine's rule (memory_manager/blob_memory_size_info.cc:21-36): linear memory is one dimension, two dimensions
// are a four-channel image, anything else has no size
int64_t GetBlobMemoryBytesSize(BlobMemorySizeInfo &info) {
    if (info.dims.size() == 1)
        return (int64_t)info.dims[0] * DataTypeUtils::GetBytesSize(info.data_type);
    if (info.dims.size() == 2)
        return (int64_t)info.dims[0] * info.dims[1] * 4 * DataTypeUtils::GetBytesSize(info.data_type);
    return 0;
}

// ---- registries (source/tnn/core/abstract_device.cc:51-64, layer_type.cc:24-270) ----------------
std::map<DeviceType, std::shared_ptr<AbstractDevice>> &GetGlobalDeviceMap() {
    static std::map<DeviceType, std::shared_ptr<AbstractDevice>> m;
    return m;
}
AbstractDevice *GetDevice(DeviceType type) {
    auto &m = GetGlobalDeviceMap();
    auto it = m.find(type);
    return it == m.end() ? nullptr : it->second.get();
}
Status AbstractDevice::Allocate(BlobHandle *handle, BlobMemorySizeInfo &size_info) {
    void *data = nullptr;
    Status st  = Allocate(&data, size_info);
    if (st == TNN_OK) {
        handle->base         = data;
        handle->bytes_offset = 0;
    }
    return st;
}
std::shared_ptr<const ImplementedPrecision> AbstractDevice::GetImplementedPrecision(LayerType) {
    auto p              = std::make_shared<ImplementedPrecision>();
    p->fp32_implemented = true;
    return p;
}
Status AbstractLayerAcc::ResolveBlobDataFormat(Blob *blob, BlobType blob_type) {
    auto &desc   = blob->GetBlobDesc();
    auto formats = SupportDataFormat(desc.data_type, (int)desc.dims.size(), blob_type);
    if (formats.empty())
        return Status(TNNERR_DEVICE_ACC_DATA_FORMAT_NOT_SUPPORT, "unsupported data format for device acc");
    if (desc.data_format == DATA_FORMAT_AUTO)
        desc.data_format = formats[0];
    else if (std::find(formats.begin(), formats.end(), desc.data_format) == formats.end())
        return Status(TNNERR_DEVICE_ACC_DATA_FORMAT_NOT_SUPPORT, "unsupported data format for device acc");
    return TNN_OK;
}

LayerType GlobalConvertLayerType(std::string s) {
    static const std::map<std::string, LayerType> m = {
        {"InnerProduct", LAYER_INNER_PRODUCT}, {"QuantizedInnerProduct", LAYER_INNER_PRODUCT},
        {"Softmax", LAYER_SOFTMAX},           {"SoftmaxCaffe", LAYER_SOFTMAX},
        {"Add", LAYER_ADD},                   {"Sub", LAYER_SUB},
        {"Mul", LAYER_MUL},                   {"Div", LAYER_DIV},
        {"Reshape", LAYER_RESHAPE},           {"Permute", LAYER_PERMUTE},
        {"Cast", LAYER_CAST},                 {"Reformat", LAYER_REFORMAT},
        {"Squeeze", LAYER_SQUEEZE},           {"Unsqueeze", LAYER_UNSQUEEZE},
        {"Tanh", LAYER_TANH},
        {"Gather", LAYER_GATHER},             {"MatMul", LAYER_MATMUL},
        {"LayerNorm", LAYER_LAYER_NORM},      {"GELU", LAYER_GELU},
        {"BlobScale", LAYER_BLOB_SCALE},      {"QuantizedAdd", LAYER_ADD},
        // weight-only int8 ("dynamic range quantisation", layer_type.cc:261-265): the layer computes in float
        {"DynamicRangeQuantizedMatMul", LAYER_MATMUL}, {"DynamicRangeQuantizedInnerProduct", LAYER_INNER_PRODUCT},
        {"DynamicRangeQuantizedGather", LAYER_GATHER},
        {"RocmFusedLinear", LAYER_ROCM_FUSED_LINEAR}, {"RocmFusedAttention", LAYER_ROCM_FUSED_ATTENTION},
        {"RocmFusedLinearInt8", LAYER_ROCM_FUSED_LINEAR_INT8}, {"RocmGeluInt8", LAYER_ROCM_GELU_INT8},
        {"RocmLayerNormQuant", LAYER_ROCM_LAYER_NORM_QUANT},
        {"RocmFusedEmbedding", LAYER_ROCM_FUSED_EMBEDDING}, {"RocmQuantLinearGelu", LAYER_ROCM_QUANT_LINEAR_GELU},
    };
    auto it = m.find(s);
    return it == m.end() ? LAYER_NOT_SUPPORT : it->second;
}

// ---- Mat / BlobConverter (source/tnn/core/mat.cc:70-87, utils/blob_converter_internal.cc:39-135) --
Mat::Mat(DeviceType device_type, MatType mat_type, DimsVector dims)
    : device_type_(device_type), mat_type_(mat_type), dims_(std::move(dims)) {
    size_t es = (mat_type == NCHW_FLOAT || mat_type == NC_INT32) ? 4 : ((mat_type == RESERVED_FP16_TEST || mat_type == RESERVED_BFP16_TEST) ? 2 : 1);
    size_t n  = (size_t)DimsVectorUtils::Count(dims_) * es;
    if (device_type != DEVICE_NAIVE) {  // memory of the Mat's own device, returned to it with the last owner (mat.cc:70-87)
        AbstractDevice *device = GetDevice(device_type);
        void *p                = nullptr;
        if (device && device->Allocate(&p, mat_type, dims_) == TNN_OK && p) {
            owned_ = std::shared_ptr<char>((char *)p, [device](char *q) { device->Free(q); });
            data_  = p;
        }
        return;
    }
    owned_    = std::shared_ptr<char>(new char[n > 0 ? n : 1](), std::default_delete<char[]>());
    data_     = owned_.get();
}
std::shared_ptr<BlobConverterManager> &BlobConverterManager::Shared() {
    static std::shared_ptr<BlobConverterManager> m = std::make_shared<BlobConverterManager>();
    return m;
}
int BlobConverterManager::RegisterBlobConverterAccCreater(DeviceType type, std::shared_ptr<BlobConverterAccCreater> creater) {
    converter_creater_map_[type] = creater;
    return 0;
}
std::shared_ptr<BlobConverterAcc> BlobConverterManager::CreateBlobConverterAcc(Blob *blob) {
    auto it = converter_creater_map_.find(blob->GetBlobDesc().device_type);
    return it == converter_creater_map_.end() ? nullptr : it->second->CreateBlobConverterAcc(blob);
}
BlobConverter::BlobConverter(Blob *blob) { impl_ = BlobConverterManager::Shared()->CreateBlobConverterAcc(blob); }
Status BlobConverter::ConvertToMat(Mat &image, MatConvertParam param, void *q) {
    if (!impl_)
        return Status(TNNERR_INIT_LAYER, "blob converter is nil, check device type");
    return impl_->ConvertToMat(image, param, q);
}
Status BlobConverter::ConvertFromMat(Mat &image, MatConvertParam param, void *q) {
    if (!impl_)
        return Status(TNNERR_INIT_LAYER, "blob converter is nil, check device type");
    return impl_->ConvertFromMat(image, param, q);
}
Status BlobConverter::ConvertToMatAsync(Mat &image, MatConvertParam param, void *q) {
    if (!impl_)
        return Status(TNNERR_INIT_LAYER, "blob converter is nil, check device type");
    return impl_->ConvertToMatAsync(image, param, q);
}
Status BlobConverter::ConvertFromMatAsync(Mat &image, MatConvertParam param, void *q) {
    if (!impl_)
        return Status(TNNERR_INIT_LAYER, "blob converter is nil, check device type");
    return impl_->ConvertFromMatAsync(image, param, q);
}

std::shared_ptr<MatConverterManager> &MatConverterManager::Shared() {
    static std::shared_ptr<MatConverterManager> m = std::make_shared<MatConverterManager>();
    return m;
}
int MatConverterManager::RegisterMatConverterAccCreater(DeviceType type, std::shared_ptr<MatConverterAccCreater> creater) {
    converter_creater_map_[type] = creater;
    return 0;
}
std::shared_ptr<MatConverterAcc> MatConverterManager::CreateMatConverterAcc(DeviceType device_type) {
    auto it = converter_creater_map_.find(device_type);
    return it == converter_creater_map_.end() ? nullptr : it->second->CreateMatConverterAcc();
}
Status MatUtils::Copy(Mat &src, Mat &dst, void *command_queue) {  // mat_utils.cc:73-100
    if (src.GetMatType() != dst.GetMatType())
        return Status(TNNERR_PARAM_ERR, "src and dst have different mat types");
    if (!DimsVectorUtils::Equal(src.GetDims(), dst.GetDims()))
        return Status(TNNERR_PARAM_ERR, "src and dst dims not equal");
    const DeviceType s = src.GetDeviceType(), d = dst.GetDeviceType();
    DeviceType where;
    if (s == d)
        where = s;
    else if (s == DEVICE_NAIVE || s == DEVICE_ARM)
        where = d;
    else if (d == DEVICE_NAIVE || d == DEVICE_ARM)
        where = s;
    else
        return Status(TNNERR_PARAM_ERR, "src and dst DeviceType need be equal or one is device cpu");
    if (dst.GetData() == nullptr)
        dst = Mat(dst.GetDeviceType(), dst.GetMatType(), dst.GetDims());
    auto converter = MatConverterManager::Shared()->CreateMatConverterAcc(where);
    if (!converter)
        return Status(TNNERR_INIT_LAYER, "image converter is nil, check device type");
    return converter->Copy(src, dst, command_queue);
}

// ---- model interpreter (source/tnn/interpreter/tnn/model_interpreter.cc:174-476) ----------------
namespace {
const uint32_t kMagicV1 = 0x0FABC0002, kMagicV2 = 0x0FABC0004;

std::vector<std::string> split(const std::string &s, char sep, bool keep_empty = false) {
    std::vector<std::string> out;
    std::string cur;
    for (char c : s) {
        if (c == sep) {
            if (keep_empty || !cur.empty())
                out.push_back(cur);
            cur.clear();
        } else {
            cur.push_back(c);
        }
    }
    if (keep_empty || !cur.empty())
        out.push_back(cur);
    return out;
}
std::string trim(const std::string &s) {
    size_t a = s.find_first_not_of(" \t\r"), b = s.find_last_not_of(" \t\r");
    return a == std::string::npos ? "" : s.substr(a, b - a + 1);
}

struct ArgReader {
    const std::vector<std::string> &a;
    size_t i;
    bool has() const { return i < a.size(); }
    size_t left() const { return i < a.size() ? a.size() - i : 0; }
    int geti(int def) { return has() ? atoi(a[i++].c_str()) : def; }
    float getf(float def) { return has() ? (float)atof(a[i++].c_str()) : def; }
};

Status ParseLayerParam(LayerType type, const std::vector<std::string> &cfg, size_t start,
                       std::shared_ptr<LayerParam> &out) {
    ArgReader r{cfg, start};
    switch (type) {
        case LAYER_INNER_PRODUCT: {  // inner_product_layer_interpreter.cc:23-34
            auto p        = std::make_shared<InnerProductLayerParam>();
            p->num_output = r.geti(0);
            p->has_bias   = r.geti(0);
            p->transpose  = r.geti(0);
            p->axis       = r.geti(0);
            out           = p;
            break;
        }
        case LAYER_MATMUL: {  // mat_mul_layer_interpreter.cc:23-30
            auto p             = std::make_shared<MatMulLayerParam>();
            p->weight_position = r.geti(-1);
            out                = p;
            break;
        }
        case LAYER_ADD:
        case LAYER_SUB:
        case LAYER_MUL:
        case LAYER_DIV: {  // add_layer_interpreter.cc:22-26
            auto p                = std::make_shared<MultidirBroadcastLayerParam>();
            p->weight_input_index = r.geti(1);
            out                   = p;
            break;
        }
        case LAYER_SOFTMAX: {
            auto p  = std::make_shared<SoftmaxLayerParam>();
            p->axis = r.geti(1);
            out     = p;
            break;
        }
        case LAYER_LAYER_NORM: {  // layer_norm_layer_interpreter.cc:21-26
            auto p              = std::make_shared<LayerNormLayerParam>();
            p->reduce_dims_size = r.geti(0);
            p->eps              = r.getf(1e-5f);
            out                 = p;
            break;
        }
        case LAYER_RESHAPE: {  // reshape_layer_interpreter.cc:23-41
            auto p      = std::make_shared<ReshapeLayerParam>();
            p->axis     = r.geti(0);
            p->num_axes = r.geti(0);
            int n       = r.geti(-1);
            if (n < 0 || (size_t)n > r.left())
                return Status(TNNERR_PARAM_ERR, "ReshapeLayerInterpreter: invalid layer param");
            for (int i = 0; i < n; ++i)
                p->shape.push_back(r.geti(0));
            p->reshape_type = r.geti(0);
            out             = p;
            break;
        }
        case LAYER_PERMUTE: {
            auto p = std::make_shared<PermuteLayerParam>();
            int n  = r.geti(0);
            if (n < 0 || (size_t)n > r.left())
                return Status(TNNERR_PARAM_ERR, "PermuteLayerInterpreter: fewer orders than the count in front of them");
            for (int i = 0; i < n; ++i)
                p->orders.push_back(r.geti(0));
            out = p;
            break;
        }
        case LAYER_GATHER: {  // gather_layer_interpreter.cc:22-28
            auto p                 = std::make_shared<GatherLayerParam>();
            p->axis                = r.geti(0);
            p->data_in_resource    = r.geti(0) != 0;
            p->indices_in_resource = r.geti(1) != 0;
            out                    = p;
            break;
        }
        case LAYER_SQUEEZE:
        case LAYER_UNSQUEEZE: {  // unsqueeze_layer_interpreter.cc:22-32: count, then the axes
            auto p = std::make_shared<SqueezeLayerParam>();
            int n  = r.geti(0);
            if (n < 0 || (size_t)n > r.left())
                return Status(TNNERR_PARAM_ERR, "SqueezeLayerInterpreter: fewer axes than the count in front of them");
            for (int i = 0; i < n; ++i)
                p->axes.push_back(r.geti(0));
            out = p;
            break;
        }
        case LAYER_CAST: {
            auto p = std::make_shared<CastLayerParam>();
            p->to  = r.geti(0);
            out    = p;
            break;
        }
        default: out = std::make_shared<LayerParam>(); break;
    }
    return TNN_OK;
}

class Deserializer {  // objseri.h:104-205
public:
    explicit Deserializer(const std::string &s) : s_(s) {}
    bool eof() const { return pos_ >= s_.size(); }
    size_t remaining() const { return pos_ >= s_.size() ? 0 : s_.size() - pos_; }
    void rewind(size_t n) { pos_ -= n; }
    int GetInt() {
        int v = 0;
        if (pos_ + 4 <= s_.size()) {
            memcpy(&v, s_.data() + pos_, 4);
        } else {
            bad_ = true;
        }
        pos_ += 4;
        return v;
    }
    std::string GetString() {
        int len = GetInt();
        if (len < 0 || pos_ + (size_t)len > s_.size()) {
            bad_ = true;
            return "";
        }
        std::string r = s_.substr(pos_, len);
        pos_ += len;
        return r;
    }
    void GetRaw(RawBuffer &value) {
        uint32_t magic = (uint32_t)GetInt();
        int dt_v       = GetInt();
        int length     = GetInt();
        if (dt_v < (int)DATA_TYPE_FLOAT || dt_v > (int)DATA_TYPE_UINT32)
            bad_ = true;  // no element type of the format (include/tnn/core/common.h:55-64)
        if (length <= 0 || bad_)
            return;
        DataType dt = (DataType)dt_v;
        DimsVector dims;
        if (magic == kMagicV2) {
            int n = GetInt();
            if (n < 0 || n > 16) {
                bad_ = true;
                return;
            }
            for (int i = 0; i < n; ++i)
                dims.push_back(GetInt());
        }
        if (pos_ + (size_t)length > s_.size()) {
            bad_ = true;
            return;
        }
        value = RawBuffer(length);
        value.SetDataType(dt);
        value.SetBufferDims(dims);
        memcpy(value.force_to<char *>(), s_.data() + pos_, length);
        pos_ += length;
    }
    bool bad() const { return bad_; }

private:
    const std::string &s_;
    size_t pos_ = 0;
    bool bad_   = false;
};

void ReadIntScaleTail(Deserializer &d, RawBuffer &zero_point, RawBuffer &scale) {
    // first buffer int8 => new layout (zero points then scale); float => old layout (scale only)
    RawBuffer first;
    d.GetRaw(first);
    if (first.GetDataType() == DATA_TYPE_INT8) {
        zero_point = first;
        d.GetRaw(scale);
    } else {
        scale      = first;
        zero_point = RawBuffer(first.GetDataCount());
        zero_point.SetDataType(DATA_TYPE_INT8);
    }
}
}  // namespace

Status ModelInterpreter::Interpret(std::vector<std::string> &params) {
    static const std::string empty;
    RETURN_ON_NEQ(InterpretProto(params.size() > 0 ? params[0] : empty), TNN_OK);
    return InterpretModel(params.size() > 1 ? params[1] : empty);
}

Status ModelInterpreter::InterpretProto(const std::string &content) {
    std::string buf;
    for (char c : content)
        if (c != '"' && c != '\n')
            buf.push_back(c);
    if (buf.empty())
        return Status(TNNERR_INVALID_NETCFG, "proto content is empty");
    auto lines = split(buf, ',', false);
    std::vector<std::string> cfg;
    for (auto &l : lines) {
        std::string t = trim(l);
        if (!t.empty())
            cfg.push_back(t);
    }
    if (cfg.size() <= 5)
        return Status(TNNERR_INVALID_NETCFG, "content line <= 5");
    auto l0 = split(cfg[0], ' ');
    if (l0.size() >= 4)
        version_magic_number_ = (uint32_t)atoll(l0[3].c_str());
    // inputs
    for (auto &one : split(cfg[1], ':')) {
        auto f = split(trim(one), ' ');
        if (f.size() < 2)
            return Status(TNNERR_INVALID_NETCFG, "split input line error");
        DimsVector &shape = structure_.inputs_shape_map[f[0]];
        if (version_magic_number_ == kMagicV1) {
            for (size_t i = 1; i < f.size(); ++i)
                shape.push_back(atoi(f[i].c_str()));
        } else if (version_magic_number_ == kMagicV2) {
            int n = atoi(f[1].c_str());
            if (n < 0 || n > 16 || (int)f.size() < n + 2)
                return Status(TNNERR_INVALID_NETCFG, "get input dims error");
            for (int i = 2; i < n + 2; ++i)
                shape.push_back(atoi(f[i].c_str()));
            const int dt = atoi(f.back().c_str());
            if (dt < (int)DATA_TYPE_FLOAT || dt > (int)DATA_TYPE_UINT32)
                return Status(TNNERR_INVALID_NETCFG, "input " + f[0] + " has no data type of the format");
            structure_.input_data_type_map[f[0]] = (DataType)dt;
        } else {
            return Status(TNNERR_INVALID_MODEL, "Do not support tnn proto type");
        }
        structure_.blobs.insert(f[0]);
    }
    for (auto &o : split(cfg[3], ' '))
        structure_.outputs.insert(o);
    if (structure_.outputs.empty())
        return Status(TNNERR_INVALID_NETCFG, "split output line error");
    for (size_t li = 5; li < cfg.size(); ++li) {
        auto f = split(cfg[li], ' ');
        if (f.size() < 4)
            return Status(TNNERR_INVALID_NETCFG, "split layer info error");
        auto layer      = std::make_shared<LayerInfo>();
        layer->type_str = f[0];
        layer->type     = GlobalConvertLayerType(f[0]);
        if (layer->type == LAYER_NOT_SUPPORT)
            return Status(TNNERR_PARAM_ERR, "layer type is not supported: " + f[0]);
        layer->name  = f[1];
        int n_in     = atoi(f[2].c_str());
        int n_out    = atoi(f[3].c_str());
        size_t idx   = 4;
        if (n_in < 0 || n_out < 0 || idx + n_in + n_out > f.size())
            return Status(TNNERR_INVALID_NETCFG, "layer blob counts exceed the line: " + layer->name);
        for (int i = 0; i < n_in; ++i, ++idx) {
            layer->inputs.push_back(f[idx]);
            structure_.blobs.insert(f[idx]);
        }
        for (int i = 0; i < n_out; ++i, ++idx) {
            layer->outputs.push_back(f[idx]);
            structure_.blobs.insert(f[idx]);
        }
        RETURN_ON_NEQ(ParseLayerParam(layer->type, f, idx, layer->param), TNN_OK);
        if (layer->type_str.compare(0, 9, "Quantized") == 0)
            layer->param->quantized = true;  // model_interpreter.cc:371-373
        if (layer->type_str.compare(0, 21, "DynamicRangeQuantized") == 0)
            layer->param->dynamic_range_quantized = true;  // model_interpreter.cc:375-378
        layer->param->type = layer->type_str;
        layer->param->name = layer->name;
        structure_.layers.push_back(layer);
    }
    return TNN_OK;
}

Status ModelInterpreter::InterpretModel(const std::string &content) {
    if (content.empty())
        return Status(TNNERR_LOAD_MODEL, "model content is invalid");
    Deserializer d(content);
    uint32_t magic = (uint32_t)d.GetInt();
    if (magic != kMagicV1 && magic != kMagicV2)
        d.rewind(4);
    int layer_cnt = d.GetInt() & 0x1FFFFFFF;
    if (layer_cnt < 0 || layer_cnt >= 10000)
        return Status(TNNERR_INVALID_MODEL, "Error: model is illegal");
    for (int i = 0; i < layer_cnt; ++i) {
        int type_v           = d.GetInt();
        std::string type_str = d.GetString();
        LayerType type       = GlobalConvertLayerType(type_str);
        if (type_v < 0 || type_v > 10000 || type == LAYER_NOT_SUPPORT || d.bad())
            return Status(TNNERR_LOAD_MODEL, "Error: layer_interpreter is nil for resource type " + type_str);
        std::string name = d.GetString();
        std::shared_ptr<LayerResource> res;
        switch (type) {
            case LAYER_INNER_PRODUCT: {  // inner_product_layer_interpreter.cc:36-70
                auto r = std::make_shared<InnerProductLayerResource>();
                d.GetString();
                d.GetRaw(r->weight_handle);
                d.GetRaw(r->bias_handle);
                if (r->weight_handle.GetDataType() == DATA_TYPE_INT8)
                    ReadIntScaleTail(d, r->zero_point_handle, r->scale_handle);
                res = r;
                break;
            }
            case LAYER_MATMUL: {
                auto r = std::make_shared<MatMulLayerResource>();
                d.GetRaw(r->weight);
                if (r->weight.GetDataType() == DATA_TYPE_INT8)
                    d.GetRaw(r->scale_handle);
                res = r;
                break;
            }
            case LAYER_ADD:
            case LAYER_SUB:
            case LAYER_MUL:
            case LAYER_DIV: {
                auto r = std::make_shared<EltwiseLayerResource>();
                d.GetRaw(r->element_handle);
                r->element_shape = r->element_handle.GetBufferDims();
                res              = r;
                break;
            }
            case LAYER_GATHER: {  // gather_layer_interpreter.cc:30-45
                auto r = std::make_shared<GatherLayerResource>();
                if (d.GetInt() == 1)
                    d.GetRaw(r->data);
                if (d.GetInt() == 1)
                    d.GetRaw(r->indices);
                if (r->data.GetDataType() == DATA_TYPE_INT8 && r->data.GetBytesSize() > 0)
                    d.GetRaw(r->scale_data);
                res = r;
                break;
            }
            case LAYER_BLOB_SCALE: {  // blob_scale_layer_interpreter.cc:25-51
                auto r = std::make_shared<IntScaleResource>();
                ReadIntScaleTail(d, r->zero_point_handle, r->scale_handle);
                d.GetRaw(r->bias_handle);
                res = r;
                break;
            }
            default: return Status(TNNERR_LOAD_MODEL, "resource of layer type " + type_str + " is not readable");
        }
        if (d.bad())
            return Status(TNNERR_INVALID_MODEL, "Error: model is truncated at resource " + name);
        res->name                   = name;
        resource_.resource_map[name] = res;
    }
    if (d.remaining() >= 8) {
        d.GetInt();  // magic
        int n = d.GetInt();
        for (int i = 0; i < n && !d.bad(); ++i) {
            std::string key = d.GetString();
            auto buf        = std::make_shared<RawBuffer>();
            d.GetRaw(*buf);
            resource_.constant_map[key] = buf;
        }
        if (d.bad())
            return Status(TNNERR_INVALID_MODEL, "Error: constant map is truncated");
    }
    return TNN_OK;
}

// ---- layers: shape inference (source/tnn/layer/*.cc) ---------------------------------------------
BaseLayer::~BaseLayer() { delete layer_acc_; }

Status BaseLayer::Init(Context *context, LayerParam *param, LayerResource *resource, std::vector<Blob *> &inputs,
                       std::vector<Blob *> &outputs, AbstractDevice *device, ConstantResource *consts) {
    input_blobs_  = inputs;
    output_blobs_ = outputs;
    param_        = param;
    resource_     = resource;
    if (output_blobs_.empty())
        return Status(TNNERR_INVALID_MODEL, "layer " + param_->name + " has no output blob");
    if (input_blobs_.empty() && type_ != LAYER_GATHER)  // a Gather may hold both operands as resources
        return Status(TNNERR_INVALID_MODEL, "layer " + param_->name + " has no input blob");
    RETURN_ON_NEQ(InferOutputDataType(), TNN_OK);
    RETURN_ON_NEQ(InferOutputShape(), TNN_OK);
    for (auto b : output_blobs_)
        if (DimsVectorUtils::Count(b->GetBlobDesc().dims) < 0)
            return Status(TNNERR_LAYER_ERR, "layer " + param_->name + " produced a negative dimension");
    layer_acc_ = device->CreateLayerAcc(type_);
    if (layer_acc_ == nullptr)  // base_layer.cc:83-86
        return Status(TNNERR_LAYER_ERR, "layer acc is nil (type " + param_->type + ")");
    if (context == nullptr) {  // planning only (no device context): the acc exists, nothing is uploaded
        delete layer_acc_;
        layer_acc_ = nullptr;
        return TNN_OK;
    }
    layer_acc_->SetConstantResource(consts);
    for (auto b : input_blobs_)
        RETURN_ON_NEQ(layer_acc_->ResolveBlobDataFormat(b, BLOB_INPUT), TNN_OK);
    for (auto b : output_blobs_)
        RETURN_ON_NEQ(layer_acc_->ResolveBlobDataFormat(b, BLOB_OUTPUT), TNN_OK);
    return layer_acc_->Init(context, param_, resource_, input_blobs_, output_blobs_);
}
Status BaseLayer::Reshape() {  // base_layer.cc:167-188
    RETURN_ON_NEQ(InferOutputShape(), TNN_OK);
    for (auto b : output_blobs_)
        for (int d : b->GetBlobDesc().dims)
            if (d < 0)
                return Status(TNNERR_LAYER_ERR, "layer output dims is invalid");
    if (layer_acc_ == nullptr)
        return Status(TNNERR_LAYER_ERR, "layer acc is nil");
    RETURN_ON_NEQ(layer_acc_->ReloadConstantBlobs(input_blobs_, true), TNN_OK);
    return layer_acc_->Reshape(input_blobs_, output_blobs_);
}
Status BaseLayer::Forward() {  // base_layer.cc:190-225
    RETURN_ON_NEQ(layer_acc_->BeforeForward(input_blobs_, output_blobs_), TNN_OK);
    RETURN_ON_NEQ(layer_acc_->Forward(input_blobs_, output_blobs_), TNN_OK);
    return layer_acc_->AfterForward(input_blobs_, output_blobs_);
}
Status BaseLayer::InferOutputDataType() {
    if (input_blobs_.empty())
        return TNN_OK;
    DataType dt = input_blobs_[0]->GetBlobDesc().data_type;
    for (auto b : output_blobs_)
        if (!dynamic_cast<BlobInt8 *>(b) || dt == DATA_TYPE_INT8)
            b->GetBlobDesc().data_type = dt;
    return TNN_OK;
}
Status BaseLayer::InferOutputShape(bool) {
    if (!input_blobs_.empty())
        for (auto b : output_blobs_)
            b->GetBlobDesc().dims = input_blobs_[0]->GetBlobDesc().dims;
    return TNN_OK;
}

namespace {
struct InnerProductLayer : BaseLayer {  // layer/inner_product_layer.cc:27-46
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        auto p = dynamic_cast<InnerProductLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        auto in = input_blobs_[0]->GetBlobDesc().dims;
        if (p->axis < 0 || p->axis > (int)in.size())
            return Status(TNNERR_PARAM_ERR, "InnerProduct axis out of range");
        DimsVector out(in.begin(), in.begin() + p->axis);
        out.push_back(p->num_output);
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

DimsVector MatMulOutputDims(DimsVector a, DimsVector b, Status *st) {  // layer/mat_mul_layer.cc:42-114
    bool sq_a = false, sq_b = false;
    if (a.size() == 1) {
        a.insert(a.begin(), 1);
        sq_a = true;
    }
    if (b.size() == 1) {
        b.push_back(1);
        sq_b = true;
    }
    DimsVector out;
    auto fail = [&]() {
        *st = Status(TNNERR_PARAM_ERR, "MatMul has wrong shape of matrix_a or matrix_b");
        return DimsVector();
    };
    if (a.size() < 2 || b.size() < 2)
        return fail();
    if (a.back() != b[b.size() - 2])
        return fail();
    if (a.size() == 2 && b.size() == 2) {
        out = {a[0], b[1]};
    } else if (a.size() == 2) {
        out                = b;
        out[b.size() - 2]  = a[0];
    } else if (b.size() == 2) {
        out        = a;
        out.back() = b.back();
    } else {
        out                   = a.size() >= b.size() ? a : b;
        out[out.size() - 2]   = a[a.size() - 2];
        out[out.size() - 1]   = b.back();
        size_t n              = std::min(a.size(), b.size());
        for (size_t i = 0; i + 2 < n; ++i) {
            int da = a[a.size() - 3 - i], db = b[b.size() - 3 - i];
            if (da != 1 && db != 1 && da != db)
                return fail();
            out[out.size() - 3 - i] = std::max(da, db);
        }
    }
    if (sq_a && out[out.size() - a.size()] == 1)
        out.erase(out.end() - a.size());
    if (sq_b && out.back() == 1)
        out.pop_back();
    return out;
}
struct MatMulLayer : BaseLayer {  // layer/mat_mul_layer.cc:116-148
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        auto p = dynamic_cast<MatMulLayerParam *>(param_);
        auto r = dynamic_cast<MatMulLayerResource *>(resource_);
        CHECK_PARAM_NULL(p);
        DimsVector a, b;
        if (input_blobs_.size() == 1) {
            if (!r)
                return Status(TNNERR_INVALID_MODEL, "MatMul with one input needs a weight resource");
            if (p->weight_position == 0) {
                a = r->weight.GetBufferDims();
                b = input_blobs_[0]->GetBlobDesc().dims;
            } else if (p->weight_position == 1) {
                a = input_blobs_[0]->GetBlobDesc().dims;
                b = r->weight.GetBufferDims();
            } else {
                return Status(TNNERR_INVALID_MODEL, "MatMul input size is error");
            }
        } else if (input_blobs_.size() == 2) {
            a = input_blobs_[0]->GetBlobDesc().dims;
            b = input_blobs_[1]->GetBlobDesc().dims;
        } else {
            return Status(TNNERR_INVALID_MODEL, "MatMul input size is error");
        }
        p->matrix_a_dims = a;
        p->matrix_b_dims = b;
        Status st        = TNN_OK;
        auto out         = MatMulOutputDims(a, b, &st);
        output_blobs_[0]->GetBlobDesc().dims = out;
        return st;
    }
};

struct BinaryLayer : BaseLayer {  // layer/multidir_broadcast_layer.cc:100-190
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        std::vector<DimsVector> shapes;
        for (auto b : input_blobs_)
            shapes.push_back(b->GetBlobDesc().dims);
        if (auto r = dynamic_cast<EltwiseLayerResource *>(resource_)) {
            DimsVector w = r->element_handle.GetBufferDims();
            if (w.empty()) {
                // weights without dims: single element, per-channel (dims[1]) or element-wise
                auto in = shapes.empty() ? DimsVector() : shapes[0];
                int n   = r->element_handle.GetDataCount();
                w       = DimsVector(in.size(), 1);
                if (in.size() > 1 && (n == 1 || n == in[1]))
                    w[1] = n;
                else if (n == DimsVectorUtils::Count(in, 1))
                    for (size_t i = 1; i < in.size(); ++i)
                        w[i] = in[i];
                else if (n != 1)
                    return Status(TNNERR_LAYER_ERR, "Error: unsupported broadcast type");
            }
            r->element_shape = w;
            shapes.push_back(w);
        }
        if (shapes.empty())
            return Status(TNNERR_LAYER_ERR, "binary layer without operands");
        size_t rank = 0;
        for (auto &s : shapes)
            rank = std::max(rank, s.size());
        DimsVector out(rank, 1);
        for (auto s : shapes) {
            s.insert(s.begin(), rank - s.size(), 1);
            for (size_t i = 0; i < rank; ++i) {
                if (s[i] != 1 && out[i] != 1 && s[i] != out[i])
                    return Status(TNNERR_LAYER_ERR, "Error: operands could not be broadcast together");
                out[i] = std::max(out[i], s[i]);
            }
        }
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

struct ReshapeLayer : BaseLayer {  // layer/reshape_layer.cc:41-63, utils/dims_function_utils.cc:105-157
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        auto p = dynamic_cast<ReshapeLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        auto in = input_blobs_[0]->GetBlobDesc().dims;
        if (p->axis < 0 || p->axis > (int)in.size() || p->num_axes > (int)p->shape.size())
            return Status(TNNERR_PARAM_ERR, "reshape param size error");
        DimsVector out(p->shape.size() + p->axis, 1);
        for (int i = 0; i < p->axis; ++i)
            out[i] = in[i];
        int infer_pos = -1, infer_cnt = 0;
        for (int i = p->axis, j = 0; j < p->num_axes; ++i, ++j) {
            if (p->shape[j] == -1) {
                ++infer_cnt;
                infer_pos = i;
                out[i]    = 1;
            } else if (p->shape[j] == 0) {
                if (i >= (int)in.size())
                    return Status(TNNERR_PARAM_ERR, "reshape copies a dimension the input does not have");
                out[i] = in[i];
            } else {
                out[i] = p->shape[j];
            }
        }
        if (infer_cnt > 1)
            return Status(TNNERR_PARAM_ERR, "reshape param size error");
        if (infer_cnt == 1) {
            int oc = DimsVectorUtils::Count(out);
            if (oc == 0)
                return Status(TNNERR_COMMON_ERROR, "Error: blob count is zero");
            out[infer_pos] = DimsVectorUtils::Count(in) / oc;
        }
        if (DimsVectorUtils::Count(out) != DimsVectorUtils::Count(in))
            return Status(TNNERR_PARAM_ERR, "reshape changes the element count");
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

struct PermuteLayer : BaseLayer {  // layer/permute_layer.cc:38-60
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        auto p = dynamic_cast<PermuteLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        auto in = input_blobs_[0]->GetBlobDesc().dims;
        // complete missing axes in order
        for (int i = 0; i < (int)in.size(); ++i)
            if (std::find(p->orders.begin(), p->orders.end(), i) == p->orders.end())
                p->orders.push_back(i);
        if (p->orders.size() != in.size())
            return Status(TNNERR_PARAM_ERR, "Permute param got wrong size");
        DimsVector out;
        for (int o : p->orders) {
            if (o < 0 || o >= (int)in.size())
                return Status(TNNERR_PARAM_ERR, "Permute param out of range");
            out.push_back(in[o]);
        }
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

struct LayerNormLayer : BaseLayer {  // layer/layer_norm_layer.cc:25-35
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        if (input_blobs_.size() < 3)
            return Status(TNNERR_PARAM_ERR, "LayerNormLayer has no input blob of scale or bias");
        return BaseLayer::InferOutputShape(ignore_error);
    }
};

struct GatherLayer : BaseLayer {  // layer/gather_layer.cc
    using BaseLayer::BaseLayer;
    Status InferOutputDataType() override {
        auto p = dynamic_cast<GatherLayerParam *>(param_);
        auto r = dynamic_cast<GatherLayerResource *>(resource_);
        CHECK_PARAM_NULL(p);
        DataType dt = DATA_TYPE_FLOAT;
        if (p->data_in_resource) {
            if (!r)
                return Status(TNNERR_MODEL_ERR, "Gather resource is invalid");
            dt = r->data.GetDataType();
        } else {
            if (input_blobs_.empty())
                return Status(TNNERR_INVALID_MODEL, "Gather without a data blob");
            dt = input_blobs_[0]->GetBlobDesc().data_type;
        }
        output_blobs_[0]->GetBlobDesc().data_type = dt;
        return TNN_OK;
    }
    Status InferOutputShape(bool ignore_error = false) override {
        auto p = dynamic_cast<GatherLayerParam *>(param_);
        auto r = dynamic_cast<GatherLayerResource *>(resource_);
        CHECK_PARAM_NULL(p);
        if ((p->data_in_resource || p->indices_in_resource) && !r)
            return Status(TNNERR_MODEL_ERR, "Gather resource is invalid");
        if (input_blobs_.size() < (size_t)(!p->data_in_resource) + (size_t)(!p->indices_in_resource))
            return Status(TNNERR_INVALID_MODEL, "Gather with fewer input blobs than operands outside its resource");
        DimsVector data = p->data_in_resource ? r->data.GetBufferDims() : input_blobs_.front()->GetBlobDesc().dims;
        DimsVector idx  = p->indices_in_resource ? r->indices.GetBufferDims() : input_blobs_.back()->GetBlobDesc().dims;
        if (p->axis < 0 || p->axis >= (int)data.size())
            return Status(TNNERR_PARAM_ERR, "Gather axis out of range");
        DimsVector out(data.begin(), data.begin() + p->axis);
        out.insert(out.end(), idx.begin(), idx.end());
        out.insert(out.end(), data.begin() + p->axis + 1, data.end());
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

struct UnsqueezeLayer : BaseLayer {  // layer/unsqueeze_layer.cc:35-59
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        auto p = dynamic_cast<SqueezeLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        DimsVector out = input_blobs_[0]->GetBlobDesc().dims;
        for (int axis : p->axes) {
            axis = axis < 0 ? axis + (int)out.size() + 1 : axis;
            if (axis < 0 || axis > (int)out.size())
                return Status(TNNERR_PARAM_ERR, "UnsqueezeLayer has invalid input axes");
            out.insert(out.begin() + axis, 1);
        }
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};
struct SqueezeLayer : BaseLayer {  // layer/squeeze_layer.cc:35-60 (axes ascending, removed from the back)
    using BaseLayer::BaseLayer;
    Status InferOutputShape(bool ignore_error = false) override {
        auto p = dynamic_cast<SqueezeLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        DimsVector out = input_blobs_[0]->GetBlobDesc().dims;
        if (out.empty())
            return Status(TNNERR_PARAM_ERR, "SqueezeLayer has invalid input size");
        for (auto it = p->axes.rbegin(); it != p->axes.rend(); ++it) {
            int axis = *it < 0 ? *it + (int)out.size() : *it;
            if (axis < 0 || axis >= (int)out.size() || out[axis] != 1)
                return Status(TNNERR_PARAM_ERR, "SqueezeLayer has invalid input axes");
            out.erase(out.begin() + axis);
        }
        output_blobs_[0]->GetBlobDesc().dims = out;
        return TNN_OK;
    }
};

struct CastLayer : BaseLayer {
    using BaseLayer::BaseLayer;
    Status InferOutputDataType() override {
        auto p = dynamic_cast<CastLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        output_blobs_[0]->GetBlobDesc().data_type = (DataType)p->to;
        return TNN_OK;
    }
};

struct ReformatLayer : BaseLayer {  // layer/reformat_layer.cc
    using BaseLayer::BaseLayer;
    Status InferOutputDataType() override {  // reformat_layer.cc:22-28
        auto p = dynamic_cast<ReformatLayerParam *>(param_);
        CHECK_PARAM_NULL(p);
        for (auto b : output_blobs_)
            b->GetBlobDesc().data_type = p->dst_type;
        return TNN_OK;
    }
};

}  // namespace

std::map<LayerType, std::shared_ptr<LayerCreator>> &GetGlobalLayerCreatorMap() {
    static std::map<LayerType, std::shared_ptr<LayerCreator>> m;
    return m;
}

BaseLayer *CreateLayer(LayerType type) {
    // layer classes that register themselves (base_layer.cc: the global creator map), e.g. the ROCm backend's fused layers
    auto &reg = GetGlobalLayerCreatorMap();
    auto it   = reg.find(type);
    if (it != reg.end())
        return it->second->CreateLayer();
    switch (type) {
        case LAYER_INNER_PRODUCT: return new InnerProductLayer(type);
        case LAYER_MATMUL: return new MatMulLayer(type);
        case LAYER_ADD:
        case LAYER_SUB:
        case LAYER_MUL:
        case LAYER_DIV: return new BinaryLayer(type);
        case LAYER_RESHAPE: return new ReshapeLayer(type);
        case LAYER_PERMUTE: return new PermuteLayer(type);
        case LAYER_LAYER_NORM: return new LayerNormLayer(type);
        case LAYER_GATHER: return new GatherLayer(type);
        case LAYER_CAST: return new CastLayer(type);
        case LAYER_SQUEEZE: return new SqueezeLayer(type);
        case LAYER_UNSQUEEZE: return new UnsqueezeLayer(type);
        case LAYER_REFORMAT: return new ReformatLayer(type);
        case LAYER_SOFTMAX:
        case LAYER_GELU:
        case LAYER_TANH: return new BaseLayer(type);
        default: return nullptr;
    }
}

// ---- optimizer manager (source/tnn/optimizer/net_optimizer_manager.cc:33-48) -----------------------
namespace {
using optimizer::NetOptimizer;
std::vector<std::pair<int, std::shared_ptr<NetOptimizer>>> &OptimizerList() {
    static std::vector<std::pair<int, std::shared_ptr<NetOptimizer>>> v;
    return v;
}
std::mutex g_optimize_mutex;

}  // namespace

void optimizer::NetOptimizerManager::RegisterNetOptimizer(NetOptimizer *opt, OptPriority prior) {
    if (opt && opt->Strategy().length() > 0)
        OptimizerList().push_back({(int)prior, std::shared_ptr<NetOptimizer>(opt)});
}
// The engine's own pass for weight-only int8 models (optimizer/net_optimizer_dynamic_range_dequant.cc:44-330, priority
// P1, ahead of every device's passes by its name): the int8 weights of MatMul (resource or constant-map form),
// InnerProduct and Gather tables become fp32 = scale * value before any layer is created, and the layers run as float
// layers from then on.
namespace {
class DynamicRangeDequantPass : public optimizer::NetOptimizer {
public:
    std::string Strategy() override { return "net_optimizer_dynamic_range_dequant"; }
    bool IsSupported(const NetworkConfig &) override { return true; }
    Status Optimize(NetStructure *structure, NetResource *resource) override {
        if (!structure)
            return Status(TNNERR_NET_ERR, "Error: empty NetStructure");
        if (structure->layers.size() <= 1)
            return TNN_OK;
        for (auto &layer : structure->layers) {
            if (!layer || !layer->param || !layer->param->dynamic_range_quantized)
                continue;
            auto it            = resource->resource_map.find(layer->name);
            LayerResource *res = it == resource->resource_map.end() ? nullptr : it->second.get();
            switch (layer->type) {
                case LAYER_MATMUL: {
                    auto p = dynamic_cast<MatMulLayerParam *>(layer->param.get());
                    auto r = dynamic_cast<MatMulLayerResource *>(res);
                    if (p && p->weight_position == 1) {
                        if (!r)
                            return Status(TNNERR_INVALID_MODEL, "dynamic range quantised MatMul without resource: " + layer->name);
                        RETURN_ON_NEQ(PerTensor(r->weight, r->scale_handle, layer->name), TNN_OK);
                    } else if (p && p->weight_position == -1 && layer->inputs.size() == 2) {
                        // the int8 operand is a constant, its scale sits next to it under a suffixed name (:203-238)
                        for (const std::string &name : layer->inputs) {
                            auto c = resource->constant_map.find(name);
                            if (c == resource->constant_map.end() || !c->second || c->second->GetDataType() != DATA_TYPE_INT8)
                                continue;
                            const std::string scale_name = name + "_dynamic_range_quant_scale";
                            auto sc                      = resource->constant_map.find(scale_name);
                            if (sc == resource->constant_map.end() || !sc->second)
                                return Status(TNNERR_PARAM_ERR, "scale is not found in constant map");
                            RETURN_ON_NEQ(PerTensor(*c->second, *sc->second, layer->name), TNN_OK);
                            resource->constant_map.erase(scale_name);
                            break;
                        }
                    }
                    break;
                }
                case LAYER_INNER_PRODUCT: {
                    auto r = dynamic_cast<InnerProductLayerResource *>(res);
                    if (!r)
                        return Status(TNNERR_INVALID_MODEL, "dynamic range quantised InnerProduct without resource: " + layer->name);
                    RETURN_ON_NEQ(PerTensor(r->weight_handle, r->scale_handle, layer->name), TNN_OK);
                    break;
                }
                case LAYER_GATHER: {  // one scale per row of the table (:277-322)
                    auto p = dynamic_cast<GatherLayerParam *>(layer->param.get());
                    auto r = dynamic_cast<GatherLayerResource *>(res);
                    if (!p || !p->data_in_resource || !r)
                        break;
                    const DimsVector dims = r->data.GetBufferDims();
                    if (r->data.GetDataType() != DATA_TYPE_INT8 || dims.size() < 2 || r->scale_data.GetDataCount() != dims[0] ||
                        r->scale_data.GetDataType() != DATA_TYPE_FLOAT)
                        break;  // "might have been dequantized before"
                    const int count = r->data.GetDataCount(), rows = dims[0];
                    if (rows <= 0 || count % rows != 0)
                        return Status(TNNERR_INVALID_MODEL, "dynamic range quantised Gather table with ragged rows: " + layer->name);
                    const int stride = count / rows;
                    RawBuffer wide(count * 4, dims);
                    wide.SetDataType(DATA_TYPE_FLOAT);
                    const int8_t *q  = r->data.force_to<int8_t *>();
                    const float *sc  = r->scale_data.force_to<float *>();
                    float *w         = wide.force_to<float *>();
                    for (int i = 0; i < rows; ++i)
                        for (int j = 0; j < stride; ++j)
                            w[(size_t)i * stride + j] = sc[i] * (float)q[(size_t)i * stride + j];
                    r->data = wide;
                    break;
                }
                default: break;
            }
            layer->param->dynamic_range_quantized = false;
        }
        return TNN_OK;
    }

private:
    // fp32 = scale[0] * int8 in place of the int8 record, dims kept (:176-192, 249-268)
    static Status PerTensor(RawBuffer &weight, const RawBuffer &scale, const std::string &layer) {
        if (weight.GetDataType() != DATA_TYPE_INT8)
            return TNN_OK;  // "might have been dequantized before"
        if (scale.GetDataCount() < 1 || scale.GetDataType() != DATA_TYPE_FLOAT)
            return Status(TNNERR_INVALID_MODEL, "dynamic range quantised weight without a float scale: " + layer);
        const int count = weight.GetDataCount();
        RawBuffer wide(count * 4, weight.GetBufferDims());
        wide.SetDataType(DATA_TYPE_FLOAT);
        const int8_t *q = weight.force_to<int8_t *>();
        const float s   = scale.force_to<float *>()[0];
        float *w        = wide.force_to<float *>();
        for (int i = 0; i < count; ++i)
            w[i] = s * (float)q[i];
        weight = wide;
        return TNN_OK;
    }
};
optimizer::NetOptimizerRegister<DynamicRangeDequantPass> g_dynamic_range_dequant(optimizer::P1);
}  // namespace

Status optimizer::NetOptimizerManager::Optimize(NetStructure *structure, NetResource *resource, const NetworkConfig &config) {
    std::lock_guard<std::mutex> lock(g_optimize_mutex);
    auto list = OptimizerList();
    std::stable_sort(list.begin(), list.end(), [](const std::pair<int, std::shared_ptr<NetOptimizer>> &a,
                                                  const std::pair<int, std::shared_ptr<NetOptimizer>> &b) {
        return a.first != b.first ? a.first < b.first : a.second->Strategy() < b.second->Strategy();
    });
    for (auto &o : list)
        if (o.second->IsSupported(config))
            RETURN_ON_NEQ(o.second->Optimize(structure, resource), TNN_OK);
    return TNN_OK;
}

// ---- network (source/tnn/core/default_network.cc:62-138, 157-331, 558-635) --------------------------
DefaultNetwork::~DefaultNetwork() {
    if (context_)
        context_->Synchronize();
    for (auto l : layers_)
        delete l;
    for (auto &kv : blobs_)
        delete kv.second;
    if (device_)
        for (void *p : allocations_)
            device_->Free(p);
    for (auto &e : prof_events_) {
        tnn_rocm_event_destroy(e.first);
        tnn_rocm_event_destroy(e.second);
    }
    delete context_;
}

Status DefaultNetwork::Plan(NetworkConfig &net_config, ModelInterpreter *interpreter, const InputShapesMap &inputs_shape) {
    config_ = net_config;
    device_ = GetDevice(net_config.device_type);
    if (!device_)
        return Status(TNNERR_DEVICE_NOT_SUPPORT, "device not support");
    structure_ = *interpreter->GetNetStructure();
    structure_.layers.clear();
    for (auto &l : interpreter->GetNetStructure()->layers)
        structure_.layers.push_back(std::make_shared<LayerInfo>(*l));
    resource_ = *interpreter->GetNetResource();
    for (auto &kv : inputs_shape) {
        auto it = structure_.inputs_shape_map.find(kv.first);
        if (it == structure_.inputs_shape_map.end())
            return Status(TNNERR_PARAM_ERR, "input shape given for " + kv.first + ", which is not an input of the model");
        if (it->second.size() != kv.second.size())
            return Status(TNNERR_PARAM_ERR, "input shape given for " + kv.first + " has another number of dimensions than the model's");
        it->second = kv.second;
    }
    RETURN_ON_NEQ(optimizer::NetOptimizerManager::Optimize(&structure_, &resource_, config_), TNN_OK);
    return InitLayers();  // context_ stays null: shapes and types only
}

Status DefaultNetwork::Init(NetworkConfig &net_config, ModelInterpreter *interpreter, const InputShapesMap &max_inputs_shape) {
    config_ = net_config;
    device_ = GetDevice(net_config.device_type);
    if (!device_)  // instance.cc:60-62
        return Status(TNNERR_DEVICE_NOT_SUPPORT, "device not support");
    context_ = device_->CreateContext(net_config.device_id);
    if (!context_)
        return Status(TNNERR_DEVICE_CONTEXT_CREATE, "create context failed");
    context_->SetPrecision(net_config.precision);
    RETURN_ON_NEQ(context_->LoadLibrary(net_config.library_path), TNN_OK);
    // deep copy: the optimizer rewrites only this instance's graph (instance.cc:64-71)
    structure_ = *interpreter->GetNetStructure();
    structure_.layers.clear();
    for (auto &l : interpreter->GetNetStructure()->layers)
        structure_.layers.push_back(std::make_shared<LayerInfo>(*l));
    resource_ = *interpreter->GetNetResource();
    for (auto &kv : max_inputs_shape) {  // instance.cc:76-83 / default_network.cc:104-108
        auto it = structure_.inputs_shape_map.find(kv.first);
        if (it == structure_.inputs_shape_map.end())
            return Status(TNNERR_PARAM_ERR, "input shape given for " + kv.first + ", which is not an input of the model");
        if (it->second.size() != kv.second.size())
            return Status(TNNERR_PARAM_ERR, "input shape given for " + kv.first + " has another number of dimensions than the model's");
        it->second = kv.second;
    }
    RETURN_ON_NEQ(optimizer::NetOptimizerManager::Optimize(&structure_, &resource_, config_), TNN_OK);
    RETURN_ON_NEQ(InitLayers(), TNN_OK);
    RETURN_ON_NEQ(AllocateBlobMemory(), TNN_OK);
    RETURN_ON_NEQ(context_->OnInstanceReshapeBegin(), TNN_OK);
    for (auto l : layers_)
        RETURN_ON_NEQ(l->Reshape(), TNN_OK);
    return context_->OnInstanceReshapeEnd();
}

Status DefaultNetwork::ReleaseBlobMemory() {
    RETURN_ON_NEQ(context_->Synchronize(), TNN_OK);
    for (auto &kv : blob_capacity_)
        kv.first->SetHandle(BlobHandle());
    blob_capacity_.clear();
    for (void *p : allocations_)
        device_->Free(p);
    allocations_.clear();
    return TNN_OK;
}

// default_network.cc:456-500 (Reshape -> PrepareDoReshape -> DoReshape -> ReshapeLayers)
Status DefaultNetwork::Reshape(const InputShapesMap &inputs) {
    bool shape_changed = false;
    for (auto &kv : inputs) {
        auto it = inputs_.find(kv.first);
        if (it == inputs_.end())
            return Status(TNNERR_PARAM_ERR, "DefaultNetwork reshape blob is empty, maybe the blob name is wrong");
        auto &dims = it->second->GetBlobDesc().dims;
        if (dims.size() != kv.second.size())
            return Status(TNNERR_PARAM_ERR, "DefaultNetwork reshape: input " + kv.first + " keeps its number of dimensions");
        for (int d : kv.second)
            if (d <= 0)
                return Status(TNNERR_PARAM_ERR, "DefaultNetwork reshape: input " + kv.first + " gets a dimension below 1");
        if (dims != kv.second) {
            dims          = kv.second;
            shape_changed = true;
        }
    }
    if (!shape_changed)
        return TNN_OK;
    // nothing of the old shape may still be running when blobs change size or move
    RETURN_ON_NEQ(context_->Synchronize(), TNN_OK);
    RETURN_ON_NEQ(context_->OnInstanceReshapeBegin(), TNN_OK);
    // shapes first (layer order = topological order), then memory, then the accs, which may look at the blobs' memory
    for (size_t i = 0; i < layers_.size(); ++i) {
        Status st = layers_[i]->InferOutputShape();
        if (st != TNN_OK)
            return Status((int)st, "reshape of layer " + layers_[i]->GetLayerName() + " failed: " + st.description());
    }
    bool fits = true;
    for (auto &kv : blob_capacity_) {
        BlobMemorySizeInfo info = device_->Calculate(kv.first->GetBlobDesc());
        fits &= GetBlobMemoryBytesSize(info) <= kv.second;
    }
    if (!fits) {
        RETURN_ON_NEQ(ReleaseBlobMemory(), TNN_OK);
        RETURN_ON_NEQ(AllocateBlobMemory(), TNN_OK);
    }
    for (size_t i = 0; i < layers_.size(); ++i) {
        Status st = layers_[i]->Reshape();
        if (st != TNN_OK)
            return Status((int)st, "reshape of layer " + layers_[i]->GetLayerName() + " failed: " + st.description());
    }
    return context_->OnInstanceReshapeEnd();
}

Blob *DefaultNetwork::GetBlob(const std::string &name) {
    auto it = blobs_.find(name);
    return it == blobs_.end() ? nullptr : it->second;
}

Status DefaultNetwork::InitLayers() {
    const bool half = config_.precision != PRECISION_HIGH &&
                      device_->GetImplementedPrecision(LAYER_MATMUL)->fp16_implemented;
    // PRECISION_LOW selects bfloat16 activations (the engine's meaning of LOW on its bfp16-capable CPU backend,
    // include/tnn/core/common.h:131-140); every other reduced precision is fp16
    const DataType half_type = config_.precision == PRECISION_LOW ? DATA_TYPE_BFP16 : DATA_TYPE_HALF;
    bool quantized_net = false;
    for (auto &l : structure_.layers)
        quantized_net |= l->param->quantized;

    auto make_blob = [&](const std::string &name, bool int8) -> Blob * {
        auto it = blobs_.find(name);
        if (it != blobs_.end() && (!int8 || dynamic_cast<BlobInt8 *>(it->second)))
            return it->second;
        BlobDesc desc;
        if (it != blobs_.end()) {
            desc = it->second->GetBlobDesc();
            delete it->second;
        }
        desc.name        = name;
        desc.device_type = config_.device_type;
        Blob *b          = nullptr;
        if (int8) {
            auto nb        = new BlobInt8(desc, BlobHandle());
            desc.data_type = DATA_TYPE_INT8;
            nb->GetBlobDesc().data_type = DATA_TYPE_INT8;
            b              = nb;
        } else {
            b = new Blob(desc);
        }
        blobs_[name] = b;
        return b;
    };

    // model inputs
    for (auto &kv : structure_.inputs_shape_map) {
        Blob *b     = make_blob(kv.first, false);
        auto &desc  = b->GetBlobDesc();
        desc.dims   = kv.second;
        auto dt_it  = structure_.input_data_type_map.find(kv.first);
        DataType dt = dt_it == structure_.input_data_type_map.end() ? DATA_TYPE_FLOAT : dt_it->second;
        if (dt == DATA_TYPE_FLOAT && half)
            dt = half_type;
        desc.data_type = dt;
        inputs_[kv.first] = b;
    }
    // constants: blobs that carry their dims; the accs upload the data (ReloadConstantBlobs)
    for (auto &kv : resource_.constant_map) {
        Blob *b                     = make_blob(kv.first, false);
        b->GetBlobDesc().dims       = kv.second->GetBufferDims();
        b->GetBlobDesc().data_type  = kv.second->GetDataType();
        b->SetConstant(true);
    }

    for (auto &info : structure_.layers) {
        BaseLayer *layer = CreateLayer(info->type);
        if (!layer)  // default_network.cc:246-250
            return Status(TNNERR_PARAM_ERR, "CreateLayer failed for type " + info->type_str);
        layers_.push_back(layer);
        auto param = info->param.get();
        std::vector<Blob *> ins, outs;
        auto want_int8 = [&](bool is_input, size_t idx) -> bool {  // default_network.cc:362-440
            return (quantized_net || info->type == LAYER_REFORMAT) &&
                   RocmBlobIsInt8(info->type, param, is_input, idx, info->outputs.size());
        };
        for (size_t i = 0; i < info->inputs.size(); ++i) {
            const auto &name = info->inputs[i];
            if (!blobs_.count(name))
                return Status(TNNERR_NET_ERR, "layer " + info->name + " reads blob " + name + " before it is produced");
            ins.push_back(make_blob(name, want_int8(true, i)));
        }
        for (size_t i = 0; i < info->outputs.size(); ++i)
            outs.push_back(make_blob(info->outputs[i], want_int8(false, i)));
        for (auto blobs : {&ins, &outs})
            for (auto b : *blobs)
                if (auto bi = dynamic_cast<BlobInt8 *>(b)) {
                    if (bi->GetIntResource())
                        continue;
                    auto it = resource_.resource_map.find(b->GetBlobDesc().name + "_scale_data_");
                    auto r  = it == resource_.resource_map.end() ? nullptr
                                                                 : dynamic_cast<IntScaleResource *>(it->second.get());
                    if (!r)  // default_network.cc:350-353
                        return Status(TNNERR_NULL_PARAM, "Error Init layer, can not get blob scale " +
                                                             b->GetBlobDesc().name + "_scale_data_");
                    bi->SetIntResource(r);
                }
        // float outputs of a dequantising Reformat (or of a fused layer that contains one) follow the network precision
        if (info->type == LAYER_REFORMAT || info->type == LAYER_ROCM_FUSED_LINEAR_INT8 ||
            info->type == LAYER_ROCM_FUSED_ATTENTION || info->type == LAYER_ROCM_FUSED_EMBEDDING)
            for (auto b : outs)
                if (!dynamic_cast<BlobInt8 *>(b))
                    b->GetBlobDesc().data_type = half ? half_type : DATA_TYPE_FLOAT;
        LayerResource *res = nullptr;
        auto rit           = resource_.resource_map.find(info->name);
        if (rit != resource_.resource_map.end())
            res = rit->second.get();
        Status st = layer->Init(context_, param, res, ins, outs, device_, &resource_.constant_map);
        if (st != TNN_OK)
            return Status((int)st, "layer " + info->name + " (" + info->type_str + ") init failed: " + st.description());
        // Gather from an fp32 table and Reformat produce the network's float type
        if (half)
            for (auto b : outs)
                if (b->GetBlobDesc().data_type == DATA_TYPE_FLOAT)
                    b->GetBlobDesc().data_type = half_type;
    }
    for (auto &name : structure_.outputs) {
        auto it = blobs_.find(name);
        if (it == blobs_.end())
            return Status(TNNERR_NET_ERR, "output blob " + name + " is not produced by any layer");
        outputs_[name] = it->second;
    }
    // a model input read directly by a quantized layer was replaced by a BlobInt8 above
    for (auto &kv : inputs_)
        kv.second = blobs_[kv.first];
    return TNN_OK;
}

// Blob memory with liveness-based reuse (the role of source/tnn/core/blob_manager.cc:156-227):
// a blob's buffer returns to the pool after its last reader; inputs, outputs and constants are
// never shared.  The output of a layer that only renames dimensions (Reshape in the ONNX order, Squeeze, Unsqueeze)
// shares its input's buffer, so the layer has nothing to copy; the buffer returns to the pool after the last reader
// of any of its names.  TNN_ROCM_ALIAS_VIEWS=0 gives every blob its own buffer again.
Status DefaultNetwork::AllocateBlobMemory() {
    std::map<std::string, int> last_use;
    for (int i = 0; i < (int)structure_.layers.size(); ++i)
        for (auto &n : structure_.layers[i]->inputs)
            last_use[n] = i;
    const char *alias_env  = getenv("TNN_ROCM_ALIAS_VIEWS");
    const bool alias_views = !(alias_env && alias_env[0] == '0');
    std::map<std::string, std::string> alias_root;  // view output -> the blob that owns the buffer
    std::map<std::string, int> group_last;          // owner -> last layer that reads the buffer under any name
    auto root_of = [&](const std::string &n) -> std::string {
        auto it = alias_root.find(n);
        return it == alias_root.end() ? n : it->second;
    };
    int64_t total_bytes = 0;
    std::multimap<int64_t, void *> pool;  // free buffers by capacity
    std::map<std::string, std::pair<int64_t, void *>> owned;
    auto alloc_for = [&](Blob *b, bool reusable) -> Status {
        BlobMemorySizeInfo info = device_->Calculate(b->GetBlobDesc());
        int64_t bytes           = std::max<int64_t>(GetBlobMemoryBytesSize(info), 16);
        void *ptr               = nullptr;
        if (reusable) {
            auto it = pool.lower_bound(bytes);
            if (it != pool.end() && it->first <= bytes * 2) {
                ptr   = it->second;
                bytes = it->first;
                pool.erase(it);
            }
        }
        if (!ptr) {
            info.data_type = DATA_TYPE_INT8;
            info.dims      = {(int)bytes};
            RETURN_ON_NEQ(device_->Allocate(&ptr, info), TNN_OK);
            allocations_.push_back(ptr);
            total_bytes += bytes;
        }
        BlobHandle h;
        h.base = ptr;
        b->SetHandle(h);
        blob_capacity_[b]            = bytes;
        owned[b->GetBlobDesc().name] = {bytes, ptr};
        return TNN_OK;
    };
    for (auto &kv : inputs_)
        RETURN_ON_NEQ(alloc_for(kv.second, false), TNN_OK);
    for (int i = 0; i < (int)structure_.layers.size(); ++i) {
        auto &info = structure_.layers[i];
        bool is_view = alias_views && info->outputs.size() == 1 && !info->inputs.empty() &&
                       (info->type == LAYER_RESHAPE || info->type == LAYER_SQUEEZE || info->type == LAYER_UNSQUEEZE);
        if (is_view && info->type == LAYER_RESHAPE) {
            auto rp = dynamic_cast<ReshapeLayerParam *>(info->param.get());
            is_view = rp == nullptr || rp->reshape_type == 0;
        }
        if (is_view) {
            const std::string &xn = info->inputs[0], &yn = info->outputs[0];
            const std::string rn  = root_of(xn);
            Blob *x = blobs_[xn], *y = blobs_[yn], *r = blobs_[rn];
            if (!y->GetHandle().base && x->GetHandle().base && owned.count(rn) && !inputs_.count(rn) &&
                !outputs_.count(yn) && !outputs_.count(rn) && !r->IsConstant() &&
                x->GetBlobDesc().data_type == y->GetBlobDesc().data_type) {
                y->SetHandle(x->GetHandle());
                blob_capacity_[y] = blob_capacity_[r];
                alias_root[yn]    = rn;
                int last          = group_last.count(rn) ? group_last[rn] : (last_use.count(rn) ? last_use[rn] : i);
                if (last_use.count(yn))
                    last = std::max(last, last_use[yn]);
                group_last[rn] = std::max(last, i);
            }
        }
        for (auto &n : info->outputs) {
            Blob *b = blobs_[n];
            if (b->GetHandle().base)
                continue;
            bool pinned = outputs_.count(n) > 0;
            RETURN_ON_NEQ(alloc_for(b, !pinned), TNN_OK);
        }
        // release buffers whose last reader (under any of their names) is this layer (never inputs/outputs/constants)
        for (auto &n : info->inputs) {
            const std::string rn = root_of(n);
            const int last       = group_last.count(rn) ? group_last[rn] : last_use[rn];
            if (last != i || inputs_.count(rn) || outputs_.count(rn) || blobs_[rn]->IsConstant())
                continue;
            auto it = owned.find(rn);
            if (it != owned.end()) {
                pool.insert({it->second.first, it->second.second});
                owned.erase(it);
            }
        }
        // an output nobody reads (a float tensor whose only reader was folded away) is free again right after its layer
        for (auto &n : info->outputs) {
            if (last_use.count(n) || outputs_.count(n) || alias_root.count(n))
                continue;
            auto it = owned.find(n);
            if (it != owned.end()) {
                pool.insert({it->second.first, it->second.second});
                owned.erase(it);
            }
        }
    }
    if (getenv("TNN_ROCM_VERBOSE"))
        fprintf(stderr, "tnn-rocm: %zu blob buffers, %.1f MiB of activation memory for %zu layers\n", allocations_.size(),
                (double)total_bytes / (1024.0 * 1024.0), structure_.layers.size());
    return TNN_OK;
}

Status DefaultNetwork::RunLayers(void *prof_stream) {
    for (size_t i = 0; i < layers_.size(); ++i) {
        const bool timed = profiling_ && prof_on_[i];
        if (timed)
            tnn_rocm_event_record(prof_events_[i].first, prof_stream);
        Status st = layers_[i]->Forward();
        if (timed)
            tnn_rocm_event_record(prof_events_[i].second, prof_stream);
        if (st != TNN_OK)  // default_network.cc:599-605
            return Status((int)st, "Forward error of layer " + layers_[i]->GetLayerName() + ": " + st.description());
    }
    return TNN_OK;
}

// The layer loop of default_network.cc:571-631 (ForwardAsync: :672-686), with the per-layer event timing of the
// profile hook.
Status DefaultNetwork::ForwardAsync(Callback) {
    RETURN_ON_NEQ(context_->OnInstanceForwardBegin(), TNN_OK);
    void *stream = nullptr;
    context_->GetCommandQueue(&stream);
    RETURN_ON_NEQ(RunLayers(stream), TNN_OK);
    if (profiling_) {
        for (size_t i = 0; i < layers_.size(); ++i) {
            float ms = 0;
            if (!prof_on_[i])
                continue;
            if (tnn_rocm_event_elapsed_ms(prof_events_[i].first, prof_events_[i].second, &ms) == 0) {
                prof_[i].ms += ms;
                prof_[i].calls += 1;
            }
        }
    }
    return context_->OnInstanceForwardEnd();
}
Status DefaultNetwork::Forward() {
    RETURN_ON_NEQ(DefaultNetwork::ForwardAsync(nullptr), TNN_OK);
    return context_->Synchronize();
}
Status DefaultNetwork::ForwardWithCallback(BlobStatisticCallback before, BlobStatisticCallback after) {
    RETURN_ON_NEQ(context_->OnInstanceForwardBegin(), TNN_OK);
    for (size_t i = 0; i < layers_.size(); ++i) {
        std::vector<Blob *> inputs = layers_[i]->GetInputBlobs(), outputs = layers_[i]->GetOutputBlobs();
        LayerInfo *info = i < structure_.layers.size() ? structure_.layers[i].get() : nullptr;
        if (before)
            before(inputs, info);
        Status st = layers_[i]->Forward();
        if (st != TNN_OK)
            return Status((int)st, "Forward error of layer " + layers_[i]->GetLayerName() + ": " + st.description());
        RETURN_ON_NEQ(context_->Synchronize(), TNN_OK);  // the callback may read the blobs
        if (after)
            after(outputs, info);
    }
    return context_->OnInstanceForwardEnd();
}
// core/abstract_network.cc:24-45
namespace {
std::map<NetworkType, std::shared_ptr<AbstractNetworkImplFactory>> &NetworkImplFactoryMap() {
    static std::map<NetworkType, std::shared_ptr<AbstractNetworkImplFactory>> m;
    return m;
}
NetworkImplFactoryRegister<NetworkImplFactory<DefaultNetwork>> g_network_impl_default_factory_register(NETWORK_TYPE_DEFAULT);
}  // namespace
std::shared_ptr<DefaultNetwork> NetworkImplManager::GetNetworkImpl(NetworkType type) {
    auto &m = NetworkImplFactoryMap();
    auto it = m.find(type);
    return it == m.end() ? nullptr : it->second->CreateNetworkImp();
}
void NetworkImplManager::RegisterNetworkImplFactory(NetworkType type, AbstractNetworkImplFactory *factory) {
    if (factory)
        NetworkImplFactoryMap()[type] = std::shared_ptr<AbstractNetworkImplFactory>(factory);
}

Status DefaultNetwork::GetCommandQueue(void **q) { return context_->GetCommandQueue(q); }
Status DefaultNetwork::ShareCommandQueue(DefaultNetwork *network) {
    if (!network || !network->GetContext())
        return Status(TNNERR_DEVICE_CONTEXT_CREATE, "network is nil");
    return context_->ShareCommandQueue(network->GetContext());
}
Status DefaultNetwork::SetCpuNumThreads(int num_threads) { return context_->SetNumThreads(num_threads); }
Status DefaultNetwork::GetAllInputBlobs(BlobMap &blobs) {
    blobs = inputs_;
    return TNN_OK;
}
Status DefaultNetwork::GetAllOutputBlobs(BlobMap &blobs) {
    blobs = outputs_;
    return TNN_OK;
}
std::string DefaultNetwork::LayerSummary() const {
    std::ostringstream os;
    for (auto &l : structure_.layers)
        os << l->type_str << " " << l->name << "\n";
    return os.str();
}
std::string DefaultNetwork::LayerIo() const {
    std::ostringstream os;
    auto names = [&](const std::vector<std::string> &v) {
        for (size_t i = 0; i < v.size(); ++i)
            os << (i ? "," : "") << v[i];
    };
    auto dims = [&](const std::vector<std::string> &v) {
        for (size_t i = 0; i < v.size(); ++i) {
            os << (i ? ";" : "");
            auto it = blobs_.find(v[i]);
            if (it == blobs_.end())
                continue;
            const auto &d = it->second->GetBlobDesc().dims;
            for (size_t k = 0; k < d.size(); ++k)
                os << (k ? "," : "") << d[k];
        }
    };
    for (auto &l : structure_.layers) {
        os << l->name << "|";
        names(l->inputs);
        os << "|";
        names(l->outputs);
        os << "|";
        dims(l->inputs);
        os << "|";
        dims(l->outputs);
        os << "\n";
    }
    return os.str();
}
void DefaultNetwork::StartProfile(const std::string &only_type) {
    prof_.clear();
    prof_on_.clear();
    for (auto &l : structure_.layers)
        prof_on_.push_back(only_type.empty() || l->type_str == only_type ? 1 : 0);
    for (size_t i = prof_events_.size(); i < layers_.size(); ++i) {
        void *a = nullptr, *b = nullptr;
        tnn_rocm_event_create(&a);
        tnn_rocm_event_create(&b);
        prof_events_.push_back({a, b});
    }
    for (auto &l : structure_.layers) {
        LayerProfile p;
        p.name = l->name;
        p.type = l->type_str;
        prof_.push_back(p);
    }
    profiling_ = true;
}
std::vector<LayerProfile> DefaultNetwork::FinishProfile() {
    profiling_ = false;
    return prof_;
}

// ---- instance (source/tnn/core/instance.cc:48-128, 166-169, 203-319) --------------------------------
Status Instance::Init() { return Init(InputShapesMap(), InputShapesMap()); }
Status Instance::Init(const InputShapesMap &, const InputShapesMap &max_inputs_shape) {
    interpreter_ = std::make_shared<ModelInterpreter>();
    RETURN_ON_NEQ(interpreter_->Interpret(model_config_.params), TNN_OK);
    auto device = GetDevice(net_config_.device_type);
    if (!device)
        return Status(TNNERR_DEVICE_NOT_SUPPORT, "device not support");
    if (net_config_.network_type == NETWORK_TYPE_AUTO)
        net_config_.network_type = device->ConvertAutoNetworkType();
    network_ = NetworkImplManager::GetNetworkImpl(net_config_.network_type);  // instance.cc:75-85
    if (!network_)
        return Status(TNNERR_NET_ERR, "network_ is nil, network_type may not support");
    return network_->Init(net_config_, interpreter_.get(), max_inputs_shape);
}
Status Instance::Reshape(const InputShapesMap &inputs) {
    if (!network_)
        return Status(TNNERR_INST_ERR, "instance not initialised");
    output_mats_.clear();
    return network_->Reshape(inputs);
}
Status Instance::Forward() { return network_ ? network_->Forward() : Status(TNNERR_INST_ERR, "instance not initialised"); }
Status Instance::ForwardAsync(Callback call_back) {
    return network_ ? network_->ForwardAsync(call_back) : Status(TNNERR_INST_ERR, "instance not initialised");
}
Status Instance::GetCommandQueue(void **q) { return network_->GetCommandQueue(q); }
Status Instance::ForwardWithCallback(BlobStatisticCallback before, BlobStatisticCallback after) {
    return network_->ForwardWithCallback(before, after);
}
Status Instance::ShareCommandQueue(Instance *instance) {
    if (!instance)
        return Status(TNNERR_NULL_PARAM, "instance is nil");
    return network_->ShareCommandQueue(instance->GetNetwork());
}
Status Instance::SetCpuNumThreads(int num_threads) { return network_->SetCpuNumThreads(num_threads); }
Status Instance::GetAllInputBlobs(BlobMap &b) { return network_->GetAllInputBlobs(b); }
Status Instance::GetAllOutputBlobs(BlobMap &b) { return network_->GetAllOutputBlobs(b); }

Status Instance::SetInputMat(std::shared_ptr<Mat> mat, MatConvertParam param, std::string input_name) {
    if (!mat)
        return Status(TNNERR_NULL_PARAM, "input mat is empty, please check!");
    BlobMap ins;
    network_->GetAllInputBlobs(ins);
    if (ins.empty())
        return Status(TNNERR_COMMON_ERROR, "instance.GetAllInputBlobs Error");
    Blob *blob = nullptr;
    if (input_name.empty()) {
        blob = ins.begin()->second;
    } else {
        auto it = ins.find(input_name);
        if (it == ins.end())
            return Status(TNNERR_MODEL_ERR, "instance dont have the input with name: " + input_name);
        blob = it->second;
    }
    if (DimsVectorUtils::Count(mat->GetDims()) != DimsVectorUtils::Count(blob->GetBlobDesc().dims))
        return Status(TNNERR_INVALID_INPUT, "input mat element count differs from the input blob");
    void *q = nullptr;
    network_->GetCommandQueue(&q);
    // one converter per input for the life of the instance (instance.cc:228-235), so device staging is allocated once
    auto &conv = input_converters_[blob->GetBlobDesc().name];
    if (!conv.second || conv.first != blob)
        conv = {blob, std::make_shared<BlobConverter>(blob)};
    return conv.second->ConvertFromMatAsync(*mat, param, q);  // instance.cc:241: the forward that follows is on the same queue
}

Status Instance::GetOutputMat(std::shared_ptr<Mat> &mat, MatConvertParam param, std::string output_name,
                              DeviceType device, MatType mat_type) {
    BlobMap outs;
    network_->GetAllOutputBlobs(outs);
    if (outs.empty())
        return Status(TNNERR_COMMON_ERROR, "instance.GetAllOutputBlobs Error");
    Blob *blob = nullptr;
    if (output_name.empty()) {
        blob        = outs.begin()->second;
        output_name = outs.begin()->first;
    } else {
        auto it = outs.find(output_name);
        if (it == outs.end())
            return Status(TNNERR_MODEL_ERR, "instance dont have the output with name: " + output_name);
        blob = it->second;
    }
    auto &cached = output_mats_[output_name];
    if (!cached || cached->GetMatType() != mat_type || cached->GetDeviceType() != device ||
        cached->GetDims() != blob->GetBlobDesc().dims) {
        cached = std::make_shared<Mat>(device, mat_type, blob->GetBlobDesc().dims);
        if (!cached->GetData()) {
            cached.reset();
            return Status(TNNERR_OUTOFMEMORY, "no memory for the output mat on the device asked for");
        }
    }
    void *q = nullptr;
    network_->GetCommandQueue(&q);
    auto &conv = output_converters_[output_name];  // instance.cc:298-305
    if (!conv.second || conv.first != blob)
        conv = {blob, std::make_shared<BlobConverter>(blob)};
    RETURN_ON_NEQ(conv.second->ConvertToMat(*cached, param, q), TNN_OK);
    mat = cached;
    return TNN_OK;
}

}  // namespace TNN_NS
