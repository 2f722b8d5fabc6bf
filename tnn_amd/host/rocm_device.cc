// RocmDevice / RocmContext / RocmLayerAcc / RocmBlobConverterAcc.
#include "rocm_device.h"
#include <immintrin.h>

#include <cstdint>
#include <cstdio>

namespace TNN_NS {

Status RocmStatus(int rc, int tnn_code, const char *what) {
    char buf[768];
    snprintf(buf, sizeof(buf), "%s failed (%d): %s", what, rc, tnn_rocm_last_error());
    // hipErrorOutOfMemory == 2
    return Status(rc == 2 ? (int)TNNERR_OUTOFMEMORY : tnn_code, buf);
}

// ---- context --------------------------------------------------------------------------------
RocmContext::RocmContext(int device_id) : device_id_(device_id) {}

Status RocmContext::Setup() {
    int n = 0;
    tnn_rocm_device_count(&n);
    if (device_id_ < 0 || device_id_ >= n)
        return Status(TNNERR_DEVICE_CONTEXT_CREATE, "no ROCm device with the requested id");
    if (tnn_rocm_set_device(device_id_) != 0 || tnn_rocm_stream_create(&stream_) != 0)
        return RocmStatus(-1, TNNERR_DEVICE_CONTEXT_CREATE, "stream creation");
    void *flag = nullptr;
    if (tnn_rocm_malloc_host(&flag, 64) != 0)
        return RocmStatus(-1, TNNERR_DEVICE_CONTEXT_CREATE, "error flag allocation");
    error_flag_ = (int32_t *)flag;
    return TNN_OK;
}

RocmContext::~RocmContext() {
    if (stream_)
        tnn_rocm_stream_sync(stream_);
    tnn_rocm_free(workspace_);
    for (auto &kv : side_buffers_)
        tnn_rocm_free(kv.second.ptr);
    tnn_rocm_free(mask_cache_.mask_f32);
    tnn_rocm_free(mask_cache_.kv_len);
    tnn_rocm_free_host(error_flag_);
    if (own_stream_)
        tnn_rocm_stream_destroy(stream_);
}

Status RocmContext::ShareCommandQueue(Context *context) {
    if (context == nullptr)
        return Status(TNNERR_NULL_PARAM, "context is nil");
    auto other = dynamic_cast<RocmContext *>(context);
    if (other == nullptr || other->device_id_ != device_id_ || other->stream_ == nullptr)
        return Status(TNNERR_DEVICE_INVALID_COMMAND_QUEUE, "the command queue of another device cannot be shared");
    if (other == this || other->stream_ == stream_)
        return TNN_OK;
    if (stream_) {
        ROCM_CALL(tnn_rocm_stream_sync(stream_));
        if (own_stream_)
            ROCM_CALL(tnn_rocm_stream_destroy(stream_));
    }
    own_stream_ = false;
    stream_     = other->stream_;
    ++memory_epoch_;
    return TNN_OK;
}

Status RocmContext::GetCommandQueue(void **command_queue) {
    if (!command_queue)
        return Status(TNNERR_DEVICE_INVALID_COMMAND_QUEUE, "command_queue is nil");
    *command_queue = stream_;
    return TNN_OK;
}

Status RocmContext::OnInstanceForwardBegin() {
    // one context per instance, used by one thread at a time; select its device for this thread
    ROCM_CALL(tnn_rocm_set_device(device_id_));
    ++forward_epoch_;
    return TNN_OK;
}

Status RocmContext::AttentionMask(const void *mask_blob, int mask_dtype, int B, int S, bool one_row, const float **mask_f32,
                                  const int32_t **kv_len) {
    auto &c = mask_cache_;
    if ((size_t)B * S > c.cap_mask || (size_t)B > c.cap_len || !c.kv_len) {
        ROCM_CALL(tnn_rocm_stream_sync(stream_));
        tnn_rocm_free(c.mask_f32);
        tnn_rocm_free(c.kv_len);
        c.mask_f32 = c.kv_len = nullptr;
        c.cap_mask = c.cap_len = 0;
        ++memory_epoch_;
        ROCM_CALL(tnn_rocm_malloc(&c.mask_f32, (size_t)B * S * sizeof(float)));
        ROCM_CALL(tnn_rocm_malloc(&c.kv_len, (size_t)B * sizeof(int32_t)));
        c.cap_mask = (size_t)B * S, c.cap_len = (size_t)B;
        c.src = nullptr;
    }
    if (c.B != B || c.S != S || c.one_row != one_row)
        c.B = B, c.S = S, c.one_row = one_row, c.src = nullptr;
    // a dense fp32 mask is read where it lies; any other (half precision, or one row for all sequences) from the copy
    const bool in_place = mask_dtype == TNN_ROCM_F32 && !one_row;
    const float *m      = in_place ? (const float *)mask_blob : (const float *)c.mask_f32;
    if (c.src != mask_blob || c.epoch != forward_epoch_) {
        // Keys after the last one whose additive mask lies within 1000 of the row's largest value contribute
        // exp(-1000 + score difference) == 0 in fp32 and are cut (a plain 0 / -10000 padding mask is flagged: the
        // attention kernel then works from the lengths alone); one launch, which also makes the fp32 copy.
        ROCM_CALL(tnn_rocm_mask_prepare_strided(stream_, mask_dtype, mask_blob, one_row ? 0L : (long)S,
                                                in_place ? nullptr : (float *)c.mask_f32, (int32_t *)c.kv_len, B, S, -1000.0f));
        c.src   = mask_blob;
        c.epoch = forward_epoch_;
    }
    *mask_f32 = m;
    *kv_len   = (const int32_t *)c.kv_len;
    return TNN_OK;
}

Status RocmContext::Synchronize() {
    int rc = tnn_rocm_stream_sync(stream_);
    if (rc != 0)
        return RocmStatus(rc, TNNERR_CUDA_SYNC_ERROR, "stream synchronize");
    if (error_flag_ && *error_flag_ != 0) {
        *error_flag_ = 0;
        // cpu_gather_layer_acc.cc:72-78 reports this as TNNERR_MODEL_ERR
        return Status(TNNERR_MODEL_ERR, "RocmGatherLayerAcc::Forward invalid slice_index");
    }
    return TNN_OK;
}

Status RocmContext::Workspace(size_t bytes, void **ptr) {
    if (bytes > workspace_sz_) {
        ROCM_CALL(tnn_rocm_stream_sync(stream_));
        tnn_rocm_free(workspace_);
        workspace_    = nullptr;
        workspace_sz_ = 0;
        ++memory_epoch_;
        size_t want   = bytes + bytes / 4;
        int rc        = tnn_rocm_malloc(&workspace_, want);
        if (rc != 0)
            return RocmStatus(rc, TNNERR_OUTOFMEMORY, "workspace allocation");
        workspace_sz_ = want;
    }
    *ptr = workspace_;
    return TNN_OK;
}

Status RocmContext::SideBuffer(const std::string &name, size_t bytes, void **ptr) {
    auto &e = side_buffers_[name];
    if (bytes > e.cap) {
        ROCM_CALL(tnn_rocm_stream_sync(stream_));
        tnn_rocm_free(e.ptr);
        e.ptr = nullptr;
        e.cap = 0;
        ++memory_epoch_;
        int rc = tnn_rocm_malloc(&e.ptr, bytes);
        if (rc != 0)
            return RocmStatus(rc, TNNERR_OUTOFMEMORY, "side buffer allocation");
        e.cap = bytes;
    }
    *ptr = e.ptr;
    return TNN_OK;
}

// ---- device ---------------------------------------------------------------------------------
std::map<LayerType, std::shared_ptr<LayerAccCreator>> &RocmDevice::GetLayerCreatorMap() {
    static std::map<LayerType, std::shared_ptr<LayerAccCreator>> m;
    return m;
}
Status RocmDevice::RegisterLayerAccCreator(LayerType type, LayerAccCreator *creator) {
    GetLayerCreatorMap()[type] = std::shared_ptr<LayerAccCreator>(creator);
    return TNN_OK;
}
AbstractLayerAcc *RocmDevice::CreateLayerAcc(LayerType type) {
    auto &m = GetLayerCreatorMap();
    auto it = m.find(type);
    return it == m.end() ? nullptr : it->second->CreateLayerAcc(type);
}
Context *RocmDevice::CreateContext(int device_id) {
    auto ctx = new RocmContext(device_id);
    if (ctx->Setup() != TNN_OK) {
        delete ctx;
        return nullptr;
    }
    return ctx;
}
std::shared_ptr<const ImplementedPrecision> RocmDevice::GetImplementedPrecision(LayerType) {
    auto p               = std::make_shared<ImplementedPrecision>();
    p->fp32_implemented  = true;
    p->fp16_implemented  = true;
    p->bfp16_implemented = false;
    return p;
}
BlobMemorySizeInfo RocmDevice::Calculate(BlobDesc &desc) {
    // plain row-major ("NCHW" of any rank) in the blob's own data type; int8 blobs are NOT padded to
    // NHWC4 as on x86 (x86_device.cc:27-38): every channel count on this path is a multiple of 4
    // One-dimensional, as every linear-memory device reports it (abstract_device.cc Calculate1DMemorySize): the engine's
    // blob manager keeps one memory pool per number of size dimensions and only the 1-D pool exists off OpenCL
    // (blob_manager.cc:30-38, 160-175).
    BlobMemorySizeInfo info;
    info.data_type = desc.data_type;
    int64_t count  = 1;
    for (int d : desc.dims)
        count *= d > 0 ? d : 0;
    info.dims = {(int)(count > 0 ? count : 1)};
    return info;
}
Status RocmDevice::Allocate(void **handle, MatType mat_type, DimsVector dims) {
    BlobMemorySizeInfo info;
    info.data_type = mat_type == NCHW_FLOAT            ? DATA_TYPE_FLOAT
                     : mat_type == NC_INT32            ? DATA_TYPE_INT32
                     : mat_type == RESERVED_FP16_TEST  ? DATA_TYPE_HALF
                     : mat_type == RESERVED_BFP16_TEST ? DATA_TYPE_BFP16
                                                       : DATA_TYPE_INT8;
    // one dimension: the engine's byte count knows linear memory only in that form (blob_memory_size_info.cc:21-36 gives 0
    // for any other rank); the image Mat types hold one byte per element of dims
    int64_t count = 1;
    for (int d : dims)
        count *= d > 0 ? d : 0;
    if (count > INT32_MAX)
        return Status(TNNERR_PARAM_ERR, "mat with more than 2^31 elements");
    info.dims = {(int)(count > 0 ? count : 1)};
    return Allocate(handle, info);
}
Status RocmDevice::Allocate(void **handle, BlobMemorySizeInfo &size_info) {
    if (!handle)
        return Status(TNNERR_NULL_PARAM, "handle is nil");
    int64_t bytes = GetBlobMemoryBytesSize(size_info);
    if (bytes < 0)
        return Status(TNNERR_PARAM_ERR, "negative blob size");
    int rc = tnn_rocm_malloc(handle, (size_t)(bytes > 0 ? bytes : 16));
    if (rc != 0)
        return RocmStatus(rc, TNNERR_OUTOFMEMORY, "hipMalloc");
    return TNN_OK;
}
Status RocmDevice::Free(void *handle) {
    int rc = tnn_rocm_free(handle);
    return rc == 0 ? Status(TNN_OK) : RocmStatus(rc, TNNERR_COMMON_ERROR, "hipFree");
}
Status RocmDevice::CopyToDevice(BlobHandle *dst, const BlobHandle *src, BlobDesc &desc, void *q) {
    auto info  = Calculate(desc);
    int rc     = tnn_rocm_memcpy_h2d((char *)dst->base + dst->bytes_offset, (const char *)src->base + src->bytes_offset,
                                     (size_t)GetBlobMemoryBytesSize(info), q);
    return rc == 0 ? Status(TNN_OK) : RocmStatus(rc, TNNERR_CUDA_MEMCPY_ERROR, "host to device copy");
}
Status RocmDevice::CopyFromDevice(BlobHandle *dst, const BlobHandle *src, BlobDesc &desc, void *q) {
    auto info = Calculate(desc);
    int rc    = tnn_rocm_memcpy_d2h((char *)dst->base + dst->bytes_offset, (const char *)src->base + src->bytes_offset,
                                    (size_t)GetBlobMemoryBytesSize(info), q);
    return rc == 0 ? Status(TNN_OK) : RocmStatus(rc, TNNERR_CUDA_MEMCPY_ERROR, "device to host copy");
}

static TypeDeviceRegister<RocmDevice> g_rocm_device_register(DEVICE_ROCM);

// ---- layer acc base -----------------------------------------------------------------------------
RocmLayerAcc::~RocmLayerAcc() {
    for (void *p : owned_device_)
        tnn_rocm_free(p);
}
Status RocmLayerAcc::Init(Context *context, LayerParam *param, LayerResource *resource,
                          const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) {
    context_ = dynamic_cast<RocmContext *>(context);
    if (!context_)
        return Status(TNNERR_NULL_PARAM, "RocmLayerAcc needs a RocmContext");
    param_    = param;
    resource_ = resource;
    return ReloadConstantBlobs(inputs, false);
}
std::vector<DataFormat> RocmLayerAcc::SupportDataFormat(DataType, int, BlobType) {
    // row-major for every rank, as the naive device does (cpu_layer_acc.cc:70-78)
    return {DATA_FORMAT_NCHW};
}
DataType RocmLayerAcc::ConstantBlobDataType(const std::vector<Blob *> &inputs, int) {
    for (auto b : inputs)
        if (!b->IsConstant())
            return b->GetBlobDesc().data_type;
    return DATA_TYPE_FLOAT;
}
Status RocmLayerAcc::UploadConverted(const void *host, size_t count, DataType src, DataType dst, void **out) {
    size_t sb = (size_t)DataTypeUtils::GetBytesSize(src), db = (size_t)DataTypeUtils::GetBytesSize(dst);
    void *dev = nullptr;
    int rc    = tnn_rocm_malloc(&dev, count * db > 0 ? count * db : 16);
    if (rc != 0)
        return RocmStatus(rc, TNNERR_OUTOFMEMORY, "constant upload");
    owned_device_.push_back(dev);
    *out = dev;
    if (count == 0)
        return TNN_OK;
    if (src == dst) {
        ROCM_CALL(tnn_rocm_memcpy_h2d(dev, host, count * sb, Stream()));
        return TNN_OK;
    }
    bool s_float = src == DATA_TYPE_FLOAT || src == DATA_TYPE_HALF || src == DATA_TYPE_BFP16;
    bool d_float = dst == DATA_TYPE_FLOAT || dst == DATA_TYPE_HALF || dst == DATA_TYPE_BFP16;
    if (!s_float || !d_float)
        return Status(TNNERR_PARAM_ERR, "constant conversion between non-float types");
    void *tmp = nullptr;
    rc        = tnn_rocm_malloc(&tmp, count * sb);
    if (rc != 0)
        return RocmStatus(rc, TNNERR_OUTOFMEMORY, "constant staging");
    rc = tnn_rocm_memcpy_h2d(tmp, host, count * sb, Stream());
    if (rc == 0)
        rc = tnn_rocm_cast(Stream(), (int)src, tmp, (int)dst, dev, count);
    if (rc == 0)
        rc = tnn_rocm_stream_sync(Stream());
    tnn_rocm_free(tmp);
    return rc == 0 ? Status(TNN_OK) : RocmStatus(rc, TNNERR_CUDA_MEMCPY_ERROR, "constant conversion");
}
Status RocmLayerAcc::ReloadConstantBlobs(const std::vector<Blob *> &inputs, bool only_reload_shape_differ_blob) {
    if (!const_resource_ || only_reload_shape_differ_blob)
        return TNN_OK;
    for (int i = 0; i < (int)inputs.size(); ++i) {
        Blob *b   = inputs[i];
        auto it   = const_resource_->find(b->GetBlobDesc().name);
        if (it == const_resource_->end() || !b->IsConstant())
            continue;
        if (const_blob_map_.count(b->GetBlobDesc().name))
            continue;
        auto &buf    = *it->second;
        DataType dst = ConstantBlobDataType(inputs, i);
        if (buf.GetDataType() == DATA_TYPE_INT32 || buf.GetDataType() == DATA_TYPE_INT8)
            dst = buf.GetDataType();
        // a constant shared by several layers may need different storage types, so each acc keeps
        // its own device copy and publishes it through a blob of its own
        void *dev = nullptr;
        RETURN_ON_NEQ(UploadConverted(buf.force_to<void *>(), (size_t)buf.GetDataCount(), buf.GetDataType(), dst, &dev),
                      TNN_OK);
        BlobDesc desc  = b->GetBlobDesc();
        desc.data_type = dst;
        BlobHandle h;
        h.base = dev;
        const_blob_map_[desc.name] = std::make_shared<Blob>(desc, h);
    }
    return TNN_OK;
}

// ---- blob converter (role of source/tnn/device/cuda/cuda_blob_converter.cc:36-234) -------------------
class RocmBlobConverterAcc : public BlobConverterAcc {
public:
    explicit RocmBlobConverterAcc(Blob *blob) : BlobConverterAcc(blob) {}
    ~RocmBlobConverterAcc() override {
        tnn_rocm_free(staging_);
        tnn_rocm_free(params_);
        tnn_rocm_free_host(bounce_);
    }

    Status ConvertFromMat(Mat &mat, MatConvertParam param, void *q) override {
        RETURN_ON_NEQ(ConvertFromMatAsync(mat, param, q), TNN_OK);
        ROCM_CALL(tnn_rocm_stream_sync(q));
        return TNN_OK;
    }
    Status ConvertToMat(Mat &mat, MatConvertParam param, void *q) override {
        // the device-to-host copy below blocks until the data has arrived
        return ConvertToMatAsync(mat, param, q);
    }

    Status ConvertFromMatAsync(Mat &mat, MatConvertParam param, void *q) override {
        auto &desc   = blob_->GetBlobDesc();
        size_t count = (size_t)DimsVectorUtils::Count(desc.dims);
        if (mat.GetDeviceType() != DEVICE_NAIVE && mat.GetDeviceType() != DEVICE_ROCM)
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: the mat lives on another device");
        if ((size_t)DimsVectorUtils::Count(mat.GetDims()) != count)
            return Status(TNNERR_INVALID_INPUT, "mat and blob element counts differ");
        void *dst = (char *)blob_->GetHandle().base + blob_->GetHandle().bytes_offset;
        if (count == 0)
            return TNN_OK;
        if (mat.GetDeviceType() == DEVICE_ROCM)
            return FromDeviceMat(mat, param, dst, count, q);
        if (mat.GetMatType() == NC_INT32) {
            if (desc.data_type != DATA_TYPE_INT32)
                return Status(TNNERR_PARAM_ERR, "NC_INT32 mat needs an int32 blob");
            ROCM_CALL(tnn_rocm_memcpy_h2d(dst, mat.GetData(), count * 4, q));
            return TNN_OK;
        }
        if (mat.GetMatType() == RESERVED_INT8_TEST) {
            if (desc.data_type != DATA_TYPE_INT8)
                return Status(TNNERR_PARAM_ERR, "int8 mat needs an int8 blob");
            ROCM_CALL(tnn_rocm_memcpy_h2d(dst, mat.GetData(), count, q));
            return TNN_OK;
        }
        if (mat.GetMatType() == RESERVED_BFP16_TEST || mat.GetMatType() == RESERVED_FP16_TEST) {
            // host values that are bfloat16 / half already (how the engine's layer test feeds a half-precision blob:
            // layer_test.cc:266-275; blob_converter_default.cc:323-330): copied as they are into a blob of that type,
            // converted on the device into a float blob of another
            const DataType mt = mat.GetMatType() == RESERVED_BFP16_TEST ? DATA_TYPE_BFP16 : DATA_TYPE_HALF;
            if (desc.data_type != DATA_TYPE_FLOAT && desc.data_type != DATA_TYPE_HALF && desc.data_type != DATA_TYPE_BFP16)
                return Status(TNNERR_PARAM_ERR, "a half or bfloat16 mat needs a float blob");
            if (desc.data_type == mt) {
                ROCM_CALL(tnn_rocm_memcpy_h2d(dst, mat.GetData(), count * 2, q));
                return TNN_OK;
            }
            RETURN_ON_NEQ(Staging(count * 2), TNN_OK);
            ROCM_CALL(tnn_rocm_memcpy_h2d(staging_, mat.GetData(), count * 2, q));
            ROCM_CALL(tnn_rocm_cast(q, (int)mt, staging_, (int)desc.data_type, dst, count));
            return TNN_OK;
        }
        if (mat.GetMatType() != NCHW_FLOAT)
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported mat type");
        const float *src = (const float *)mat.GetData();
        std::vector<float> scaled;
        if (NeedsScaleBias(param, desc.dims)) {  // per-channel x*scale+bias over dims[1] (blob_converter_default.cc:281-291)
            scaled.resize(count);
            ApplyScaleBias(src, scaled.data(), desc.dims, param);
            src = scaled.data();
        }
        if (desc.data_type == DATA_TYPE_FLOAT) {
            ROCM_CALL(tnn_rocm_memcpy_h2d(dst, src, count * 4, q));
            return TNN_OK;
        }
        RETURN_ON_NEQ(Staging(count * 4), TNN_OK);
        ROCM_CALL(tnn_rocm_memcpy_h2d(staging_, src, count * 4, q));
        if (desc.data_type == DATA_TYPE_HALF || desc.data_type == DATA_TYPE_BFP16) {
            ROCM_CALL(tnn_rocm_cast(q, TNN_ROCM_F32, staging_, (int)desc.data_type, dst, count));
        } else if (desc.data_type == DATA_TYPE_INT8) {
            // float mat into an int8 blob goes through the blob's scale (blob_converter_default.cc:396-403),
            // with the reciprocal-multiply quantiser of the x86 path
            auto bi = dynamic_cast<BlobInt8 *>(blob_);
            if (!bi || !bi->GetIntResource() || bi->GetIntResource()->scale_handle.GetDataCount() < 1)
                return Status(TNNERR_NULL_PARAM, "int8 blob without scale resource");
            const int n_scale = bi->GetIntResource()->scale_handle.GetDataCount();
            const float *sc   = bi->GetIntResource()->scale_handle.force_to<float *>();
            if (n_scale > 1) {
                // one scale per channel (dims[1]), NaiveQuantBias's indexing (naive_compute.cc:1671-1690): a rare path
                // (model inputs are per-tensor as a rule), quantised on the host with the device quantiser's arithmetic
                // (multiply by float(1.0 / scale), add +-0.5, truncate, clamp) and copied as int8
                const int ch    = desc.dims.size() > 1 ? desc.dims[1] : 1;
                const size_t hw = (size_t)std::max(1, DimsVectorUtils::Count(desc.dims, 2));
                if (n_scale < ch)
                    return Status(TNNERR_PARAM_ERR, "int8 blob with fewer scales than channels");
                std::vector<int8_t> qv(count);
                for (size_t i = 0; i < count; ++i) {
                    const float s = sc[(i / hw) % (size_t)ch];
                    float v       = s != 0.f ? src[i] * (float)(1.0 / s) : 0.f;
                    v             = v < 0.f ? v - 0.5f : v + 0.5f;
                    v             = v > 127.f ? 127.f : (v < -128.f ? -128.f : v);
                    qv[i]         = (int8_t)(int)v;
                }
                ROCM_CALL(tnn_rocm_memcpy_h2d(dst, qv.data(), count, q));
                ROCM_CALL(tnn_rocm_stream_sync(q));  // the host vector goes away with this call
                return TNN_OK;
            }
            float s   = sc[0];
            float inv = (float)(1.0 / s);
            ROCM_CALL(tnn_rocm_quantize(q, TNN_ROCM_F32, staging_, inv, (int8_t *)dst, count));
        } else {
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported blob data type");
        }
        return TNN_OK;
    }

    Status ConvertToMatAsync(Mat &mat, MatConvertParam param, void *q) override {
        auto &desc   = blob_->GetBlobDesc();
        size_t count = (size_t)DimsVectorUtils::Count(desc.dims);
        if ((size_t)DimsVectorUtils::Count(mat.GetDims()) != count)
            return Status(TNNERR_INVALID_INPUT, "mat and blob element counts differ");
        void *src = (char *)blob_->GetHandle().base + blob_->GetHandle().bytes_offset;
        if (count == 0)
            return TNN_OK;
        if (mat.GetDeviceType() == DEVICE_ROCM)
            return ToDeviceMat(mat, param, src, count, q);
        if (mat.GetDeviceType() != DEVICE_NAIVE)
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: the mat lives on another device");
        if (mat.GetMatType() == NC_INT32 && desc.data_type == DATA_TYPE_INT32) {
            ROCM_CALL(tnn_rocm_memcpy_d2h(mat.GetData(), src, count * 4, q));
            return TNN_OK;
        }
        if (mat.GetMatType() == RESERVED_INT8_TEST && desc.data_type == DATA_TYPE_INT8) {
            ROCM_CALL(tnn_rocm_memcpy_d2h(mat.GetData(), src, count, q));
            return TNN_OK;
        }
        if (mat.GetMatType() == RESERVED_BFP16_TEST || mat.GetMatType() == RESERVED_FP16_TEST) {
            // the blob's values as bfloat16 / half on the host (blob_converter_default.cc:205-208, 245-249): copied from a
            // blob of that type, rounded to it on the device from a float blob of another
            const DataType mt = mat.GetMatType() == RESERVED_BFP16_TEST ? DATA_TYPE_BFP16 : DATA_TYPE_HALF;
            if (desc.data_type != DATA_TYPE_FLOAT && desc.data_type != DATA_TYPE_HALF && desc.data_type != DATA_TYPE_BFP16)
                return Status(TNNERR_PARAM_ERR, "a half or bfloat16 mat needs a float blob");
            if (desc.data_type == mt)
                return ToHost(mat.GetData(), src, count * 2, q);
            RETURN_ON_NEQ(Staging(count * 2), TNN_OK);
            ROCM_CALL(tnn_rocm_cast(q, (int)desc.data_type, src, (int)mt, staging_, count));
            return ToHost(mat.GetData(), staging_, count * 2, q);
        }
        if (mat.GetMatType() != NCHW_FLOAT)
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported mat type");
        if (desc.data_type == DATA_TYPE_INT32) {
            // an int32 blob read as a float Mat: the values converted, then scale and bias as for a float blob
            // (blob_converter_default.cc:213-221)
            std::vector<int32_t> iv(count);
            RETURN_ON_NEQ(ToHost(iv.data(), src, count * 4, q), TNN_OK);
            float *out = (float *)mat.GetData();
            for (size_t i = 0; i < count; ++i)
                out[i] = (float)iv[i];
        } else if (desc.data_type == DATA_TYPE_FLOAT) {
            RETURN_ON_NEQ(ToHost(mat.GetData(), src, count * 4, q), TNN_OK);
        } else if (desc.data_type == DATA_TYPE_HALF && count * 2 >= kBounceMinBytes && CpuWidensHalf()) {
            // a large half-precision blob crosses the bus as it is (half the bytes of its fp32 form) and is widened on
            // the way from the page-locked buffer into the Mat, which replaces the plain copy of that step
            RETURN_ON_NEQ(HalfToHostFloat((float *)mat.GetData(), src, count, q), TNN_OK);
        } else {
            RETURN_ON_NEQ(Staging(count * 4), TNN_OK);
            if (desc.data_type == DATA_TYPE_HALF || desc.data_type == DATA_TYPE_BFP16) {
                ROCM_CALL(tnn_rocm_cast(q, (int)desc.data_type, src, TNN_ROCM_F32, staging_, count));
            } else if (desc.data_type == DATA_TYPE_INT8) {
                auto bi = dynamic_cast<BlobInt8 *>(blob_);
                if (!bi || !bi->GetIntResource() || bi->GetIntResource()->scale_handle.GetDataCount() < 1)
                    return Status(TNNERR_NULL_PARAM, "int8 blob without scale resource");
                const int n_scale = bi->GetIntResource()->scale_handle.GetDataCount();
                const float *sc   = bi->GetIntResource()->scale_handle.force_to<float *>();
                if (n_scale > 1) {  // per-channel scales: NaiveDequant's indexing (naive_compute.cc:1617-1633), on the host
                    const int ch    = desc.dims.size() > 1 ? desc.dims[1] : 1;
                    const size_t hw = (size_t)std::max(1, DimsVectorUtils::Count(desc.dims, 2));
                    if (n_scale < ch)
                        return Status(TNNERR_PARAM_ERR, "int8 blob with fewer scales than channels");
                    std::vector<int8_t> qv(count);
                    RETURN_ON_NEQ(ToHost(qv.data(), src, count, q), TNN_OK);
                    float *out = (float *)mat.GetData();
                    for (size_t i = 0; i < count; ++i)
                        out[i] = sc[(i / hw) % (size_t)ch] * (float)qv[i];
                    if (NeedsScaleBias(param, desc.dims)) {
                        std::vector<float> tmp(count);
                        ApplyScaleBias(out, tmp.data(), desc.dims, param);
                        memcpy(out, tmp.data(), count * 4);
                    }
                    return TNN_OK;
                }
                float s = sc[0];
                ROCM_CALL(tnn_rocm_dequantize(q, (const int8_t *)src, s, TNN_ROCM_F32, staging_, count));
            } else {
                return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported blob data type");
            }
            RETURN_ON_NEQ(ToHost(mat.GetData(), staging_, count * 4, q), TNN_OK);
        }
        if (NeedsScaleBias(param, desc.dims)) {
            std::vector<float> tmp(count);
            ApplyScaleBias((const float *)mat.GetData(), tmp.data(), desc.dims, param);
            memcpy(mat.GetData(), tmp.data(), count * 4);
        }
        return TNN_OK;
    }

private:
    // ---- Mats whose memory is on this device (role of the DEVICE_CUDA branches of cuda_blob_converter.cc:62-81, 141-161):
    // nothing crosses the bus and nothing waits for the stream except the few bytes of scale and bias ----
    static bool IsFloatBlob(DataType t) { return t == DATA_TYPE_FLOAT || t == DATA_TYPE_HALF || t == DATA_TYPE_BFP16; }
    // per-channel x * scale + bias over dims[1], in place on fp32 device data: a multiply and an add with the operand
    // broadcast along every other axis (two roundings, as the host form has)
    Status ScaleBiasOnDevice(float *data, const DimsVector &dims, const MatConvertParam &p, void *q) {
        const int rank = (int)dims.size();
        if (rank < 1 || rank > 6)
            return Status(TNNERR_PARAM_ERR, "scale and bias on a device mat need a rank between 1 and 6");
        const int c = rank > 1 ? dims[1] : 1;
        std::vector<float> host(2 * (size_t)c);
        for (int j = 0; j < c; ++j) {
            host[j]     = j < (int)p.scale.size() ? p.scale[j] : 1.0f;
            host[c + j] = j < (int)p.bias.size() ? p.bias[j] : 0.0f;
        }
        if (host.size() * 4 > params_sz_) {
            tnn_rocm_free(params_);
            params_    = nullptr;
            params_sz_ = 0;
            int rc     = tnn_rocm_malloc(&params_, host.size() * 4);
            if (rc != 0)
                return RocmStatus(rc, TNNERR_OUTOFMEMORY, "converter scale and bias");
            params_sz_ = host.size() * 4;
        }
        ROCM_CALL(tnn_rocm_memcpy_h2d(params_, host.data(), host.size() * 4, q));  // returns when the bytes have left the vector
        DimsVector pd((size_t)rank, 1);
        if (rank > 1)
            pd[1] = c;
        const float *sc = (const float *)params_;
        ROCM_CALL(tnn_rocm_binary(q, TNN_ROCM_F32, 2, data, dims.data(), rank, sc, pd.data(), rank, data, dims.data(), rank));
        ROCM_CALL(tnn_rocm_binary(q, TNN_ROCM_F32, 0, data, dims.data(), rank, sc + c, pd.data(), rank, data, dims.data(), rank));
        return TNN_OK;
    }
    Status FromDeviceMat(Mat &mat, const MatConvertParam &param, void *dst, size_t count, void *q) {
        auto &desc      = blob_->GetBlobDesc();
        const void *src = mat.GetData();
        if (!src)
            return Status(TNNERR_NULL_PARAM, "device mat without memory");
        const MatType mt = mat.GetMatType();
        if (mt == NC_INT32 || mt == RESERVED_INT8_TEST) {
            const DataType want = mt == NC_INT32 ? DATA_TYPE_INT32 : DATA_TYPE_INT8;
            if (desc.data_type != want)
                return Status(TNNERR_PARAM_ERR, mt == NC_INT32 ? "NC_INT32 mat needs an int32 blob" : "int8 mat needs an int8 blob");
            ROCM_CALL(tnn_rocm_memcpy_d2d(dst, src, count * (mt == NC_INT32 ? 4 : 1), q));
            return TNN_OK;
        }
        if (mt == RESERVED_BFP16_TEST || mt == RESERVED_FP16_TEST) {
            const DataType half_type = mt == RESERVED_BFP16_TEST ? DATA_TYPE_BFP16 : DATA_TYPE_HALF;
            if (!IsFloatBlob(desc.data_type))
                return Status(TNNERR_PARAM_ERR, "a half or bfloat16 mat needs a float blob");
            if (desc.data_type == half_type)
                ROCM_CALL(tnn_rocm_memcpy_d2d(dst, src, count * 2, q));
            else
                ROCM_CALL(tnn_rocm_cast(q, (int)half_type, src, (int)desc.data_type, dst, count));
            return TNN_OK;
        }
        if (mt != NCHW_FLOAT)
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported mat type");
        const float *f = (const float *)src;
        if (NeedsScaleBias(param, desc.dims)) {  // the caller's Mat stays as it is: the scaled values go through the staging buffer
            RETURN_ON_NEQ(Staging(count * 4), TNN_OK);
            ROCM_CALL(tnn_rocm_memcpy_d2d(staging_, src, count * 4, q));
            RETURN_ON_NEQ(ScaleBiasOnDevice((float *)staging_, desc.dims, param, q), TNN_OK);
            f = (const float *)staging_;
        }
        if (desc.data_type == DATA_TYPE_FLOAT) {
            ROCM_CALL(tnn_rocm_memcpy_d2d(dst, f, count * 4, q));
        } else if (desc.data_type == DATA_TYPE_HALF || desc.data_type == DATA_TYPE_BFP16) {
            ROCM_CALL(tnn_rocm_cast(q, TNN_ROCM_F32, f, (int)desc.data_type, dst, count));
        } else if (desc.data_type == DATA_TYPE_INT8) {
            auto bi = dynamic_cast<BlobInt8 *>(blob_);
            if (!bi || !bi->GetIntResource() || bi->GetIntResource()->scale_handle.GetDataCount() < 1)
                return Status(TNNERR_NULL_PARAM, "int8 blob without scale resource");
            if (bi->GetIntResource()->scale_handle.GetDataCount() != 1)
                return Status(TNNERR_PARAM_ERR, "a device mat into an int8 blob needs a per-tensor blob scale");
            const float s = bi->GetIntResource()->scale_handle.force_to<float *>()[0];
            ROCM_CALL(tnn_rocm_quantize(q, TNN_ROCM_F32, f, (float)(1.0 / s), (int8_t *)dst, count));
        } else {
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported blob data type");
        }
        return TNN_OK;
    }
    Status ToDeviceMat(Mat &mat, const MatConvertParam &param, const void *src, size_t count, void *q) {
        auto &desc = blob_->GetBlobDesc();
        void *out  = mat.GetData();
        if (!out)
            return Status(TNNERR_NULL_PARAM, "device mat without memory");
        const MatType mt = mat.GetMatType();
        if (mt == NC_INT32 && desc.data_type == DATA_TYPE_INT32) {
            ROCM_CALL(tnn_rocm_memcpy_d2d(out, src, count * 4, q));
            return TNN_OK;
        }
        if (mt == RESERVED_INT8_TEST && desc.data_type == DATA_TYPE_INT8) {
            ROCM_CALL(tnn_rocm_memcpy_d2d(out, src, count, q));
            return TNN_OK;
        }
        if (mt == RESERVED_BFP16_TEST || mt == RESERVED_FP16_TEST) {
            const DataType half_type = mt == RESERVED_BFP16_TEST ? DATA_TYPE_BFP16 : DATA_TYPE_HALF;
            if (!IsFloatBlob(desc.data_type))
                return Status(TNNERR_PARAM_ERR, "a half or bfloat16 mat needs a float blob");
            if (desc.data_type == half_type)
                ROCM_CALL(tnn_rocm_memcpy_d2d(out, src, count * 2, q));
            else
                ROCM_CALL(tnn_rocm_cast(q, (int)desc.data_type, src, (int)half_type, out, count));
            return TNN_OK;
        }
        if (mt != NCHW_FLOAT)
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported mat type");
        if (desc.data_type == DATA_TYPE_FLOAT) {
            ROCM_CALL(tnn_rocm_memcpy_d2d(out, src, count * 4, q));
        } else if (desc.data_type == DATA_TYPE_HALF || desc.data_type == DATA_TYPE_BFP16 || desc.data_type == DATA_TYPE_INT32) {
            ROCM_CALL(tnn_rocm_cast(q, (int)desc.data_type, src, TNN_ROCM_F32, out, count));
        } else if (desc.data_type == DATA_TYPE_INT8) {
            auto bi = dynamic_cast<BlobInt8 *>(blob_);
            if (!bi || !bi->GetIntResource() || bi->GetIntResource()->scale_handle.GetDataCount() < 1)
                return Status(TNNERR_NULL_PARAM, "int8 blob without scale resource");
            if (bi->GetIntResource()->scale_handle.GetDataCount() != 1)
                return Status(TNNERR_PARAM_ERR, "an int8 blob into a device mat needs a per-tensor blob scale");
            const float s = bi->GetIntResource()->scale_handle.force_to<float *>()[0];
            ROCM_CALL(tnn_rocm_dequantize(q, (const int8_t *)src, s, TNN_ROCM_F32, out, count));
        } else {
            return Status(TNNERR_PARAM_ERR, "RocmBlobConverter: unsupported blob data type");
        }
        if (NeedsScaleBias(param, desc.dims))
            RETURN_ON_NEQ(ScaleBiasOnDevice((float *)out, desc.dims, param, q), TNN_OK);
        return TNN_OK;
    }

    static bool NeedsScaleBias(const MatConvertParam &p, const DimsVector &dims) {
        for (float s : p.scale)
            if (s != 1.0f)
                return true;
        for (float b : p.bias)
            if (b != 0.0f)
                return true;
        (void)dims;
        return false;
    }
    static void ApplyScaleBias(const float *src, float *dst, const DimsVector &dims, const MatConvertParam &p) {
        int n = dims.size() > 0 ? dims[0] : 1, c = dims.size() > 1 ? dims[1] : 1;
        int hw = DimsVectorUtils::Count(dims, 2);
        for (int i = 0; i < n; ++i)
            for (int j = 0; j < c; ++j) {
                float s = j < (int)p.scale.size() ? p.scale[j] : 1.0f;
                float b = j < (int)p.bias.size() ? p.bias[j] : 0.0f;
                for (int k = 0; k < hw; ++k) {
                    size_t o = ((size_t)i * c + j) * hw + k;
                    dst[o]   = src[o] * s + b;
                }
            }
    }
    Status Staging(size_t bytes) {
        if (bytes > staging_sz_) {
            tnn_rocm_free(staging_);
            staging_    = nullptr;
            staging_sz_ = 0;
            int rc      = tnn_rocm_malloc(&staging_, bytes);
            if (rc != 0)
                return RocmStatus(rc, TNNERR_OUTOFMEMORY, "converter staging");
            staging_sz_ = bytes;
        }
        return TNN_OK;
    }
    Status Bounce(size_t bytes) {
        if (bytes > bounce_sz_) {
            tnn_rocm_free_host(bounce_);
            bounce_    = nullptr;
            bounce_sz_ = 0;
            int rc     = tnn_rocm_malloc_host(&bounce_, bytes);
            if (rc != 0)
                return RocmStatus(rc, TNNERR_OUTOFMEMORY, "converter page-locked buffer");
            bounce_sz_ = bytes;
        }
        return TNN_OK;
    }
    static bool CpuWidensHalf() {
        static const bool yes = __builtin_cpu_supports("f16c") && __builtin_cpu_supports("avx");
        return yes;
    }
    // IEEE half -> float (exact) with the CPU's conversion instruction, eight at a time; without it the blob is widened on
    // the device and crosses the bus as fp32 (the branch above)
    __attribute__((target("avx,f16c"))) static void WidenF16C(const uint16_t *s, float *d, size_t n) {
        size_t i = 0;
        for (; i + 8 <= n; i += 8)
            _mm256_storeu_ps(d + i, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(s + i))));
        for (; i < n; ++i)
            d[i] = _cvtsh_ss(s[i]);
    }
    Status HalfToHostFloat(float *host_dst, const void *dev_src, size_t count, void *q) {
        RETURN_ON_NEQ(Bounce(count * 2), TNN_OK);
        ROCM_CALL(tnn_rocm_memcpy_d2h(bounce_, dev_src, count * 2, q));
        const int parts = 4;
#pragma omp parallel for num_threads(parts) schedule(static)
        for (int i = 0; i < parts; ++i) {
            size_t lo = (count / parts * i) & ~(size_t)31, hi = i + 1 == parts ? count : (count / parts * (i + 1)) & ~(size_t)31;
            WidenF16C((const uint16_t *)bounce_ + lo, host_dst + lo, hi - lo);
        }
        return TNN_OK;
    }
    // Device to host.  A Mat's memory is pageable, and a copy into pageable memory is staged by the runtime in small
    // pieces on one thread (about 8 GB/s: 1.1 ms for the 9.4 MB fp32 output of a batch-8 encoder).  Large outputs
    // therefore go by DMA into a page-locked buffer the converter keeps, and from there into the Mat on a few threads.
    Status ToHost(void *host_dst, const void *dev_src, size_t bytes, void *q) {
        if (bytes < kBounceMinBytes) {
            ROCM_CALL(tnn_rocm_memcpy_d2h(host_dst, dev_src, bytes, q));
            return TNN_OK;
        }
        RETURN_ON_NEQ(Bounce(bytes), TNN_OK);
        ROCM_CALL(tnn_rocm_memcpy_d2h(bounce_, dev_src, bytes, q));
        const int parts = bytes >= (4u << 20) ? 4 : 2;
#pragma omp parallel for num_threads(parts) schedule(static)
        for (int i = 0; i < parts; ++i) {
            size_t lo = (bytes / parts * i) & ~(size_t)63, hi = i + 1 == parts ? bytes : (bytes / parts * (i + 1)) & ~(size_t)63;
            memcpy((char *)host_dst + lo, (const char *)bounce_ + lo, hi - lo);
        }
        return TNN_OK;
    }
    static constexpr size_t kBounceMinBytes = 1u << 20;
    void *staging_     = nullptr;
    size_t staging_sz_ = 0;
    void *bounce_      = nullptr;
    size_t bounce_sz_  = 0;
    void *params_      = nullptr;  // scale and bias of a device mat's conversion, on the device
    size_t params_sz_  = 0;
};

// ---- Mat converter (role of source/tnn/device/cuda/cuda_mat_converter.cc): MatUtils::Copy between a host Mat and a
// DEVICE_ROCM Mat, or between two DEVICE_ROCM Mats.  The image operations (resize, crop, warp, colour conversion, border)
// prepare camera frames for vision models and are not part of this backend. ----
class RocmMatConverterAcc : public MatConverterAcc {
public:
    Status Copy(Mat &src, Mat &dst, void *command_queue = nullptr) override {
        if (!src.GetData() || !dst.GetData())
            return Status(TNNERR_NULL_PARAM, "mat without memory");
        if (src.GetMatType() != dst.GetMatType())
            return Status(TNNERR_PARAM_ERR, "src and dst have different mat types");
        size_t elem = 0;
        switch (src.GetMatType()) {
            case NCHW_FLOAT:
            case NC_INT32: elem = 4; break;
            case RESERVED_BFP16_TEST:
            case RESERVED_FP16_TEST: elem = 2; break;
            case RESERVED_INT8_TEST:
            case N8UC3:
            case N8UC4:
            case NGRAY: elem = 1; break;
            default: return Status(TNNERR_PARAM_ERR, "RocmMatConverter: mat type without a plain element layout");
        }
        const size_t bytes = (size_t)DimsVectorUtils::Count(src.GetDims()) * elem;
        if ((size_t)DimsVectorUtils::Count(dst.GetDims()) * elem != bytes)
            return Status(TNNERR_PARAM_ERR, "src and dst dims not equal");
        const bool src_dev = src.GetDeviceType() == DEVICE_ROCM, dst_dev = dst.GetDeviceType() == DEVICE_ROCM;
        if (src_dev && dst_dev) {
            ROCM_CALL(tnn_rocm_memcpy_d2d(dst.GetData(), src.GetData(), bytes, command_queue));
            ROCM_CALL(tnn_rocm_stream_sync(command_queue));
        } else if (dst_dev) {
            ROCM_CALL(tnn_rocm_memcpy_h2d(dst.GetData(), src.GetData(), bytes, command_queue));  // waits for the stream
        } else if (src_dev) {
            ROCM_CALL(tnn_rocm_memcpy_d2h(dst.GetData(), src.GetData(), bytes, command_queue));
        } else {
            return Status(TNNERR_PARAM_ERR, "RocmMatConverter: neither mat is on DEVICE_ROCM");
        }
        return TNN_OK;
    }
    Status Resize(Mat &, Mat &, ResizeParam, void * = nullptr) override { return NotBuilt("Resize"); }
    Status Crop(Mat &, Mat &, CropParam, void * = nullptr) override { return NotBuilt("Crop"); }
    Status WarpAffine(Mat &, Mat &, WarpAffineParam, void * = nullptr) override { return NotBuilt("WarpAffine"); }
    Status CvtColor(Mat &, Mat &, ColorConversionType, void * = nullptr) override { return NotBuilt("CvtColor"); }
    Status CopyMakeBorder(Mat &, Mat &, CopyMakeBorderParam, void * = nullptr) override { return NotBuilt("CopyMakeBorder"); }

private:
    static Status NotBuilt(const char *what) {
        return Status(TNNERR_PARAM_ERR, std::string("RocmMatConverter: ") + what + " (image preparation) is not part of DEVICE_ROCM");
    }
};
DECLARE_MAT_CONVERTER_CREATER(Rocm);
REGISTER_MAT_CONVERTER(Rocm, DEVICE_ROCM);

DECLARE_BLOB_CONVERTER_CREATER(Rocm);
REGISTER_BLOB_CONVERTER(Rocm, DEVICE_ROCM);

}  // namespace TNN_NS
