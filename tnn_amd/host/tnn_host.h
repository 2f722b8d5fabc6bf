// Host-side engine surface for the DEVICE_ROCM backend.
//
// The backend classes (RocmDevice, RocmContext, Rocm*LayerAcc, RocmBlobConverterAcc) are written
// against the engine's plug-in contract: AbstractDevice / Context / AbstractLayerAcc with static
// registration.  This header declares that contract with the engine's own names, member signatures
// and error codes so the backend sources stay source-compatible with the engine tree, and adds the
// minimum host around it (model interpreter, layers with shape inference, network, instance) needed
// to run unchanged .tnnproto / .tnnmodel files when the engine itself is not linked.
//
// Reference declarations mirrored here (paths relative to the reference tree):
//   Status / error codes      include/tnn/core/status.h:29-162
//   DataType, DeviceType ...  include/tnn/core/common.h:31-197
//   BlobDesc / BlobHandle     include/tnn/core/blob.h:32-92 ; BlobInt8  source/tnn/core/blob_int8.h:24-40
//   RawBuffer                 source/tnn/interpreter/raw_buffer.h:30-71
//   LayerParam structs        source/tnn/interpreter/layer_param.h
//   LayerResource structs     source/tnn/interpreter/layer_resource.h:35-173
//   NetStructure/NetResource  source/tnn/interpreter/net_structure.h:34-66, net_resource.h:24-47
//   AbstractDevice            source/tnn/core/abstract_device.h:40-121
//   Context                   source/tnn/core/context.h:29-95
//   AbstractLayerAcc          source/tnn/core/abstract_layer_acc.h:39-143
//   BlobConverterAcc          source/tnn/utils/blob_converter_internal.h:27-81
//   Instance                  include/tnn/core/instance.h:42-144
#ifndef TNN_AMD_HOST_TNN_HOST_H_
#define TNN_AMD_HOST_TNN_HOST_H_

#include <cstdint>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#define TNN_NS tnn

namespace TNN_NS {

// ---- status -----------------------------------------------------------------------------------
enum StatusCode {
    TNN_OK                                    = 0x0,
    TNNERR_PARAM_ERR                          = 0x1000,
    TNNERR_INVALID_NETCFG                     = 0x1002,
    TNNERR_NULL_PARAM                         = 0x1004,
    TNNERR_NET_ERR                            = 0x2000,
    TNNERR_UNSUPPORT_NET                      = 0x2001,
    TNNERR_LAYER_ERR                          = 0x3000,
    TNNERR_UNKNOWN_LAYER                      = 0x3001,
    TNNERR_CREATE_LAYER                       = 0x3002,
    TNNERR_INIT_LAYER                         = 0x3003,
    TNNERR_MODEL_ERR                          = 0x4000,
    TNNERR_INVALID_MODEL                      = 0x4001,
    TNNERR_INST_ERR                           = 0x5000,
    TNNERR_COMMON_ERROR                       = 0x6000,
    TNNERR_OUTOFMEMORY                        = 0x6001,
    TNNERR_INVALID_INPUT                      = 0x6002,
    TNNERR_NO_RESULT                          = 0x6004,
    TNNERR_LOAD_MODEL                         = 0x6005,
    TNNERR_DEVICE_NOT_SUPPORT                 = 0x9000,
    TNNERR_DEVICE_CONTEXT_CREATE              = 0x9002,
    TNNERR_DEVICE_INVALID_COMMAND_QUEUE       = 0x9003,
    TNNERR_DEVICE_ACC_DATA_FORMAT_NOT_SUPPORT = 0x9004,
    // the GPU-runtime codes the CUDA backend uses, reused for HIP failures
    TNNERR_CUDA_SYNC_ERROR          = 0xF002,
    TNNERR_CUDA_MEMCPY_ERROR        = 0xF003,
    TNNERR_CUDA_KERNEL_LAUNCH_ERROR = 0xF004,
};

class Status {
public:
    Status(int code = TNN_OK, std::string message = "") : code_(code), message_(std::move(message)) {}
    Status &operator=(int code) {
        code_ = code;
        message_.clear();
        return *this;
    }
    bool operator==(int code) const { return code_ == code; }
    bool operator!=(int code) const { return code_ != code; }
    operator int() const { return code_; }
    operator bool() const { return code_ == TNN_OK; }
    std::string description() const;

private:
    int code_;
    std::string message_;
};

#define RETURN_ON_NEQ(expr, expected)                                                                                 \
    do {                                                                                                              \
        auto _status = (expr);                                                                                        \
        if (_status != (expected))                                                                                    \
            return _status;                                                                                           \
    } while (0)
#define CHECK_PARAM_NULL(p)                                                                                           \
    do {                                                                                                              \
        if (!(p))                                                                                                     \
            return Status(TNNERR_NULL_PARAM, "Error: param is nil");                                                  \
    } while (0)

// ---- enums ------------------------------------------------------------------------------------
typedef enum {
    DATA_TYPE_AUTO  = -1,
    DATA_TYPE_FLOAT = 0,
    DATA_TYPE_HALF  = 1,
    DATA_TYPE_INT8  = 2,
    DATA_TYPE_INT32 = 3,
    DATA_TYPE_BFP16 = 4,
    DATA_TYPE_INT64 = 5,
    DATA_TYPE_UINT32 = 6
} DataType;

typedef enum {
    DATA_FORMAT_AUTO   = -1,
    DATA_FORMAT_NCHW   = 0,
    DATA_FORMAT_NHWC   = 1,
    DATA_FORMAT_NHWC4  = 2,
    DATA_FORMAT_NC2HW2 = 3,
    DATA_FORMAT_NC4HW4 = 4,
    DATA_FORMAT_NC8HW8 = 5,
    DATA_FORMAT_NC16HW16 = 6,
    DATA_FORMAT_NCDHW  = 7,
    DATA_FORMAT_NHC4W4 = 8,
    DATA_FORMAT_CNH4   = 1000,
} DataFormat;

typedef enum {
    PRECISION_AUTO   = -1,  // fp16 activations where the device implements them (the ROCm backend does)
    PRECISION_NORMAL = 0,
    PRECISION_HIGH   = 1,   // fp32 everywhere
    PRECISION_LOW    = 2,
} Precision;

typedef enum { NETWORK_TYPE_AUTO = -1, NETWORK_TYPE_DEFAULT = 0, NETWORK_TYPE_TENSORRT = 0x8000 } NetworkType;  // the engine's smallest and largest values: the enum's range is the engine's

typedef enum {
    DEVICE_NAIVE = 0x0000,
    DEVICE_X86   = 0x0010,
    DEVICE_ARM   = 0x0020,
    DEVICE_CUDA  = 0x1020,
} DeviceType;  // DEVICE_ROCM is added by rocm_engine_additions.h, as it is inside the engine tree

typedef enum { MODEL_TYPE_TNN = 0x0001 } ModelType;

typedef enum {
    INVALID            = -1,
    N8UC3              = 0x00,
    N8UC4              = 0x01,
    NGRAY              = 0x10,
    NNV21              = 0x11,
    NNV12              = 0x12,
    NCHW_FLOAT         = 0x20,
    NC_INT32           = 0x21,
    RESERVED_BFP16_TEST = 0x200,
    RESERVED_FP16_TEST  = 0x201,
    RESERVED_INT8_TEST  = 0x202,
} MatType;

using DimsVector = std::vector<int>;

struct NetworkConfig {
    DeviceType device_type   = DEVICE_ARM;  // include/tnn/core/common.h:148
    int device_id            = 0;
    DataFormat data_format   = DATA_FORMAT_AUTO;
    NetworkType network_type = NETWORK_TYPE_AUTO;
    Precision precision      = PRECISION_AUTO;
    std::vector<std::string> library_path;
    std::string cache_path;
    bool enable_tune_kernel = false;
};

struct ModelConfig {
    ModelType model_type = MODEL_TYPE_TNN;
    // params[0] = proto text, params[1] = model bytes
    std::vector<std::string> params;
};

struct DimsVectorUtils {
    static int Count(const DimsVector &dims, int start = 0, int end = -1);
    static bool Equal(const DimsVector &a, const DimsVector &b);
};
struct DataTypeUtils {
    static int GetBytesSize(DataType dt);
};

// ---- blobs ------------------------------------------------------------------------------------
struct BlobDesc {
    DeviceType device_type = DEVICE_NAIVE;
    DataType data_type     = DATA_TYPE_FLOAT;
    DataFormat data_format = DATA_FORMAT_AUTO;
    DimsVector dims;
    std::string name = "";
};

struct BlobHandle {
    void *base            = nullptr;
    uint64_t bytes_offset = 0;
};

class Blob {
public:
    explicit Blob(BlobDesc desc) : desc_(std::move(desc)) {}
    Blob(BlobDesc desc, BlobHandle handle) : desc_(std::move(desc)), handle_(handle) {}
    virtual ~Blob() {}
    BlobDesc &GetBlobDesc() { return desc_; }
    void SetBlobDesc(BlobDesc desc) { desc_ = std::move(desc); }
    BlobHandle GetHandle() { return handle_; }
    void SetHandle(BlobHandle handle) { handle_ = handle; }
    bool IsConstant() const { return constant_; }
    void SetConstant(bool c) { constant_ = c; }

private:
    BlobDesc desc_;
    BlobHandle handle_;
    bool constant_ = false;
};

using BlobMap        = std::map<std::string, Blob *>;
using InputShapesMap = std::map<std::string, DimsVector>;
using InputDataTypeMap = std::map<std::string, DataType>;

// ---- raw buffers and resources ----------------------------------------------------------------
class RawBuffer {
public:
    RawBuffer() {}
    explicit RawBuffer(int bytes) : buff_(new char[bytes > 0 ? bytes : 1](), std::default_delete<char[]>()), bytes_(bytes) {}
    RawBuffer(int bytes, DimsVector dims) : RawBuffer(bytes) { dims_ = std::move(dims); }
    void SetDataType(DataType dt) { data_type_ = dt; }
    DataType GetDataType() const { return data_type_; }
    void SetBufferDims(DimsVector dims) { dims_ = std::move(dims); }
    DimsVector GetBufferDims() const { return dims_; }
    int GetBytesSize() const { return bytes_; }
    int GetDataCount() const {
        int es = DataTypeUtils::GetBytesSize(data_type_);
        return es > 0 ? bytes_ / es : 0;
    }
    template <typename T> T force_to() const { return reinterpret_cast<T>(buff_.get()); }

private:
    std::shared_ptr<char> buff_;
    int bytes_          = 0;
    DataType data_type_ = DATA_TYPE_FLOAT;
    DimsVector dims_;
};

struct LayerResource {
    std::string name = "";
    virtual ~LayerResource() {}
};
struct InnerProductLayerResource : public LayerResource {
    RawBuffer weight_handle;  // [num_output, K] row-major
    RawBuffer bias_handle;
    RawBuffer scale_handle;   // int8: per-output-channel (or single) weight scale
    RawBuffer zero_point_handle;
};
struct MatMulLayerResource : public LayerResource {
    RawBuffer weight;  // [K, N] for weight_position 1
    RawBuffer scale_handle;
};
struct EltwiseLayerResource : public LayerResource {
    RawBuffer element_handle;
    DimsVector element_shape;
};
struct GatherLayerResource : public LayerResource {
    RawBuffer data;
    RawBuffer indices;
    RawBuffer scale_data;
};
struct IntScaleResource : public LayerResource {
    RawBuffer scale_handle;
    RawBuffer zero_point_handle;
    RawBuffer bias_handle;
};
using ConstantResource = std::map<std::string, std::shared_ptr<RawBuffer>>;

class BlobInt8 : public Blob {
public:
    BlobInt8(BlobDesc desc, BlobHandle handle) : Blob(std::move(desc), handle) {}
    IntScaleResource *GetIntResource() { return resource_; }
    void SetIntResource(IntScaleResource *r) { resource_ = r; }

private:
    IntScaleResource *resource_ = nullptr;
};

// ---- layer types and params -------------------------------------------------------------------
enum LayerType {
    LAYER_NOT_SUPPORT   = 0,
    LAYER_RESHAPE       = 9,
    LAYER_INNER_PRODUCT = 19,
    LAYER_SOFTMAX       = 21,
    LAYER_PERMUTE       = 32,
    LAYER_ADD           = 38,
    LAYER_TANH          = 39,
    LAYER_MUL           = 42,
    LAYER_CAST          = 103,
    LAYER_GATHER        = 104,
    LAYER_MATMUL        = 105,
    LAYER_SUB           = 108,
    LAYER_SQUEEZE       = 118,
    LAYER_UNSQUEEZE     = 164,
    LAYER_REFORMAT      = 170,
    LAYER_DIV           = 175,
    LAYER_LAYER_NORM    = 326,
    LAYER_GELU          = 327,
    LAYER_BLOB_SCALE    = 600,
    LAYER_ANY_TYPE      = 1001,  // the engine's largest value (layer_type.h:243): the enum's range is the engine's
};
LayerType GlobalConvertLayerType(std::string type_str);

struct LayerParam {
    virtual ~LayerParam() {}
    std::string type;
    std::string name;
    bool quantized               = false;
    bool dynamic_range_quantized = false;
};
struct InnerProductLayerParam : public LayerParam {
    int num_output = 0;
    int has_bias   = 0;
    int transpose  = 0;
    int axis       = 0;
};
struct MatMulLayerParam : public LayerParam {
    int weight_position = -1;
    DimsVector matrix_a_dims;
    DimsVector matrix_b_dims;
    int axis = 0;
};
struct MultidirBroadcastLayerParam : public LayerParam {
    int weight_input_index = 1;
};
struct SoftmaxLayerParam : public LayerParam {
    int axis = 1;
};
struct LayerNormLayerParam : public LayerParam {
    int reduce_dims_size = 0;
    float eps            = 1e-5f;
};
struct ReshapeLayerParam : public LayerParam {
    int reshape_type = 0;
    int axis         = 0;
    int num_axes     = 0;
    std::vector<int> shape;
};
struct SqueezeLayerParam : public LayerParam {  // interpreter/layer_param.h:570-580 (Unsqueeze uses the same fields)
    std::vector<int> axes;
};
struct PermuteLayerParam : public LayerParam {
    std::vector<int> orders;
};
struct CastLayerParam : public LayerParam {
    int to   = 0;
    int from = 0;
};
typedef enum {  // layer_param.h:446-466; the accs set it from src_type / dst_type (x86_reformat_layer_acc.cc:32-44)
    QUANT_ONLY   = 0,
    DEQUANT_ONLY = 1,
    QUANT_NCHW4_2_NHWC   = 2,
    DEQUANT_NHWC_2_NCHW4 = 3,
    NC4HW4FP32_2_NC8HW8FP16 = 4,
    NC8HW8FP16_2_NC4HW4FP32 = 5,
    NC4HW4FP32_2_NCHWFP32 = 6,
    NCHWFP32_2_NC4HW4FP32 = 7,
    NC8HW8FP16_2_NCHWFP16 = 8,
    NCHWFP16_2_NC8HW8FP16 = 9,
    NC4HW4INT32_2_NCHWINT32 = 10,
    NCHWINT32_2_NC4HW4INT32 = 11,
} ReformatType;
struct ReformatLayerParam : public LayerParam {
    DataType src_type     = DATA_TYPE_AUTO;
    DataType dst_type     = DATA_TYPE_AUTO;
    DataFormat src_format = DATA_FORMAT_AUTO;
    DataFormat dst_format = DATA_FORMAT_AUTO;
    ReformatType type     = QUANT_ONLY;
};
struct GatherLayerParam : public LayerParam {
    int axis                 = 0;
    bool data_in_resource    = false;
    bool indices_in_resource = true;
};
struct LayerInfo {
    LayerType type = LAYER_NOT_SUPPORT;
    std::string type_str;
    std::string name;
    std::vector<std::string> inputs;
    std::vector<std::string> outputs;
    std::shared_ptr<LayerParam> param;
};

struct NetStructure {
    InputShapesMap inputs_shape_map;
    InputDataTypeMap input_data_type_map;
    std::set<std::string> outputs;
    std::vector<std::shared_ptr<LayerInfo>> layers;
    std::set<std::string> blobs;
};
struct NetResource {
    std::map<std::string, std::shared_ptr<LayerResource>> resource_map;
    ConstantResource constant_map;
};

// Parses the text proto and the binary model into a NetStructure / NetResource
// (source/tnn/interpreter/tnn/model_interpreter.cc:104-476).
class ModelInterpreter {
public:
    Status Interpret(std::vector<std::string> &params);
    NetStructure *GetNetStructure() { return &structure_; }
    NetResource *GetNetResource() { return &resource_; }

private:
    Status InterpretProto(const std::string &content);
    Status InterpretModel(const std::string &content);
    NetStructure structure_;
    NetResource resource_;
    uint32_t version_magic_number_ = 0;
};

// ---- the plug-in contract ---------------------------------------------------------------------
struct BlobMemorySizeInfo {
    DataType data_type = DATA_TYPE_FLOAT;
    std::vector<int> dims;
};
int64_t GetBlobMemoryBytesSize(BlobMemorySizeInfo &size_info);

class Context {
public:
    virtual ~Context() {}
    virtual Status LoadLibrary(std::vector<std::string> path) = 0;
    virtual Status GetCommandQueue(void **command_queue)      = 0;
    virtual Status ShareCommandQueue(Context *context) { return Status(TNNERR_COMMON_ERROR, "not supported"); }
    virtual Status OnInstanceForwardBegin() { return TNN_OK; }
    virtual Status OnInstanceForwardEnd() = 0;
    virtual Status OnInstanceReshapeBegin() { return TNN_OK; }
    virtual Status OnInstanceReshapeEnd() { return TNN_OK; }
    virtual Status Synchronize() = 0;
    virtual Status SetNumThreads(int) { return TNN_OK; }
    void SetPrecision(Precision p) { precision_ = p; }
    Precision GetPrecision() { return precision_; }

protected:
    Precision precision_ = PRECISION_AUTO;
};

enum BlobType { BLOB_INPUT = 0, BLOB_OUTPUT = 1 };

class AbstractLayerAcc {
public:
    virtual ~AbstractLayerAcc() {}
    virtual Status Init(Context *context, LayerParam *param, LayerResource *resource,
                        const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs)          = 0;
    virtual Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs)       = 0;
    virtual Status Forward(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs)       = 0;
    virtual Status BeforeForward(const std::vector<Blob *> &, const std::vector<Blob *> &) { return TNN_OK; }
    virtual Status AfterForward(const std::vector<Blob *> &, const std::vector<Blob *> &) { return TNN_OK; }
    virtual Status ReloadConstantBlobs(const std::vector<Blob *> &inputs, bool only_reload_shape_differ_blob = false) {
        return TNN_OK;
    }
    virtual Status ResolveBlobDataFormat(Blob *blob, BlobType blob_type);
    void SetConstantResource(ConstantResource *consts) { const_resource_ = consts; }

private:
    virtual std::vector<DataFormat> SupportDataFormat(DataType data_type, int dims_size, BlobType blob_type) = 0;

protected:
    ConstantResource *const_resource_ = nullptr;
    std::map<std::string, std::shared_ptr<Blob>> const_blob_map_;
};

class LayerAccCreator {
public:
    virtual AbstractLayerAcc *CreateLayerAcc(LayerType layer_type) = 0;
    virtual ~LayerAccCreator() {}
};
template <typename T> class TypeLayerAccCreator : public LayerAccCreator {
    AbstractLayerAcc *CreateLayerAcc(LayerType) { return new T(); }
};

struct ImplementedPrecision {
    bool fp32_implemented  = false;
    bool fp16_implemented  = false;
    bool bfp16_implemented = false;
};

class AbstractDevice {
public:
    explicit AbstractDevice(DeviceType t) : device_type_(t) {}
    virtual ~AbstractDevice() {}
    virtual BlobMemorySizeInfo Calculate(BlobDesc &desc)                               = 0;
    virtual Status Allocate(void **handle, MatType mat_type, DimsVector dims)          = 0;
    virtual Status Allocate(void **handle, BlobMemorySizeInfo &size_info)              = 0;
    virtual Status Allocate(BlobHandle *handle, BlobMemorySizeInfo &size_info);
    virtual Status Free(void *handle)                                                  = 0;
    virtual Status CopyToDevice(BlobHandle *dst, const BlobHandle *src, BlobDesc &desc, void *command_queue)   = 0;
    virtual Status CopyFromDevice(BlobHandle *dst, const BlobHandle *src, BlobDesc &desc, void *command_queue) = 0;
    virtual AbstractLayerAcc *CreateLayerAcc(LayerType type)                           = 0;
    virtual Context *CreateContext(int device_id)                                      = 0;
    virtual std::shared_ptr<const ImplementedPrecision> GetImplementedPrecision(LayerType type);
    virtual NetworkType ConvertAutoNetworkType()                                       = 0;
    DeviceType GetDeviceType() { return device_type_; }

private:
    DeviceType device_type_;
};

std::map<DeviceType, std::shared_ptr<AbstractDevice>> &GetGlobalDeviceMap();
AbstractDevice *GetDevice(DeviceType type);

template <typename T> class TypeDeviceRegister {
public:
    explicit TypeDeviceRegister(DeviceType type) {
        auto &device_map = GetGlobalDeviceMap();
        if (device_map.find(type) == device_map.end())
            device_map[type] = std::shared_ptr<T>(new T(type));
    }
};

// ---- Mat and blob conversion --------------------------------------------------------------------
class Mat {
public:
    Mat(DeviceType device_type, MatType mat_type, DimsVector dims, void *data)
        : device_type_(device_type), mat_type_(mat_type), data_(data), dims_(std::move(dims)) {}
    Mat(DeviceType device_type, MatType mat_type, DimsVector dims);  // allocates: host memory, or the device's through AbstractDevice::Allocate
    DeviceType GetDeviceType() { return device_type_; }
    MatType GetMatType() { return mat_type_; }
    void *GetData() { return data_; }
    DimsVector GetDims() { return dims_; }

private:
    DeviceType device_type_;
    MatType mat_type_;
    void *data_ = nullptr;
    DimsVector dims_;
    std::shared_ptr<char> owned_;
};

struct MatConvertParam {
    std::vector<float> scale = {1.0f, 1.0f, 1.0f, 1.0f};
    std::vector<float> bias  = {0.0f, 0.0f, 0.0f, 0.0f};
    bool reverse_channel     = false;
};

class BlobConverterAcc {
public:
    explicit BlobConverterAcc(Blob *blob) : blob_(blob) {}
    virtual ~BlobConverterAcc() {}
    virtual Status ConvertToMat(Mat &image, MatConvertParam param, void *command_queue = nullptr)        = 0;
    virtual Status ConvertToMatAsync(Mat &image, MatConvertParam param, void *command_queue = nullptr)   = 0;
    virtual Status ConvertFromMat(Mat &image, MatConvertParam param, void *command_queue = nullptr)      = 0;
    virtual Status ConvertFromMatAsync(Mat &image, MatConvertParam param, void *command_queue = nullptr) = 0;

protected:
    Blob *blob_ = nullptr;
};
class BlobConverterAccCreater {
public:
    virtual ~BlobConverterAccCreater() {}
    virtual std::shared_ptr<BlobConverterAcc> CreateBlobConverterAcc(Blob *blob) = 0;
};
// utils/blob_converter_internal.h:46-81: the per-device creator registry and its registration macros
class BlobConverterManager {
public:
    static std::shared_ptr<BlobConverterManager> &Shared();
    std::shared_ptr<BlobConverterAcc> CreateBlobConverterAcc(Blob *blob);
    int RegisterBlobConverterAccCreater(DeviceType type, std::shared_ptr<BlobConverterAccCreater> creater);

private:
    std::map<DeviceType, std::shared_ptr<BlobConverterAccCreater>> converter_creater_map_;
};
template <typename T> class BlobConverterAccRegister {
public:
    explicit BlobConverterAccRegister(DeviceType type) {
        BlobConverterManager::Shared()->RegisterBlobConverterAccCreater(type, std::make_shared<T>());
    }
};
#define DECLARE_BLOB_CONVERTER_CREATER(device)                                                                        \
    class device##BlobConverterAccCreater : public BlobConverterAccCreater {                                          \
    public:                                                                                                           \
        virtual ~device##BlobConverterAccCreater() {}                                                                 \
        virtual std::shared_ptr<BlobConverterAcc> CreateBlobConverterAcc(Blob *blob) {                                \
            return std::make_shared<device##BlobConverterAcc>(blob);                                                  \
        }                                                                                                             \
    }
#define REGISTER_BLOB_CONVERTER(device, device_type)                                                                  \
    BlobConverterAccRegister<device##BlobConverterAccCreater> g_blob_converter_##device(device_type)

class BlobConverter {
public:
    explicit BlobConverter(Blob *blob);
    Status ConvertToMat(Mat &image, MatConvertParam param, void *command_queue);
    Status ConvertFromMat(Mat &image, MatConvertParam param, void *command_queue);
    Status ConvertToMatAsync(Mat &image, MatConvertParam param, void *command_queue);
    Status ConvertFromMatAsync(Mat &image, MatConvertParam param, void *command_queue);

private:
    std::shared_ptr<BlobConverterAcc> impl_;
};

// ---- Mat utilities (include/tnn/utils/mat_utils.h:90-114, source/tnn/utils/mat_converter_acc.h:28-86): of the
// engine's operations on Mats only Copy concerns this path (the rest prepares camera images); the parameter structs of
// the others are declared so that a device's converter has the engine's interface ----
struct ResizeParam {};
struct CropParam {};
struct WarpAffineParam {};
struct CopyMakeBorderParam {};
typedef enum { COLOR_CONVERT_NV12TOBGR = 0 } ColorConversionType;
class MatConverterAcc {
public:
    virtual ~MatConverterAcc() {}
    virtual Status Copy(Mat &src, Mat &dst, void *command_queue = nullptr)                                      = 0;
    virtual Status Resize(Mat &src, Mat &dst, ResizeParam param, void *command_queue = nullptr)                 = 0;
    virtual Status Crop(Mat &src, Mat &dst, CropParam param, void *command_queue = nullptr)                     = 0;
    virtual Status WarpAffine(Mat &src, Mat &dst, WarpAffineParam param, void *command_queue = nullptr)         = 0;
    virtual Status CvtColor(Mat &src, Mat &dst, ColorConversionType type, void *command_queue = nullptr)        = 0;
    virtual Status CopyMakeBorder(Mat &src, Mat &dst, CopyMakeBorderParam param, void *command_queue = nullptr) = 0;
};
class MatConverterAccCreater {
public:
    virtual ~MatConverterAccCreater() {}
    virtual std::shared_ptr<MatConverterAcc> CreateMatConverterAcc() = 0;
};
class MatConverterManager {
public:
    static std::shared_ptr<MatConverterManager> &Shared();
    std::shared_ptr<MatConverterAcc> CreateMatConverterAcc(DeviceType device_type);
    int RegisterMatConverterAccCreater(DeviceType type, std::shared_ptr<MatConverterAccCreater> creater);

private:
    std::map<DeviceType, std::shared_ptr<MatConverterAccCreater>> converter_creater_map_;
};
template <typename T> class MatConverterAccRegister {
public:
    explicit MatConverterAccRegister(DeviceType type) {
        MatConverterManager::Shared()->RegisterMatConverterAccCreater(type, std::make_shared<T>());
    }
};
#define DECLARE_MAT_CONVERTER_CREATER(device)                                                                          \
    class device##MatConverterAccCreater : public MatConverterAccCreater {                                             \
    public:                                                                                                            \
        virtual ~device##MatConverterAccCreater() {}                                                                   \
        virtual std::shared_ptr<MatConverterAcc> CreateMatConverterAcc() {                                             \
            return std::make_shared<device##MatConverterAcc>();                                                        \
        }                                                                                                              \
    }
#define REGISTER_MAT_CONVERTER(device, device_type)                                                                    \
    MatConverterAccRegister<device##MatConverterAccCreater> g_mat_converter_##device(device_type)
class MatUtils {
public:
    // copy between a host Mat and a device Mat, or two Mats of one device, of equal dims (mat_utils.cc:73-100)
    static Status Copy(Mat &src, Mat &dst, void *command_queue);
};

// ---- layers (device independent): shape and dtype inference -------------------------------------
class DefaultNetwork;
class BaseLayer {
public:
    explicit BaseLayer(LayerType type) : type_(type) {}
    virtual ~BaseLayer();
    Status Init(Context *context, LayerParam *param, LayerResource *resource, std::vector<Blob *> &inputs,
                std::vector<Blob *> &outputs, AbstractDevice *device, ConstantResource *consts);
    Status Reshape();
    Status Forward();
    std::string GetLayerName() { return param_ ? param_->name : ""; }
    LayerType GetLayerType() { return type_; }
    std::vector<Blob *> &GetInputBlobs() { return input_blobs_; }
    std::vector<Blob *> &GetOutputBlobs() { return output_blobs_; }

protected:
    friend class DefaultNetwork;  // this host's Reshape infers every shape before it touches blob memory
    // base_layer.h:101-105
    virtual Status InferOutputShape(bool ignore_error = false);
    virtual Status InferOutputDataType();
    LayerType type_;
    LayerParam *param_       = nullptr;
    LayerResource *resource_ = nullptr;
    std::vector<Blob *> input_blobs_, output_blobs_;
    AbstractLayerAcc *layer_acc_ = nullptr;
};
// layer registry (base_layer.h:108-143)
class LayerCreator {
public:
    virtual ~LayerCreator() {}
    virtual BaseLayer *CreateLayer() = 0;
};
template <typename T> class TypeLayerCreator : public LayerCreator {
public:
    explicit TypeLayerCreator(LayerType type) : type_(type) {}
    BaseLayer *CreateLayer() override { return new T(type_); }

protected:
    LayerType type_;
};
std::map<LayerType, std::shared_ptr<LayerCreator>> &GetGlobalLayerCreatorMap();
template <typename T> class TypeLayerRegister {
public:
    explicit TypeLayerRegister(LayerType type) { GetGlobalLayerCreatorMap()[type] = std::shared_ptr<T>(new T(type)); }
};
BaseLayer *CreateLayer(LayerType type);

// ---- optimizer passes (optimizer/net_optimizer.h:25-37, net_optimizer_manager.h:32-66) -------------
namespace optimizer {
class NetOptimizer {
public:
    virtual ~NetOptimizer() {}
    virtual std::string Strategy()                                           = 0;
    virtual bool IsSupported(const NetworkConfig &net_config)                = 0;
    virtual Status Optimize(NetStructure *structure, NetResource *resource)  = 0;
};
typedef enum { P0 = 0, P1 = 1, P2 = 2, PLAST = 1000 } OptPriority;
class NetOptimizerManager {
public:
    // passes run in priority order, passes of one priority in the order of their strategy names
    static Status Optimize(NetStructure *structure, NetResource *resource, const NetworkConfig &net_config);
    static void RegisterNetOptimizer(NetOptimizer *optimizer, OptPriority prior);
};
template <typename T> class NetOptimizerRegister {
public:
    explicit NetOptimizerRegister(OptPriority p) { NetOptimizerManager::RegisterNetOptimizer(new T(), p); }
};
}  // namespace optimizer

// ---- network + instance -----------------------------------------------------------------------
struct LayerProfile {
    std::string name, type;
    double ms = 0;
    int calls = 0;
};

typedef std::function<void(void)> Callback;  // include/tnn/core/common.h:207
// include/tnn/core/instance.h:39: called around every layer by ForwardWithCallback
typedef std::function<void(std::vector<Blob *> &blobs, LayerInfo *info)> BlobStatisticCallback;

// core/default_network.h:37-160.  Forward, ForwardAsync, Reshape and the profile switches are virtual and the members
// a derived network needs are protected, as in the engine, so a device can bring its own network (core/abstract_network.h:
// 102-136: one factory per NetworkType, chosen by AbstractDevice::ConvertAutoNetworkType()).
class DefaultNetwork {
public:
    DefaultNetwork() {}
    virtual ~DefaultNetwork();
    // max_inputs_shape (may be empty: the model's own input shapes) is what the instance is created and its blob
    // memory planned at (instance.cc:48-128, default_network.cc:86-137)
    virtual Status Init(NetworkConfig &net_config, ModelInterpreter *interpreter,
                        const InputShapesMap &max_inputs_shape = InputShapesMap());
    // Everything Init does short of touching a device: the instance's copy of the graph is optimised, layers are
    // created (an unknown type or a type without an acc fails as in Init), blob types and shapes are inferred.  For
    // LayerSummary() / LayerIo() on a machine without a GPU.
    Status Plan(NetworkConfig &net_config, ModelInterpreter *interpreter, const InputShapesMap &inputs_shape = InputShapesMap());
    // default_network.cc:456-500: new dims for the named input blobs, then every layer infers its output shape again
    // and its acc is reshaped.  Weights stay on the device.  Blob memory is planned again only when a blob outgrows
    // its buffer.
    virtual Status Reshape(const InputShapesMap &inputs);
    virtual Status Forward();                           // default_network.cc:558-635: the layer loop, then Synchronize
    virtual Status ForwardAsync(Callback call_back);    // default_network.cc:672-686: the layer loop alone
    // default_network.cc:637-668: `before` sees a layer's inputs, `after` its outputs once the layer has finished
    virtual Status ForwardWithCallback(BlobStatisticCallback before, BlobStatisticCallback after);
    virtual Status GetCommandQueue(void **command_queue);
    // default_network.cc:537-556: this network's context adopts the other network's command queue; set the threads
    // the device may use on the host
    virtual Status ShareCommandQueue(DefaultNetwork *network);
    virtual Status SetCpuNumThreads(int num_threads);
    Context *GetContext() { return context_; }
    virtual Status GetAllInputBlobs(BlobMap &blobs);
    virtual Status GetAllOutputBlobs(BlobMap &blobs);
    Blob *GetBlob(const std::string &name);
    int LayerCount() const { return (int)layers_.size(); }
    std::string LayerSummary() const;
    // one line per layer: name|input blob names (comma separated)|output blob names|input dims (d0,d1,..;d0,..)|output dims
    std::string LayerIo() const;
    // per-layer event timing (the engine's TNN_PROFILE hook, source/tnn/core/profile.cc:111-201)
    // only layers whose type string equals `only_type` are timed when it is non-empty
    virtual void StartProfile(const std::string &only_type = "");
    virtual std::vector<LayerProfile> FinishProfile();

protected:
    virtual Status InitLayers();
    virtual Status AllocateBlobMemory();
    Status ReleaseBlobMemory();
    AbstractDevice *device_ = nullptr;
    Context *context_       = nullptr;
    std::vector<BaseLayer *> layers_;
    NetworkConfig config_;
    bool profiling_ = false;

private:
    std::map<Blob *, int64_t> blob_capacity_;  // bytes behind each planned blob
    NetStructure structure_;  // per-instance copy: optimizer rewrites never touch the interpreter
    NetResource resource_;
    std::map<std::string, Blob *> blobs_;
    std::vector<void *> allocations_;
    BlobMap inputs_, outputs_;
    std::vector<char> prof_on_;
    Status RunLayers(void *prof_stream);
    std::vector<std::pair<void *, void *>> prof_events_;
    std::vector<LayerProfile> prof_;
};

// core/abstract_network.h:102-136
class AbstractNetworkImplFactory {
public:
    virtual ~AbstractNetworkImplFactory() {}
    virtual std::shared_ptr<DefaultNetwork> CreateNetworkImp() = 0;
};
template <typename T> class NetworkImplFactory : public AbstractNetworkImplFactory {
public:
    virtual std::shared_ptr<DefaultNetwork> CreateNetworkImp() { return std::make_shared<T>(); }
};
class NetworkImplManager {
public:
    static std::shared_ptr<DefaultNetwork> GetNetworkImpl(NetworkType type);
    static void RegisterNetworkImplFactory(NetworkType type, AbstractNetworkImplFactory *factory);
};
template <typename T> class NetworkImplFactoryRegister {
public:
    explicit NetworkImplFactoryRegister(NetworkType type) { NetworkImplManager::RegisterNetworkImplFactory(type, new T()); }
};

class Instance {
public:
    Instance(NetworkConfig &net_config, ModelConfig &model_config) : net_config_(net_config), model_config_(model_config) {}
    Status Init();
    // instance.cc:48-128: created at max_inputs_shape (min_inputs_shape only bounds later Reshape calls in the engine;
    // it is accepted and not used here)
    Status Init(const InputShapesMap &min_inputs_shape, const InputShapesMap &max_inputs_shape);
    Status Reshape(const InputShapesMap &inputs);  // instance.cc:143-152
    Status Forward();
    Status ForwardAsync(Callback call_back);
    Status ForwardWithCallback(BlobStatisticCallback before, BlobStatisticCallback after);  // instance.cc:171-174
    Status GetCommandQueue(void **command_queue);
    Status ShareCommandQueue(Instance *instance);  // instance.cc:158-160
    Status SetCpuNumThreads(int num_threads);      // instance.cc:198-200
    Status GetAllInputBlobs(BlobMap &blobs);
    Status GetAllOutputBlobs(BlobMap &blobs);
    Status SetInputMat(std::shared_ptr<Mat> mat, MatConvertParam param, std::string input_name = "");
    Status GetOutputMat(std::shared_ptr<Mat> &mat, MatConvertParam param = MatConvertParam(),
                        std::string output_name = "", DeviceType device = DEVICE_NAIVE, MatType mat_type = NCHW_FLOAT);
    DefaultNetwork *GetNetwork() { return network_.get(); }

private:
    NetworkConfig net_config_;
    ModelConfig model_config_;
    std::shared_ptr<ModelInterpreter> interpreter_;
    std::shared_ptr<DefaultNetwork> network_;
    std::map<std::string, std::shared_ptr<Mat>> output_mats_;
    // blob name -> (the blob the converter was made for, converter)
    std::map<std::string, std::pair<Blob *, std::shared_ptr<BlobConverter>>> input_converters_, output_converters_;
};

}  // namespace TNN_NS

#include "rocm_engine_additions.h"
#endif
