// DEVICE_ROCM: the device, its context and the layer-acc base class.
//
// Role of each class in the engine (reference tree):
//   RocmDevice   : AbstractDevice   source/tnn/core/abstract_device.h:40-103 ; the CUDA backend's
//                  counterpart is source/tnn/device/cuda/cuda_device.cc:53-174
//   RocmContext  : Context          source/tnn/core/context.h:29-95 ; cuda_context.cc:47-154
//   RocmLayerAcc : AbstractLayerAcc source/tnn/core/abstract_layer_acc.h:39-127 ; cuda_layer_acc.cc:23-110
// All GPU work goes through the C ABI in tnn_rocm.h; no HIP header is included on the host side.
#ifndef TNN_AMD_HOST_ROCM_DEVICE_H_
#define TNN_AMD_HOST_ROCM_DEVICE_H_

#ifdef TNN_ROCM_ENGINE_TREE
// inside the engine tree: the engine's own headers, plus the additions this backend needs from the engine
// (DEVICE_ROCM, the fused layer types with their params / resources)
#include "tnn/core/abstract_device.h"
#include "tnn/core/abstract_layer_acc.h"
#include "tnn/core/blob_int8.h"
#include "tnn/core/context.h"
#include "tnn/interpreter/layer_param.h"
#include "tnn/interpreter/layer_resource.h"
#include "tnn/optimizer/net_optimizer.h"
#include "tnn/optimizer/net_optimizer_manager.h"
#include "tnn/utils/blob_converter_internal.h"
#include "tnn/utils/data_type_utils.h"
#include "tnn/utils/mat_converter_acc.h"
#include "tnn/utils/dims_utils.h"
#include "rocm_engine_additions.h"
#else
#include "tnn_host.h"
#endif
#include <map>
#include <string>

#include "tnn_rocm.h"

namespace TNN_NS {

// maps a failed C-ABI call to a Status carrying the library's message
Status RocmStatus(int rc, int tnn_code, const char *what);
#define ROCM_CALL(expr)                                                                                               \
    do {                                                                                                              \
        int _rc = (expr);                                                                                             \
        if (_rc != 0)                                                                                                 \
            return RocmStatus(_rc, TNNERR_CUDA_KERNEL_LAUNCH_ERROR, #expr);                                           \
    } while (0)

class RocmContext : public Context {
public:
    explicit RocmContext(int device_id);
    ~RocmContext() override;
    Status Setup();
    Status LoadLibrary(std::vector<std::string> path) override { return TNN_OK; }
    Status GetCommandQueue(void **command_queue) override;
    // This context launches on the other context's stream from now on (role of cuda_context.cc:91-122); the other
    // context must outlive this one.  Recordings made on the old stream are dropped (a new memory epoch).
    Status ShareCommandQueue(Context *context) override;
    Status OnInstanceForwardBegin() override;
    Status OnInstanceForwardEnd() override { return TNN_OK; }
    Status Synchronize() override;
    // Counts the (re)allocations of device memory the context owns (scratch that grows with the shapes).  A recorded
    // launch sequence holds raw pointers into that memory, so RocmNetwork only replays it while this number stands still.
    uint64_t MemoryEpoch() const { return memory_epoch_; }

    void *Stream() { return stream_; }
    // grow-only scratch owned by the context; valid until the next call with a larger size
    Status Workspace(size_t bytes, void **ptr);
    // Small named device buffers that one layer of a forward writes and a later one reads without a blob in between
    // (the rows' LayerNorm statistics: fp32 in a net whose blobs are half precision).  Grow-only per name; a
    // (re)allocation counts as a memory epoch.
    Status SideBuffer(const std::string &name, size_t bytes, void **ptr);
    // a number the writer of a side buffer leaves for its reader (how many blocks of row sums the launch produced)
    int &SideBufferTag(const std::string &name) { return side_buffers_[name].tag; }
    // page-locked word kernels raise on a data error (e.g. Gather index out of range)
    int32_t *ErrorFlag() { return error_flag_; }
    // The padding mask is one blob shared by every attention layer of a forward pass: the first layer that asks
    // derives its fp32 copy and the per-sequence key counts, later layers of the same forward reuse them.
    // one_row: the blob holds S values that serve every sequence (an additive mask [1,1,1,S])
    Status AttentionMask(const void *mask_blob, int mask_dtype, int B, int S, bool one_row, const float **mask_f32,
                         const int32_t **kv_len);

private:
    int device_id_       = 0;
    void *stream_        = nullptr;
    bool own_stream_     = true;
    void *workspace_     = nullptr;
    size_t workspace_sz_ = 0;
    int32_t *error_flag_ = nullptr;
    uint64_t forward_epoch_ = 0;
    uint64_t memory_epoch_  = 0;
    struct MaskEntry {
        const void *src = nullptr;
        uint64_t epoch  = 0;
        int B = 0, S = 0;
        bool one_row = false;
        size_t cap_mask = 0, cap_len = 0;  // elements allocated (grow-only, so recorded launch sequences stay valid)
        void *mask_f32 = nullptr, *kv_len = nullptr;
    } mask_cache_;
    struct SideEntry {
        void *ptr  = nullptr;
        size_t cap = 0;
        int tag    = 0;
    };
    std::map<std::string, SideEntry> side_buffers_;
};

class RocmDevice : public AbstractDevice {
public:
    explicit RocmDevice(DeviceType device_type) : AbstractDevice(device_type) {}
    BlobMemorySizeInfo Calculate(BlobDesc &desc) override;
    Status Allocate(void **handle, MatType mat_type, DimsVector dims) override;
    Status Allocate(void **handle, BlobMemorySizeInfo &size_info) override;
    Status Free(void *handle) override;
    Status CopyToDevice(BlobHandle *dst, const BlobHandle *src, BlobDesc &desc, void *command_queue) override;
    Status CopyFromDevice(BlobHandle *dst, const BlobHandle *src, BlobDesc &desc, void *command_queue) override;
    AbstractLayerAcc *CreateLayerAcc(LayerType type) override;
    Context *CreateContext(int device_id) override;
    std::shared_ptr<const ImplementedPrecision> GetImplementedPrecision(LayerType type) override;
    // RocmNetwork (rocm_network.h): DefaultNetwork plus whole-forward graph replay
    NetworkType ConvertAutoNetworkType() override { return NETWORK_TYPE_ROCM; }
    static Status RegisterLayerAccCreator(LayerType type, LayerAccCreator *creator);

private:
    static std::map<LayerType, std::shared_ptr<LayerAccCreator>> &GetLayerCreatorMap();
};

template <typename T> class RocmTypeLayerAccRegister {
public:
    explicit RocmTypeLayerAccRegister(LayerType type) { RocmDevice::RegisterLayerAccCreator(type, new T()); }
};
#define REGISTER_ROCM_ACC(cls, layer_type)                                                                            \
    static RocmTypeLayerAccRegister<TypeLayerAccCreator<cls>> g_rocm_##layer_type##_acc_register(layer_type)

class RocmLayerAcc : public AbstractLayerAcc {
public:
    ~RocmLayerAcc() override;
    Status Init(Context *context, LayerParam *param, LayerResource *resource, const std::vector<Blob *> &inputs,
                const std::vector<Blob *> &outputs) override;
    Status Reshape(const std::vector<Blob *> &inputs, const std::vector<Blob *> &outputs) override { return TNN_OK; }
    // uploads constant_map entries bound to input blobs (gamma/beta, masks, bias operands)
    Status ReloadConstantBlobs(const std::vector<Blob *> &inputs, bool only_reload_shape_differ_blob = false) override;

protected:
    // dtype a constant input should be stored in; default: the dtype of the first non-constant input
    virtual DataType ConstantBlobDataType(const std::vector<Blob *> &inputs, int index);
    // device copy of host data converted from src_type to dst_type (fp32 -> fp16/bf16 on device); owned by the acc
    Status UploadConverted(const void *host, size_t count, DataType src_type, DataType dst_type, void **out);
    void *Stream() { return context_->Stream(); }
    // the blob an input resolves to: this acc's device copy for constants, the blob itself otherwise
    Blob *In(Blob *b) {
        auto it = const_blob_map_.find(b->GetBlobDesc().name);
        return it == const_blob_map_.end() ? b : it->second.get();
    }
    static void *Ptr(Blob *b) { return (char *)b->GetHandle().base + b->GetHandle().bytes_offset; }

    RocmContext *context_    = nullptr;
    LayerParam *param_       = nullptr;
    LayerResource *resource_ = nullptr;
    std::vector<void *> owned_device_;

private:
    std::vector<DataFormat> SupportDataFormat(DataType data_type, int dims_size, BlobType blob_type) override;
};

}  // namespace TNN_NS
#endif
