#include "rocm_network.h"

#include <cstdlib>

namespace TNN_NS {

static NetworkImplFactoryRegister<NetworkImplFactory<RocmNetwork>> g_network_impl_rocm_factory_register(NETWORK_TYPE_ROCM);

namespace {
constexpr size_t kMaxRecordings = 16;  // input-shape signatures kept at once; beyond that all are dropped
}

RocmNetwork::RocmNetwork() {
    if (const char *g = getenv("TNN_ROCM_GRAPH"))
        enabled_ = atoi(g) != 0;
}

RocmNetwork::~RocmNetwork() {
    if (context_)
        context_->Synchronize();
    DropGraphs();
}

void RocmNetwork::DropGraphs() {
    for (auto &r : recordings_)
        tnn_rocm_graph_destroy(r.exec);
    recordings_.clear();
}

void RocmNetwork::Signature(std::vector<uint64_t> *sig) {
    sig->clear();
    auto rocm = dynamic_cast<RocmContext *>(context_);
    sig->push_back(rocm ? rocm->MemoryEpoch() : 0);
    for (auto layer : layers_) {
        const std::vector<Blob *> ins = layer->GetInputBlobs(), outs = layer->GetOutputBlobs();
        for (auto blobs : {&ins, &outs})
            for (Blob *b : *blobs) {
                auto h = b->GetHandle();
                sig->push_back((uint64_t)(uintptr_t)h.base + h.bytes_offset);
                const auto &dims = b->GetBlobDesc().dims;
                uint64_t packed  = dims.size();
                for (int d : dims) {
                    if (packed >> 40) {  // keep every dimension: start a new word when this one is full
                        sig->push_back(packed);
                        packed = 0;
                    }
                    packed = (packed << 20) ^ (uint64_t)(uint32_t)d;
                }
                sig->push_back(packed);
            }
    }
}

#ifdef TNN_ROCM_ENGINE_TREE
Status RocmNetwork::InitLayers(NetStructure *net_structure, NetResource *net_resource) {
    // float blobs follow the network precision (PRECISION_HIGH: fp32; PRECISION_LOW: bfloat16; otherwise fp16), the
    // blobs a quantised layer reads or writes become BlobInt8 with their scale resource, integer blobs stay
    const bool half          = config_.precision != PRECISION_HIGH;
    const DataType half_type = config_.precision == PRECISION_LOW ? DATA_TYPE_BFP16 : DATA_TYPE_HALF;
    bool quantized_net       = false;
    for (auto &info : net_structure->layers)
        quantized_net |= info->param && info->param->quantized;
    auto &consts = net_resource->constant_map;
    for (auto &info : net_structure->layers) {
        for (int side = 0; side < 2; ++side) {
            auto &names = side == 0 ? info->inputs : info->outputs;
            for (size_t i = 0; i < names.size(); ++i) {
                if (consts.find(names[i]) != consts.end())
                    continue;
                Blob *blob = blob_manager_->GetBlob(names[i]);
                if (!blob)
                    return Status(TNNERR_PARAM_ERR, "layer " + info->name + " names a blob the blob manager does not have");
                if (quantized_net && RocmBlobIsInt8(info->type, info->param.get(), side == 0, i, info->outputs.size())) {
                    if (!dynamic_cast<BlobInt8 *>(blob))
                        RETURN_ON_NEQ(GenerateInt8Blob(names[i], net_resource, &blob), TNN_OK);
                    blob->GetBlobDesc().data_type = DATA_TYPE_INT8;
                    continue;
                }
                DataType &dt = blob->GetBlobDesc().data_type;
                if (dt == DATA_TYPE_FLOAT || dt == DATA_TYPE_HALF || dt == DATA_TYPE_BFP16)
                    dt = half ? half_type : DATA_TYPE_FLOAT;
            }
        }
    }
    return DefaultNetwork::InitLayers(net_structure, net_resource);
}
#endif

Status RocmNetwork::Forward() {
    RETURN_ON_NEQ(RocmNetwork::ForwardAsync(nullptr), TNN_OK);
    return context_->Synchronize();
}

Status RocmNetwork::ForwardAsync(Callback call_back) {
    void *stream = nullptr;
    context_->GetCommandQueue(&stream);
#ifdef TNN_ROCM_ENGINE_TREE
    const bool profiling = false;  // a TNN_PROFILE build times layers through the context; build it with TNN_ROCM_GRAPH=0
#else
    const bool profiling = profiling_;
#endif
    if (!enabled_ || profiling || stream == nullptr)
        return DefaultNetwork::ForwardAsync(call_back);

    std::vector<uint64_t> sig;
    Signature(&sig);
    for (auto &r : recordings_)
        if (r.signature == sig) {
            RETURN_ON_NEQ(context_->OnInstanceForwardBegin(), TNN_OK);
            if (tnn_rocm_graph_launch(r.exec, stream) != 0)
                return Status(TNNERR_CUDA_KERNEL_LAUNCH_ERROR, std::string("graph launch failed: ") + tnn_rocm_last_error());
            return context_->OnInstanceForwardEnd();
        }
    if (sig != eager_signature_) {
        eager_signature_ = sig;
        eager_forwards_  = 0;
    }
    if (eager_forwards_ < 2) {
        ++eager_forwards_;
        return DefaultNetwork::ForwardAsync(call_back);
    }
    // third pass under this signature: record it
    if (tnn_rocm_graph_begin_capture(stream) != 0) {
        enabled_ = false;
        return DefaultNetwork::ForwardAsync(call_back);
    }
    Status st  = DefaultNetwork::ForwardAsync(call_back);
    void *exec = nullptr;
    int rc     = tnn_rocm_graph_end_capture(stream, &exec);
    if (st != TNN_OK) {
        tnn_rocm_graph_destroy(exec);
        return st;
    }
    if (rc != 0 || !exec) {  // this sequence of layers cannot be recorded: stay eager from now on
        enabled_ = false;
        return DefaultNetwork::ForwardAsync(call_back);
    }
    std::vector<uint64_t> after;
    Signature(&after);
    if (after != sig) {  // something was still allocated during the recorded pass: its pointers are already stale
        tnn_rocm_graph_destroy(exec);
        eager_forwards_ = 0;
        return DefaultNetwork::ForwardAsync(call_back);
    }
    if (recordings_.size() >= kMaxRecordings) {
        RETURN_ON_NEQ(context_->Synchronize(), TNN_OK);
        DropGraphs();
    }
    Recording r;
    r.signature = sig;
    r.exec      = exec;
    recordings_.push_back(r);
    if (tnn_rocm_graph_launch(exec, stream) != 0)
        return Status(TNNERR_CUDA_KERNEL_LAUNCH_ERROR, std::string("graph launch failed: ") + tnn_rocm_last_error());
    return TNN_OK;
}

}  // namespace TNN_NS
