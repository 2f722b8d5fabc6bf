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
    DropProfileEvents();
}

void RocmNetwork::DropProfileEvents() {
    for (void *e : profile_events_)
        tnn_rocm_event_destroy(e);
    profile_events_.clear();
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
                // a Reformat's blobs follow its src / dst type in any net (default_network.cc:404-421), the others' only in a
                // quantised one
                if ((quantized_net || info->type == LAYER_REFORMAT) &&
                    RocmBlobIsInt8(info->type, info->param.get(), side == 0, i, info->outputs.size())) {
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

#if defined(TNN_ROCM_ENGINE_TREE) && TNN_PROFILE
// The engine's forward loop (default_network.cc:558-635) with a hipEvent pair around each layer; after the one
// synchronisation at the end every layer's ProfilingData (name, op type, dims, kernel time in ms: the fields
// AbstractLayerAcc::UpdateProfilingData fills, abstract_layer_acc.cc:102-125) goes to Context::AddProfilingData, from
// where Instance::FinishProfile prints the tables of core/profile.cc:111-201.
Status RocmNetwork::ProfiledForward() {
    RETURN_ON_NEQ(blob_manager_->CheckBlobMemoryState(), TNN_OK);
    if (runtime_blob_pool_)
        runtime_blob_pool_->ClearBlobMemoryPool();
    void *stream = nullptr;
    context_->GetCommandQueue(&stream);
    while (profile_events_.size() < 2 * layers_.size()) {
        void *e = nullptr;
        if (tnn_rocm_event_create(&e) != 0)
            return Status(TNNERR_CUDA_TENSORRT_ERROR, std::string("event create failed: ") + tnn_rocm_last_error());
        profile_events_.push_back(e);
    }
    RETURN_ON_NEQ(context_->OnInstanceForwardBegin(), TNN_OK);
    for (size_t i = 0; i < layers_.size(); ++i) {
        tnn_rocm_event_record(profile_events_[2 * i], stream);
        Status st = layers_[i]->Forward();
        tnn_rocm_event_record(profile_events_[2 * i + 1], stream);
        if (st != TNN_OK)
            return st;
    }
    context_->OnInstanceForwardEnd();
    RETURN_ON_NEQ(context_->Synchronize(), TNN_OK);
    for (size_t i = 0; i < layers_.size(); ++i) {
        auto pdata = std::make_shared<ProfilingData>();
        pdata->layer_name = layers_[i]->GetLayerName();
        if (i < net_structure_->layers.size() && net_structure_->layers[i])
            pdata->op_name = net_structure_->layers[i]->type_str;
        const auto ins = layers_[i]->GetInputBlobs(), outs = layers_[i]->GetOutputBlobs();
        if (!ins.empty())
            pdata->input_dims = ins[0]->GetBlobDesc().dims;
        if (!outs.empty())
            pdata->output_dims = outs[0]->GetBlobDesc().dims;
        float ms = 0.f;
        tnn_rocm_event_elapsed_ms(profile_events_[2 * i], profile_events_[2 * i + 1], &ms);
        pdata->kernel_time = ms;
        context_->AddProfilingData(pdata);
    }
    return TNN_OK;
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
#if TNN_PROFILE
    // a profiler build of the engine (TNN_PROFILER_ENABLE): between Instance::StartProfile and FinishProfile every layer
    // is timed with an event pair and reported to the context, as the engine's own accs do around their DoForward
    // (x86_layer_acc.cc:55-72); no graph replay then - a replayed graph has no layer boundaries on the host
    if (context_->profile_layer)
        return ProfiledForward();
#endif
    const bool profiling = false;
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
