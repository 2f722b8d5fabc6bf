// RocmNetwork: the engine's DefaultNetwork plus, behind a switch, whole-forward graph replay.
//
// On this device the launches of a forward pass are fixed once the instance is initialised (static shapes, stable
// blob and workspace addresses), so after two eager passes - which also perform every lazy allocation - the third can
// be recorded into an executable graph that later calls submit at once (TNN_ROCM_GRAPH=1).  The default is the
// engine's eager layer loop: with the sixty-odd launches a fused encoder is left with, the host stays ahead of the
// device, the gaps between kernels on the device are the same either way, and submitting the recorded graph costs
// more up front than the first eager launch (12-layer encoder, three machines: the replay is 0.5 - 1.8 % slower).
// The replay is for callers whose host thread is slow or busy.  The engine picks the network implementation
// per NetworkType (source/tnn/core/abstract_network.h:102-136, instance.cc:75-85); RocmDevice::ConvertAutoNetworkType()
// names this one, and it registers itself like the engine's other networks (default_network.cc:39-40).
#ifndef TNN_AMD_HOST_ROCM_NETWORK_H_
#define TNN_AMD_HOST_ROCM_NETWORK_H_

#include "rocm_device.h"
#ifdef TNN_ROCM_ENGINE_TREE
#include "tnn/core/default_network.h"
#endif

namespace TNN_NS {

class RocmNetwork : public DefaultNetwork {
public:
    RocmNetwork();
    ~RocmNetwork() override;
    Status Forward() override;
    Status ForwardAsync(Callback call_back) override;

#ifdef TNN_ROCM_ENGINE_TREE
protected:
    // The engine settles every blob's data type in UpdateBlobPrecision (default_network.cc:362-440), which returns
    // at once for a device it does not know; this override does that pass for DEVICE_ROCM and then runs the engine's
    // own InitLayers.
    Status InitLayers(NetStructure *net_structure, NetResource *net_resource) override;
#if TNN_PROFILE
    Status ProfiledForward();  // the forward loop with every layer timed (a profiler build of the engine)
#endif
#endif

private:
    // Everything a recording depends on: dims and device address of every blob the layers touch, and the context's
    // scratch allocation count.  A recording is replayed only under the signature it was made with, so a Reshape, a
    // re-planned blob pool or a grown workspace lead back to eager passes and a new recording by themselves.
    void Signature(std::vector<uint64_t> *sig);
    void DropGraphs();
    void DropProfileEvents();
    std::vector<void *> profile_events_;  // two per layer, created at the first profiled forward
    struct Recording {
        std::vector<uint64_t> signature;
        void *exec = nullptr;
    };
    std::vector<Recording> recordings_;
    std::vector<uint64_t> eager_signature_;
    int eager_forwards_ = 0;
    bool enabled_       = false;  // TNN_ROCM_GRAPH=1 turns the replay on; the default is the engine's eager loop
};

}  // namespace TNN_NS
#endif
