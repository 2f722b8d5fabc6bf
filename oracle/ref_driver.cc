// Drives the reference engine's own CPU paths (DEVICE_NAIVE / DEVICE_X86) through its public API
// (include/tnn/core/tnn.h:34-66, instance.h:42-144, mat.h:53-87) from a .tnnproto text and a .tnnmodel
// blob held in memory.  TEST INFRASTRUCTURE ONLY: it is built into oracle/_ref/ together with the
// reference library, serves as the checker for the model-file writer and the DEVICE_ROCM host, and is
// the timed CPU baseline ("reference") of the benchmark.  Nothing shipped links against it.
#include <chrono>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "tnn/core/blob.h"
#include "tnn/core/instance.h"
#include "tnn/core/mat.h"
#include "tnn/core/tnn.h"
#include "tnn/utils/blob_converter.h"
#include "tnn/utils/mat_utils.h"

using namespace TNN_NS;

namespace {
struct Session {
    TNN net;
    std::shared_ptr<Instance> inst;
    std::string err;
    std::vector<std::pair<std::string, std::shared_ptr<Mat>>> inputs;  // the host Mats last given per input name
    std::shared_ptr<Mat> device_output;                                // the device Mat last handed out
};
void put_err(char *buf, size_t n, const std::string &s) {
    if (buf && n) {
        snprintf(buf, n, "%s", s.c_str());
    }
}
}  // namespace

extern "C" {

#define REF_API __attribute__((visibility("default")))

// "name:d0,d1,...;name:..." -> InputShapesMap
static InputShapesMap parse_shapes(const char *spec) {
    InputShapesMap m;
    std::string s(spec ? spec : "");
    size_t pos = 0;
    while (pos < s.size()) {
        size_t end = s.find(';', pos);
        if (end == std::string::npos)
            end = s.size();
        const std::string item = s.substr(pos, end - pos);
        const size_t colon     = item.find(':');
        if (colon != std::string::npos) {
            DimsVector d;
            size_t p = colon + 1;
            while (p < item.size()) {
                size_t q = item.find(',', p);
                if (q == std::string::npos)
                    q = item.size();
                d.push_back(atoi(item.substr(p, q - p).c_str()));
                p = q + 1;
            }
            m[item.substr(0, colon)] = d;
        }
        pos = end + 1;
    }
    return m;
}

// device: "NAIVE", "X86", or "ROCM" / "ROCM:fp32" (see below).  Returns nullptr and fills err on failure.
// min_shapes / max_shapes ("name:d0,d1;..."; both empty: the model's own shapes): the ranges Instance::Reshape may move in
REF_API void *tnn_ref_create_shaped(const char *proto, size_t proto_len, const char *model, size_t model_len,
                                    const char *device, int threads, const char *min_shapes, const char *max_shapes,
                                    char *err, size_t err_len) {
    std::unique_ptr<Session> s(new Session);
    ModelConfig mc;
    mc.model_type = MODEL_TYPE_TNN;
    mc.params.push_back(std::string(proto, proto_len));
    mc.params.push_back(std::string(model, model_len));
    Status st = s->net.Init(mc);
    if (st != TNN_OK) {
        put_err(err, err_len, "TNN::Init: " + st.description());
        return nullptr;
    }
    NetworkConfig nc;
    std::string dev(device);
    // "+extmem" behind the device: the caller brings the blob memory (SHARE_MEMORY_MODE_SET_FROM_EXTERNAL,
    // Instance::GetForwardMemorySize / SetForwardMemory)
    const size_t ext = dev.find("+extmem");
    if (ext != std::string::npos) {
        dev.erase(ext);
        nc.share_memory_mode = SHARE_MEMORY_MODE_SET_FROM_EXTERNAL;
    }
    nc.device_type  = dev == "X86" ? DEVICE_X86 : DEVICE_NAIVE;
    nc.network_type = NETWORK_TYPE_DEFAULT;
    nc.precision    = PRECISION_HIGH;
    if (dev.compare(0, 4, "ROCM") == 0) {
        // the DEVICE_ROCM backend of this repository built against this engine (oracle/_ref/libtnn_rocm_engine.so, which
        // the caller has loaded into the process: its static registrations made the device known).  The device and
        // network type values are the backend's own; "ROCM:fp32" asks for fp32 blobs (PRECISION_HIGH), "ROCM:bf16" for
        // bf16 (PRECISION_LOW), "ROCM" for the default (PRECISION_AUTO: fp16).
        nc.device_type  = static_cast<DeviceType>(0x1080);
        nc.network_type = NETWORK_TYPE_AUTO;  // RocmDevice::ConvertAutoNetworkType() names the backend's network
        nc.precision    = dev == "ROCM:fp32" ? PRECISION_HIGH : (dev == "ROCM:bf16" ? PRECISION_LOW : PRECISION_AUTO);
    }
    const InputShapesMap lo = parse_shapes(min_shapes), hi = parse_shapes(max_shapes);
    s->inst = hi.empty() ? s->net.CreateInst(nc, st) : s->net.CreateInst(nc, st, lo.empty() ? hi : lo, hi);
    if (st != TNN_OK || !s->inst) {
        put_err(err, err_len, "TNN::CreateInst: " + st.description());
        return nullptr;
    }
    if (threads > 0)
        s->inst->SetCpuNumThreads(threads);
    return s.release();
}

REF_API void *tnn_ref_create(const char *proto, size_t proto_len, const char *model, size_t model_len,
                             const char *device, int threads, char *err, size_t err_len) {
    return tnn_ref_create_shaped(proto, proto_len, model, model_len, device, threads, "", "", err, err_len);
}

REF_API void tnn_ref_destroy(void *h) { delete static_cast<Session *>(h); }

// Instance::Reshape to the input shapes named ("name:d0,d1;...")
REF_API int tnn_ref_reshape(void *h, const char *shapes) {
    Session *s = static_cast<Session *>(h);
    Status st  = s->inst->Reshape(parse_shapes(shapes));
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    s->inputs.clear();
    return 0;
}

// The flow of the reference's blob-converter unit test (test/unit_test/blob_converter_test.cc:287-349) on an input blob of
// this session: a BlobConverter of the blob's own device takes an fp32 NCHW Mat in with per-channel scale and bias
// (ConvertFromMat) and gives the blob back as an fp32 NCHW Mat with the same scale and bias applied again
// (ConvertToMat).  in / out hold the blob's element count; scale / bias hold n_param values.
REF_API int tnn_ref_input_blob_round_trip(void *h, const char *name, const float *in, const float *scale, const float *bias,
                                          int n_param, float *out, int on_device) {
    Session *s = static_cast<Session *>(h);
    BlobMap blobs;
    Status st = s->inst->GetAllInputBlobs(blobs);
    if (st != TNN_OK || blobs.find(name) == blobs.end()) {
        s->err = st != TNN_OK ? st.description() : std::string("no input blob named ") + name;
        return st != TNN_OK ? (int)st : -1;
    }
    Blob *blob = blobs[name];
    void *queue = nullptr;
    s->inst->GetCommandQueue(&queue);
    MatConvertParam param;
    param.scale.assign(scale, scale + n_param);
    param.bias.assign(bias, bias + n_param);
    DimsVector dims = blob->GetBlobDesc().dims;
    BlobConverter converter(blob);
    // on_device: in / out are addresses in the memory of the blob's own device, the Mats are Mats of that device
    const DeviceType where = on_device ? blob->GetBlobDesc().device_type : DEVICE_NAIVE;
    Mat mat_in(where, NCHW_FLOAT, dims, const_cast<float *>(in));
    st = converter.ConvertFromMat(mat_in, param, queue);
    if (st == TNN_OK) {
        Mat mat_out(where, NCHW_FLOAT, dims, out);
        st = converter.ConvertToMat(mat_out, param, queue);
    }
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    return 0;
}

// MatUtils::Copy of the reference (include/tnn/utils/mat_utils.h:77-79) three times: host Mat `in` -> a Mat of `device` the
// engine allocates -> a second Mat of that device, allocated by the copy -> host Mat `out`.  fp32 values.
REF_API int tnn_ref_mat_copy_round_trip(const char *device, const float *in, float *out, const int *dims, int ndims, char *err,
                                        size_t err_len) {
    DeviceType dt = DEVICE_NAIVE;
    std::string name(device ? device : "");
    if (name.compare(0, 4, "ROCM") == 0)
        dt = (DeviceType)0x1080;
    DimsVector d(dims, dims + ndims);
    Mat src(DEVICE_NAIVE, NCHW_FLOAT, d, const_cast<float *>(in));
    Mat first(dt, NCHW_FLOAT, d), second(dt, NCHW_FLOAT, d, nullptr);
    Mat back(DEVICE_NAIVE, NCHW_FLOAT, d, out);
    Status st = MatUtils::Copy(src, first, nullptr);
    if (st == TNN_OK)
        st = MatUtils::Copy(first, second, nullptr);
    if (st == TNN_OK)
        st = MatUtils::Copy(second, back, nullptr);
    if (st != TNN_OK) {
        put_err(err, err_len, st.description());
        return (int)st;
    }
    return 0;
}

// SetInputMat / GetOutputMat with Mats in the memory of the session's own device (instance.cc:214-320 with a device other
// than DEVICE_NAIVE): the input Mat wraps the caller's device address, the output Mat is allocated by the engine through
// AbstractDevice::Allocate(mat type, dims) and stays with the session until the next call for that output.
REF_API int tnn_ref_set_input_device(void *h, const char *name, const void *device_data, int is_int32, const int *dims,
                                     int ndims) {
    Session *s = static_cast<Session *>(h);
    BlobMap blobs;
    s->inst->GetAllInputBlobs(blobs);
    if (blobs.find(name) == blobs.end()) {
        s->err = std::string("no input blob named ") + name;
        return -1;
    }
    DimsVector d(dims, dims + ndims);
    auto mat  = std::make_shared<Mat>(blobs[name]->GetBlobDesc().device_type, is_int32 ? NC_INT32 : NCHW_FLOAT, d,
                                     const_cast<void *>(device_data));
    Status st = s->inst->SetInputMat(mat, MatConvertParam(), name);
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    return 0;
}

REF_API int tnn_ref_get_output_device(void *h, const char *name, void **device_data, int *dims, int *ndims) {
    Session *s = static_cast<Session *>(h);
    BlobMap blobs;
    s->inst->GetAllOutputBlobs(blobs);
    if (blobs.find(name) == blobs.end()) {
        s->err = std::string("no output blob named ") + name;
        return -1;
    }
    std::shared_ptr<Mat> mat;
    Status st = s->inst->GetOutputMat(mat, MatConvertParam(), name, blobs[name]->GetBlobDesc().device_type, NCHW_FLOAT);
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    s->device_output = mat;
    DimsVector d     = mat->GetDims();
    *ndims           = (int)d.size();
    for (size_t i = 0; i < d.size() && i < 8; ++i)
        dims[i] = d[i];
    *device_data = mat->GetData();
    return 0;
}

// mat_type: 0 = NCHW_FLOAT (fp32 data), 1 = NC_INT32 (int32 data), 2 = RESERVED_INT8_TEST (int8 data copied as it is
// into an int8 blob: what the reference's layer unit tests feed quantised layers with, layer_test.cc:258-261)
static MatType mat_type_of(int code) { return code == 1 ? NC_INT32 : (code == 2 ? RESERVED_INT8_TEST : NCHW_FLOAT); }

REF_API int tnn_ref_set_input(void *h, const char *name, const void *data, int mat_type, const int *dims, int ndims) {
    Session *s = static_cast<Session *>(h);
    DimsVector d(dims, dims + ndims);
    auto mat = std::make_shared<Mat>(DEVICE_NAIVE, mat_type_of(mat_type), d, const_cast<void *>(data));
    Status st = s->inst->SetInputMat(mat, MatConvertParam(), name);
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    bool known = false;
    for (auto &kv : s->inputs)
        if (kv.first == name) {
            kv.second = mat;
            known     = true;
        }
    if (!known)
        s->inputs.push_back({name, mat});
    return 0;
}

// blob memory brought by the caller (a pointer the session's device can use): instance.cc GetForwardMemorySize / SetForwardMemory
REF_API int tnn_ref_forward_memory_size(void *h, int *bytes) {
    Session *s = static_cast<Session *>(h);
    Status st  = s->inst->GetForwardMemorySize(*bytes);
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    return 0;
}

REF_API int tnn_ref_set_forward_memory(void *h, void *memory) {
    Session *s = static_cast<Session *>(h);
    Status st  = s->inst->SetForwardMemory(memory);
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    return 0;
}

REF_API int tnn_ref_forward(void *h) {
    Session *s = static_cast<Session *>(h);
    Status st  = s->inst->Forward();
    if (st != TNN_OK) {
        s->err = st.description();
        return (int)st;
    }
    return 0;
}

// Copies output blob `name` as fp32 into out (capacity in elements); dims/ndims receive its shape.
REF_API int tnn_ref_get_output(void *h, const char *name, float *out, size_t capacity, int *dims, int *ndims) {
    Session *s = static_cast<Session *>(h);
    std::shared_ptr<Mat> mat;
    Status st = s->inst->GetOutputMat(mat, MatConvertParam(), name, DEVICE_NAIVE, NCHW_FLOAT);
    if (st != TNN_OK || !mat) {
        s->err = st.description();
        return st != TNN_OK ? (int)st : -1;
    }
    DimsVector d = mat->GetDims();
    size_t count = 1;
    for (int v : d)
        count *= (size_t)v;
    if (ndims)
        *ndims = (int)d.size();
    if (dims)
        for (size_t i = 0; i < d.size() && i < 8; ++i)
            dims[i] = d[i];
    if (count > capacity) {
        s->err = "output buffer too small";
        return -2;
    }
    memcpy(out, mat->GetData(), count * sizeof(float));
    return 0;
}

// The data type of output blob `name` as the network settled it (DATA_TYPE_FLOAT 0, HALF 1, INT8 2, INT32 3, BFP16 4),
// -1 if there is no such output: the reference's layer tests choose their comparison rule by it (layer_test.cc:386-404).
REF_API int tnn_ref_output_data_type(void *h, const char *name) {
    Session *s = static_cast<Session *>(h);
    BlobMap blobs;
    if (s->inst->GetAllOutputBlobs(blobs) != TNN_OK || !blobs.count(name))
        return -1;
    return (int)blobs[name]->GetBlobDesc().data_type;
}

// As tnn_ref_get_output with the Mat type chosen by the caller (codes of tnn_ref_set_input); capacity in bytes.
REF_API int tnn_ref_get_output_as(void *h, const char *name, int mat_type, void *out, size_t capacity_bytes, int *dims,
                                  int *ndims) {
    Session *s = static_cast<Session *>(h);
    std::shared_ptr<Mat> mat;
    Status st = s->inst->GetOutputMat(mat, MatConvertParam(), name, DEVICE_NAIVE, mat_type_of(mat_type));
    if (st != TNN_OK || !mat) {
        s->err = st.description();
        return st != TNN_OK ? (int)st : -1;
    }
    DimsVector d = mat->GetDims();
    size_t count = 1;
    for (int v : d)
        count *= (size_t)v;
    if (ndims)
        *ndims = (int)d.size();
    if (dims)
        for (size_t i = 0; i < d.size() && i < 8; ++i)
            dims[i] = d[i];
    const size_t bytes = count * (mat_type == 2 ? 1 : 4);
    if (bytes > capacity_bytes) {
        s->err = "output buffer too small";
        return -2;
    }
    memcpy(out, mat->GetData(), bytes);
    return 0;
}

#if TNN_PROFILE
// A profiler build of the engine only: Instance::StartProfile, `forwards` Forward calls, Instance::FinishProfile
// (instance.cc:321-340); the report (the per-layer table and the per-type summary of core/profile.cc:111-201) is
// copied into buf.  Returns 0, or the failing Forward's status.
REF_API int tnn_ref_profile(void *h, int forwards, char *buf, size_t buf_len) {
    Session *s = static_cast<Session *>(h);
    s->inst->StartProfile();
    for (int i = 0; i < forwards; ++i) {
        Status st = s->inst->Forward();
        if (st != TNN_OK) {
            s->err = st.description();
            s->inst->FinishProfile(false);
            return (int)st;
        }
    }
    put_err(buf, buf_len, s->inst->FinishProfile(false));
    return 0;
}
#endif

REF_API const char *tnn_ref_last_error(void *h) { return static_cast<Session *>(h)->err.c_str(); }

// Mean wall time (seconds) of `iters` Forward() calls after `warmup` untimed ones.
REF_API double tnn_ref_time_forward(void *h, int warmup, int iters) {
    Session *s = static_cast<Session *>(h);
    for (int i = 0; i < warmup; ++i)
        if (s->inst->Forward() != TNN_OK)
            return -1.0;
    auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i)
        if (s->inst->Forward() != TNN_OK)
            return -1.0;
    auto t1 = std::chrono::steady_clock::now();
    return std::chrono::duration<double>(t1 - t0).count() / (iters > 0 ? iters : 1);
}

// The measurement loop of the reference's own benchmark tool (test/test.cc:101-152): `warmup` untimed iterations,
// then `iters` timed ones, each iteration = SetInputMat of every input (ConvertFromMat) + Forward + GetOutputMat of
// `out_name` (ConvertToMat).  stats receives {min, avg, max} seconds per iteration.  The caller keeps the input
// buffers given to tnn_ref_set_input alive.
REF_API int tnn_ref_time_loop(void *h, int warmup, int iters, const char *out_name, double *stats) {
    Session *s = static_cast<Session *>(h);
    double mn = 1e30, mx = 0.0, sum = 0.0;
    for (int i = 0; i < warmup + iters; ++i) {
        auto t0 = std::chrono::steady_clock::now();
        for (auto &kv : s->inputs) {
            Status st = s->inst->SetInputMat(kv.second, MatConvertParam(), kv.first);
            if (st != TNN_OK) {
                s->err = st.description();
                return (int)st;
            }
        }
        Status st = s->inst->Forward();
        std::shared_ptr<Mat> mat;
        if (st == TNN_OK)
            st = s->inst->GetOutputMat(mat, MatConvertParam(), out_name, DEVICE_NAIVE, NCHW_FLOAT);
        if (st != TNN_OK) {
            s->err = st.description();
            return (int)st;
        }
        double dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        if (i >= warmup) {
            mn = dt < mn ? dt : mn;
            mx = dt > mx ? dt : mx;
            sum += dt;
        }
    }
    stats[0] = mn;
    stats[1] = sum / (iters > 0 ? iters : 1);
    stats[2] = mx;
    return 0;
}

}  // extern "C"
