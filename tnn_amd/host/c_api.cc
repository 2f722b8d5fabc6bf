// C entry points over the host (Instance on DEVICE_ROCM) for drivers written in other languages:
// the Python bench and tests create an instance from proto text + model bytes, feed host arrays,
// call Forward and read outputs back — the same sequence as the engine's TNNTest
// (test/test.cc:101-152: ConvertFromMat -> Forward -> ConvertToMat).
#include <chrono>
#include <map>
#include <cstdio>
#include <cstring>
#include <sstream>
#include <string>

#include "tnn_host.h"
#include "tnn_rocm.h"
#include "tnn_rocm_host.h"

using namespace TNN_NS;

namespace {
struct Handle {
    std::shared_ptr<Instance> inst;
    std::string err;
    std::string summary;
    std::map<std::string, std::shared_ptr<Mat>> inputs;  // host copies of the last Mats set, for tnn_host_time_loop
    std::map<std::string, std::shared_ptr<Mat>> device_inputs;  // the device Mats last set (the caller's memory)
};
int fail(Handle *h, const Status &st) {
    h->err = st.description();
    return (int)st == 0 ? -1 : (int)st;
}
}  // namespace

extern "C" {
#define HOST_API __attribute__((visibility("default")))

// precision: 0 = fp32 blobs (PRECISION_HIGH), 1 = fp16 activations (PRECISION_AUTO), 2 = bf16 activations
// (PRECISION_LOW).  Returns NULL on failure and
// writes the status text to err.
HOST_API void *tnn_host_create(const char *proto, size_t proto_len, const char *model, size_t model_len, int device_id,
                               int precision, char *err, size_t err_len) {
    auto h = new Handle;
    NetworkConfig nc;
    nc.device_type = DEVICE_ROCM;
    nc.device_id   = device_id;
    nc.precision   = precision == 0 ? PRECISION_HIGH : (precision == 2 ? PRECISION_LOW : PRECISION_AUTO);
    ModelConfig mc;
    mc.params.push_back(std::string(proto, proto_len));
    mc.params.push_back(std::string(model, model_len));
    h->inst   = std::make_shared<Instance>(nc, mc);
    Status st = h->inst->Init();
    if (st != TNN_OK) {
        if (err && err_len)
            snprintf(err, err_len, "%s", st.description().c_str());
        delete h;
        return nullptr;
    }
    return h;
}

// As tnn_host_create, at other input shapes than the proto's (the max_inputs_shape of instance.cc:48-128): n_inputs
// names, ndims[i] dimensions each, taken one after another from dims.
HOST_API void *tnn_host_create_shaped(const char *proto, size_t proto_len, const char *model, size_t model_len, int device_id,
                                      int precision, int n_inputs, const char *const *names, const int *ndims, const int *dims,
                                      char *err, size_t err_len) {
    auto h = new Handle;
    NetworkConfig nc;
    nc.device_type = DEVICE_ROCM;
    nc.device_id   = device_id;
    nc.precision   = precision == 0 ? PRECISION_HIGH : (precision == 2 ? PRECISION_LOW : PRECISION_AUTO);
    ModelConfig mc;
    mc.params.push_back(std::string(proto, proto_len));
    mc.params.push_back(std::string(model, model_len));
    InputShapesMap shapes;
    for (int i = 0, k = 0; i < n_inputs; k += ndims[i], ++i)
        shapes[names[i]] = DimsVector(dims + k, dims + k + ndims[i]);
    h->inst   = std::make_shared<Instance>(nc, mc);
    Status st = h->inst->Init(InputShapesMap(), shapes);
    if (st != TNN_OK) {
        if (err && err_len)
            snprintf(err, err_len, "%s", st.description().c_str());
        delete h;
        return nullptr;
    }
    return h;
}

// Interprets the model, runs the optimizer passes and infers every blob's type and shape, without a device context
// (works on a machine without a GPU).  Writes the optimised graph as tnn_host_layer_io does, each line prefixed with the
// layer's type and a '|'.  Returns 0, a status code (text in err), or -2 when out is too small.
HOST_API int tnn_host_plan(const char *proto, size_t proto_len, const char *model, size_t model_len, int precision,
                           int n_inputs, const char *const *names, const int *ndims, const int *dims, char *out,
                           size_t out_len, char *err, size_t err_len) {
    NetworkConfig nc;
    nc.device_type = DEVICE_ROCM;
    nc.precision   = precision == 0 ? PRECISION_HIGH : (precision == 2 ? PRECISION_LOW : PRECISION_AUTO);
    ModelConfig mc;
    mc.params.push_back(std::string(proto, proto_len));
    mc.params.push_back(std::string(model, model_len));
    InputShapesMap shapes;
    for (int i = 0, k = 0; i < n_inputs; k += ndims[i], ++i)
        shapes[names[i]] = DimsVector(dims + k, dims + k + ndims[i]);
    ModelInterpreter interp;
    Status st = interp.Interpret(mc.params);
    DefaultNetwork net;
    if (st == TNN_OK)
        st = net.Plan(nc, &interp, shapes);
    if (st != TNN_OK) {
        if (err && err_len)
            snprintf(err, err_len, "%s", st.description().c_str());
        return (int)st == 0 ? -1 : (int)st;
    }
    std::istringstream types(net.LayerSummary()), io(net.LayerIo());
    std::string text, t, l;
    while (std::getline(types, t) && std::getline(io, l))
        text += t.substr(0, t.find(' ')) + "|" + l + "\n";
    if (text.size() + 1 > out_len)
        return -2;
    memcpy(out, text.c_str(), text.size() + 1);
    return 0;
}

// Instance::Reshape (instance.cc:143-152): new dims for the named inputs; the other inputs keep theirs.
HOST_API int tnn_host_reshape(void *hp, int n_inputs, const char *const *names, const int *ndims, const int *dims) {
    auto h = static_cast<Handle *>(hp);
    InputShapesMap shapes;
    for (int i = 0, k = 0; i < n_inputs; k += ndims[i], ++i)
        shapes[names[i]] = DimsVector(dims + k, dims + k + ndims[i]);
    Status st = h->inst->Reshape(shapes);
    return st == TNN_OK ? 0 : fail(h, st);
}

HOST_API void tnn_host_destroy(void *hp) { delete static_cast<Handle *>(hp); }
HOST_API const char *tnn_host_last_error(void *hp) { return static_cast<Handle *>(hp)->err.c_str(); }

// mat_type: 0 NCHW_FLOAT (fp32 host data), 1 NC_INT32, 2 RESERVED_INT8_TEST (int8 host data, copied as it is into an
// int8 blob: blob_converter_default.cc:190-193, 347-350)
// 3 RESERVED_BFP16_TEST (bfloat16 bit patterns), 4 RESERVED_FP16_TEST (IEEE half): the Mats the engine's layer test
// feeds half-precision blobs with (layer_test.cc:266-275)
static MatType MatTypeOf(int code) {
    switch (code) {
        case 1: return NC_INT32;
        case 2: return RESERVED_INT8_TEST;
        case 3: return RESERVED_BFP16_TEST;
        case 4: return RESERVED_FP16_TEST;
        default: return NCHW_FLOAT;
    }
}
static size_t MatElemBytes(int code) { return code == 2 ? 1 : ((code == 3 || code == 4) ? 2 : 4); }

HOST_API int tnn_host_set_input(void *hp, const char *name, const void *data, int mat_type, const int *dims, int ndims) {
    auto h = static_cast<Handle *>(hp);
    DimsVector d(dims, dims + ndims);
    auto mat  = std::make_shared<Mat>(DEVICE_NAIVE, MatTypeOf(mat_type), d, const_cast<void *>(data));
    Status st = h->inst->SetInputMat(mat, MatConvertParam(), name ? name : "");
    if (st != TNN_OK)
        return fail(h, st);
    auto keep = std::make_shared<Mat>(DEVICE_NAIVE, mat->GetMatType(), d);  // owns its memory
    if (keep->GetData() && data)
        memcpy(keep->GetData(), data, (size_t)DimsVectorUtils::Count(d) * MatElemBytes(mat_type));
    h->inputs[name ? name : ""] = keep;
    return 0;
}

// SetInputMat with a Mat whose memory is on the device already (Mat(DEVICE_ROCM, type, dims, pointer)): nothing crosses
// the bus, the converter copies or converts on the instance's stream.  The caller keeps the memory alive and unchanged
// until that stream has passed the conversion (tnn_host_sync, or any Forward).
HOST_API int tnn_host_set_input_device(void *hp, const char *name, const void *device_data, int mat_type, const int *dims,
                                       int ndims) {
    auto h = static_cast<Handle *>(hp);
    DimsVector d(dims, dims + ndims);
    auto mat  = std::make_shared<Mat>(DEVICE_ROCM, MatTypeOf(mat_type), d, const_cast<void *>(device_data));
    Status st = h->inst->SetInputMat(mat, MatConvertParam(), name ? name : "");
    if (st != TNN_OK)
        return fail(h, st);
    h->device_inputs[name ? name : ""] = mat;
    return 0;
}

// GetOutputMat on the device: the output as a Mat of the given type in device memory the instance owns (valid until the
// next call for this output or the instance's end).  *device_data receives its address.
HOST_API int tnn_host_get_output_device(void *hp, const char *name, int mat_type, void **device_data, int *dims, int *ndims) {
    auto h = static_cast<Handle *>(hp);
    std::shared_ptr<Mat> mat;
    Status st = h->inst->GetOutputMat(mat, MatConvertParam(), name ? name : "", DEVICE_ROCM, MatTypeOf(mat_type));
    if (st != TNN_OK)
        return fail(h, st);
    DimsVector d = mat->GetDims();
    if (ndims)
        *ndims = (int)d.size();
    if (dims)
        for (size_t i = 0; i < d.size() && i < 8; ++i)
            dims[i] = d[i];
    if (device_data)
        *device_data = mat->GetData();
    return 0;
}

// MatUtils::Copy (include/tnn/utils/mat_utils.h:77-79) three times: the host Mat `in` into a DEVICE_ROCM Mat the engine
// allocates, that one into a second DEVICE_ROCM Mat, and that one back into the host Mat `out`.
HOST_API int tnn_host_mat_copy_round_trip(const void *in, void *out, int mat_type, const int *dims, int ndims, char *err,
                                          size_t err_len) {
    DimsVector d(dims, dims + ndims);
    Mat src(DEVICE_NAIVE, MatTypeOf(mat_type), d, const_cast<void *>(in));
    Mat first(DEVICE_ROCM, MatTypeOf(mat_type), d), second(DEVICE_ROCM, MatTypeOf(mat_type), d, nullptr);
    Mat back(DEVICE_NAIVE, MatTypeOf(mat_type), d, out);
    Status st = MatUtils::Copy(src, first, nullptr);
    if (st == TNN_OK)
        st = MatUtils::Copy(first, second, nullptr);  // `second` has no memory yet: Copy allocates it on its device
    if (st == TNN_OK)
        st = MatUtils::Copy(second, back, nullptr);
    if (st != TNN_OK) {
        if (err && err_len)
            snprintf(err, err_len, "%s", st.description().c_str());
        return (int)st == 0 ? -1 : (int)st;
    }
    return 0;
}

// The flow of the engine's blob-converter unit test (test/unit_test/blob_converter_test.cc:287-349) on an input blob of
// this instance: fp32 NCHW Mat in with per-channel scale and bias, the blob back out as an fp32 NCHW Mat with the same
// scale and bias applied again.
HOST_API int tnn_host_input_blob_round_trip(void *hp, const char *name, const float *in, const float *scale,
                                            const float *bias, int n_param, float *out, int on_device) {
    auto h = static_cast<Handle *>(hp);
    BlobMap blobs;
    Status st = h->inst->GetAllInputBlobs(blobs);
    if (st != TNN_OK)
        return fail(h, st);
    auto it = blobs.find(name ? name : "");
    if (it == blobs.end())
        return fail(h, Status(TNNERR_PARAM_ERR, std::string("no input blob named ") + (name ? name : "")));
    void *queue = nullptr;
    h->inst->GetCommandQueue(&queue);
    MatConvertParam param;
    param.scale.assign(scale, scale + n_param);
    param.bias.assign(bias, bias + n_param);
    DimsVector dims = it->second->GetBlobDesc().dims;
    BlobConverter converter(it->second);
    const DeviceType where = on_device ? DEVICE_ROCM : DEVICE_NAIVE;  // in / out are device addresses then
    Mat mat_in(where, NCHW_FLOAT, dims, const_cast<float *>(in));
    st = converter.ConvertFromMat(mat_in, param, queue);
    if (st != TNN_OK)
        return fail(h, st);
    Mat mat_out(where, NCHW_FLOAT, dims, out);
    st = converter.ConvertToMat(mat_out, param, queue);
    return st == TNN_OK ? 0 : fail(h, st);
}

// The loop of the engine's benchmark tool (test/test.cc:101-152): per iteration every input Mat goes in
// (SetInputMat with the Mats of the last tnn_host_set_input calls), Forward, and the output Mat comes out
// (GetOutputMat as fp32 NCHW on the host).  stats = {min, avg, max} seconds over the timed iterations.
HOST_API int tnn_host_time_loop(void *hp, int warmup, int iters, const char *out_name, double *stats) {
    auto h = static_cast<Handle *>(hp);
    double mn = 1e30, mx = 0.0, sum = 0.0;
    for (int i = 0; i < warmup + iters; ++i) {
        auto t0 = std::chrono::steady_clock::now();
        for (auto &kv : h->inputs) {
            Status st = h->inst->SetInputMat(kv.second, MatConvertParam(), kv.first);
            if (st != TNN_OK)
                return fail(h, st);
        }
        Status st = h->inst->Forward();
        std::shared_ptr<Mat> mat;
        if (st == TNN_OK)
            st = h->inst->GetOutputMat(mat, MatConvertParam(), out_name ? out_name : "", DEVICE_NAIVE, NCHW_FLOAT);
        if (st != TNN_OK)
            return fail(h, st);
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

// The same loop for a caller whose data lives on the device: SetInputMat with the device Mats last given
// (tnn_host_set_input_device), Forward, GetOutputMat as a device Mat of `out_mat_type`; nothing crosses the bus.
HOST_API int tnn_host_time_loop_device(void *hp, int warmup, int iters, const char *out_name, int out_mat_type, double *stats) {
    auto h = static_cast<Handle *>(hp);
    if (h->device_inputs.empty())
        return fail(h, Status(TNNERR_PARAM_ERR, "no device Mat has been set as an input"));
    double mn = 1e30, mx = 0.0, sum = 0.0;
    for (int i = 0; i < warmup + iters; ++i) {
        auto t0 = std::chrono::steady_clock::now();
        for (auto &kv : h->device_inputs) {
            Status st = h->inst->SetInputMat(kv.second, MatConvertParam(), kv.first);
            if (st != TNN_OK)
                return fail(h, st);
        }
        Status st = h->inst->Forward();
        std::shared_ptr<Mat> mat;
        if (st == TNN_OK)
            st = h->inst->GetOutputMat(mat, MatConvertParam(), out_name ? out_name : "", DEVICE_ROCM, MatTypeOf(out_mat_type));
        if (st != TNN_OK)
            return fail(h, st);
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

HOST_API int tnn_host_forward(void *hp) {
    auto h    = static_cast<Handle *>(hp);
    Status st = h->inst->Forward();
    return st == TNN_OK ? 0 : fail(h, st);
}

// enqueue only; pair with tnn_host_sync
HOST_API int tnn_host_forward_async(void *hp) {
    auto h    = static_cast<Handle *>(hp);
    Status st = h->inst->ForwardAsync(nullptr);
    return st == TNN_OK ? 0 : fail(h, st);
}

HOST_API int tnn_host_sync(void *hp) {
    auto h  = static_cast<Handle *>(hp);
    void *q = nullptr;
    h->inst->GetCommandQueue(&q);
    int rc = tnn_rocm_stream_sync(q);
    if (rc != 0)
        h->err = tnn_rocm_last_error();
    return rc;
}

// Instance::ForwardWithCallback for C callers: `before` / `after` receive the layer's name and type, whether the blobs
// are the layer's outputs, their count and, per blob, name, element count and data type
HOST_API int tnn_host_forward_with_callback(void *hp, tnn_host_layer_callback before, tnn_host_layer_callback after, void *user) {
    auto h    = static_cast<Handle *>(hp);
    auto wrap = [user](tnn_host_layer_callback cb, int is_output) -> BlobStatisticCallback {
        if (!cb)
            return nullptr;
        return [cb, user, is_output](std::vector<Blob *> &blobs, LayerInfo *info) {
            std::vector<const char *> names;
            std::vector<long long> counts;
            std::vector<int> types;
            for (auto b : blobs) {
                names.push_back(b->GetBlobDesc().name.c_str());
                counts.push_back((long long)DimsVectorUtils::Count(b->GetBlobDesc().dims));
                types.push_back((int)b->GetBlobDesc().data_type);
            }
            cb(user, info ? info->name.c_str() : "", info ? info->type_str.c_str() : "", is_output, (int)blobs.size(),
               names.data(), counts.data(), types.data());
        };
    };
    Status st = h->inst->ForwardWithCallback(wrap(before, 0), wrap(after, 1));
    return st == TNN_OK ? 0 : fail(h, st);
}

HOST_API int tnn_host_share_command_queue(void *hp, void *other) {
    auto h    = static_cast<Handle *>(hp);
    Status st = h->inst->ShareCommandQueue(other ? static_cast<Handle *>(other)->inst.get() : nullptr);
    return st == TNN_OK ? 0 : fail(h, st);
}

HOST_API int tnn_host_set_cpu_num_threads(void *hp, int num_threads) {
    auto h    = static_cast<Handle *>(hp);
    Status st = h->inst->SetCpuNumThreads(num_threads);
    return st == TNN_OK ? 0 : fail(h, st);
}

HOST_API void *tnn_host_stream(void *hp) {
    void *q = nullptr;
    static_cast<Handle *>(hp)->inst->GetCommandQueue(&q);
    return q;
}

HOST_API int tnn_host_get_output(void *hp, const char *name, float *out, size_t capacity, int *dims, int *ndims) {
    auto h = static_cast<Handle *>(hp);
    std::shared_ptr<Mat> mat;
    Status st = h->inst->GetOutputMat(mat, MatConvertParam(), name ? name : "", DEVICE_NAIVE, NCHW_FLOAT);
    if (st != TNN_OK)
        return fail(h, st);
    DimsVector d = mat->GetDims();
    size_t count = (size_t)DimsVectorUtils::Count(d);
    if (ndims)
        *ndims = (int)d.size();
    if (dims)
        for (size_t i = 0; i < d.size() && i < 8; ++i)
            dims[i] = d[i];
    if (count > capacity) {
        h->err = "output buffer too small";
        return -2;
    }
    memcpy(out, mat->GetData(), count * sizeof(float));
    return 0;
}

// GetOutputMat through a Mat of the caller's choice (codes of tnn_host_set_input); capacity in bytes
HOST_API int tnn_host_get_output_as(void *hp, const char *name, int mat_type, void *out, size_t capacity_bytes, int *dims,
                                    int *ndims) {
    auto h = static_cast<Handle *>(hp);
    std::shared_ptr<Mat> mat;
    Status st = h->inst->GetOutputMat(mat, MatConvertParam(), name ? name : "", DEVICE_NAIVE, MatTypeOf(mat_type));
    if (st != TNN_OK)
        return fail(h, st);
    DimsVector d = mat->GetDims();
    size_t bytes = (size_t)DimsVectorUtils::Count(d) * MatElemBytes(mat_type);
    if (ndims)
        *ndims = (int)d.size();
    if (dims)
        for (size_t i = 0; i < d.size() && i < 8; ++i)
            dims[i] = d[i];
    if (bytes > capacity_bytes) {
        h->err = "output buffer too small";
        return -2;
    }
    memcpy(out, mat->GetData(), bytes);
    return 0;
}

HOST_API int tnn_host_layer_count(void *hp) { return static_cast<Handle *>(hp)->inst->GetNetwork()->LayerCount(); }

// "Type name\n" per layer of the optimised graph
HOST_API const char *tnn_host_layer_summary(void *hp) {
    auto h     = static_cast<Handle *>(hp);
    h->summary = h->inst->GetNetwork()->LayerSummary();
    return h->summary.c_str();
}

HOST_API const char *tnn_host_layer_io(void *hp) {
    auto h     = static_cast<Handle *>(hp);
    h->summary = h->inst->GetNetwork()->LayerIo();
    return h->summary.c_str();
}

// only_type: NULL or "" times every layer, otherwise only layers of that type string
HOST_API void tnn_host_profile_start(void *hp, const char *only_type) {
    static_cast<Handle *>(hp)->inst->GetNetwork()->StartProfile(only_type ? only_type : "");
}

// Fills up to `capacity` entries with the per-layer mean milliseconds since tnn_host_profile_start; returns the
// number of layers.  Names come from tnn_host_layer_summary (same order).
HOST_API int tnn_host_profile_finish(void *hp, double *ms, int capacity) {
    auto prof = static_cast<Handle *>(hp)->inst->GetNetwork()->FinishProfile();
    for (int i = 0; i < (int)prof.size() && i < capacity; ++i)
        ms[i] = prof[i].calls > 0 ? prof[i].ms / prof[i].calls : 0.0;
    return (int)prof.size();
}
}
