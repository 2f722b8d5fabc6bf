/* C entry points of libtnn_rocm_host.so: the engine-side host (Instance on DEVICE_ROCM) behind plain pointers, for
 * drivers written in other languages.  Each call maps onto one method of the engine's public Instance
 * (reference include/tnn/core/instance.h:42-135) in the order the engine's own test driver uses them
 * (reference test/test.cc:101-152: SetInputMat -> Forward -> GetOutputMat).
 *
 * All int-returning functions return 0 on success and a non-zero engine status code otherwise; the text of the last
 * failure of a handle is tnn_host_last_error(handle). */
#ifndef TNN_ROCM_HOST_H_
#define TNN_ROCM_HOST_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Instance(net_config{DEVICE_ROCM, device_id, precision}, model_config{proto text, model bytes}) + Init()
 * (reference include/tnn/core/instance.h:44-49, include/tnn/core/common.h:142-183).
 * precision: 0 = PRECISION_HIGH (fp32 blobs), 1 = PRECISION_AUTO (fp16 activations), 2 = PRECISION_LOW (bf16
 * activations).
 * Returns NULL on failure and writes the status text to err[err_len]. */
void *tnn_host_create(const char *proto, size_t proto_len, const char *model, size_t model_len, int device_id,
                      int precision, char *err, size_t err_len);
/* The same with the instance created at other input shapes than the proto's: Instance::Init(interpreter,
 * min_inputs_shape, max_inputs_shape) (reference source/tnn/core/instance.cc:48-128; include/tnn/core/tnn.h:77-85
 * CreateInst(config, status, inputs_shape)).  names[i] has ndims[i] dimensions, taken one after another from dims.
 * Blob memory is planned at these shapes; later tnn_host_reshape calls to anything that fits stay allocation-free. */
void *tnn_host_create_shaped(const char *proto, size_t proto_len, const char *model, size_t model_len, int device_id,
                             int precision, int n_inputs, const char *const *names, const int *ndims, const int *dims,
                             char *err, size_t err_len);
/* Instance::Reshape (instance.h:62, reference source/tnn/core/instance.cc:143-152 ->
 * source/tnn/core/default_network.cc:456-500): new dims for the named inputs (same rank), every layer infers its
 * output shape again and its acc is reshaped; weights stay on the device.  An unknown name is TNNERR_PARAM_ERR. */
int tnn_host_reshape(void *handle, int n_inputs, const char *const *names, const int *ndims, const int *dims);
/* The first half of Instance::Init without a device: interpret the model (reference
 * source/tnn/interpreter/tnn/model_interpreter.cc:104-476), run the optimizer passes on the instance's copy of the
 * graph (source/tnn/core/default_network.cc:86-137 -> optimizer/net_optimizer_manager.cc) and infer every blob's type
 * and shape (default_network.cc:157-331).  out receives one line per layer of the optimised graph:
 * type|name|input blobs|output blobs|input dims|output dims.  Works on a machine without a GPU.
 * Returns 0, an engine status code (text in err), or -2 when out is too small. */
int tnn_host_plan(const char *proto, size_t proto_len, const char *model, size_t model_len, int precision, int n_inputs,
                  const char *const *names, const int *ndims, const int *dims, char *out, size_t out_len, char *err,
                  size_t err_len);
/* ~Instance (instance.h:46) */
void tnn_host_destroy(void *handle);
const char *tnn_host_last_error(void *handle);

/* Instance::SetInputMat (instance.h:123) from a host array.  mat_type: 0 = NCHW_FLOAT (fp32), 1 = NC_INT32,
 * 2 = RESERVED_INT8_TEST (int8 values copied as they are into an int8 blob, blob_converter_default.cc:190-193),
 * 3 = RESERVED_BFP16_TEST (bfloat16 bit patterns), 4 = RESERVED_FP16_TEST (IEEE half): the Mats the engine's layer test
 * feeds half-precision blobs with (layer_test.cc:266-275); they go into a float blob of any type.
 * name NULL or "" selects the only input. */
int tnn_host_set_input(void *handle, const char *name, const void *data, int mat_type, const int *dims, int ndims);
/* Instance::Forward (instance.h:78): runs every layer and waits for the stream */
int tnn_host_forward(void *handle);
/* Instance::ForwardAsync (instance.h:92): enqueue only; pair with tnn_host_sync */
int tnn_host_forward_async(void *handle);
int tnn_host_sync(void *handle);
/* Instance::ForwardWithCallback (instance.h:82, default_network.cc:637-668): the layers one by one, `before` called with a
 * layer's input blobs, `after` with its output blobs once the layer has finished on the device (either may be NULL). */
typedef void (*tnn_host_layer_callback)(void *user, const char *layer_name, const char *layer_type, int blobs_are_outputs,
                                        int n_blobs, const char *const *blob_names, const long long *blob_elements,
                                        const int *blob_data_types);
int tnn_host_forward_with_callback(void *handle, tnn_host_layer_callback before, tnn_host_layer_callback after, void *user);
/* Instance::ShareCommandQueue (instance.h:74): `handle` launches on `other`'s stream from now on (other must outlive
 * it); Instance::SetCpuNumThreads (instance.h:135): accepted, the device does no host-side threading of layers */
int tnn_host_share_command_queue(void *handle, void *other);
int tnn_host_set_cpu_num_threads(void *handle, int num_threads);
/* Instance::GetCommandQueue (instance.h:71): the hipStream_t the instance launches on */
void *tnn_host_stream(void *handle);
/* Instance::GetOutputMat (instance.h:128) converted to fp32 NCHW on the host.  dims must hold 8 ints. */
int tnn_host_get_output(void *handle, const char *name, float *out, size_t capacity, int *dims, int *ndims);
/* The same through a Mat of the caller's choice (mat_type as for tnn_host_set_input; RESERVED_INT8_TEST hands out an int8
 * blob's values as they are, blob_converter_default.cc:347-350); capacity in bytes. */
int tnn_host_get_output_as(void *handle, const char *name, int mat_type, void *out, size_t capacity_bytes, int *dims,
                           int *ndims);
/* The same two calls with Mats whose memory is on the device (Mat(DEVICE_ROCM, ...), the counterpart of the DEVICE_CUDA
 * branches of source/tnn/device/cuda/cuda_blob_converter.cc:62-81, 141-161): nothing crosses the bus.  The input memory
 * is the caller's and must stay unchanged until the instance's stream has passed the conversion; the output Mat belongs
 * to the instance and lives until the next call for that output. */
int tnn_host_set_input_device(void *handle, const char *name, const void *device_data, int mat_type, const int *dims,
                              int ndims);
int tnn_host_get_output_device(void *handle, const char *name, int mat_type, void **device_data, int *dims, int *ndims);
/* MatUtils::Copy (include/tnn/utils/mat_utils.h:77-79) host Mat -> DEVICE_ROCM Mat -> a second DEVICE_ROCM Mat (allocated by
 * the copy) -> host Mat `out`; mat_type as for tnn_host_set_input.  No instance is involved. */
int tnn_host_mat_copy_round_trip(const void *in, void *out, int mat_type, const int *dims, int ndims, char *err,
                                 size_t err_len);
/* BlobConverter::ConvertFromMat followed by ConvertToMat on the input blob `name` (include/tnn/utils/blob_converter.h:
 * 60-78), the flow of the engine's blob-converter unit test (test/unit_test/blob_converter_test.cc:287-349): the fp32 NCHW
 * Mat `in` enters the blob with per-channel scale and bias (n_param values each, channel = dims[1]) and the blob comes
 * back in `out` with the same scale and bias applied again.  in / out hold the blob's element count; with on_device
 * they are device addresses and the Mats are DEVICE_ROCM Mats. */
int tnn_host_input_blob_round_trip(void *handle, const char *name, const float *in, const float *scale, const float *bias,
                                   int n_param, float *out, int on_device);

/* The loop of the engine's benchmark tool (test/test.cc:101-152): `warmup` untimed and `iters` timed iterations of
 * SetInputMat for every input set so far (host copies of those Mats are kept), Forward, GetOutputMat(out_name) as
 * fp32 NCHW on the host.  stats[3] = {min, avg, max} seconds per iteration. */
int tnn_host_time_loop(void *handle, int warmup, int iters, const char *out_name, double *stats);
/* The same loop with Mats in device memory: SetInputMat with the device Mats last given to tnn_host_set_input_device,
 * Forward, GetOutputMat(out_name) as a device Mat of out_mat_type. */
int tnn_host_time_loop_device(void *handle, int warmup, int iters, const char *out_name, int out_mat_type, double *stats);

/* The optimised layer list ("Type name\n" per layer) and per-layer timing with events on the instance's stream
 * (the engine's TNN_PROFILE facility, reference source/tnn/core/profile.h:29-100).  only_type NULL or "" times every
 * layer.  tnn_host_profile_finish fills up to `capacity` mean milliseconds (layer order) and returns the layer count. */
int tnn_host_layer_count(void *handle);
const char *tnn_host_layer_summary(void *handle);
/* one line per layer of the optimised graph, layer order: name|input blobs|output blobs|input dims|output dims (blob
 * names comma separated, dims as d0,d1,..;d0,d1,.. per blob): what a per-layer profile table or a per-blob check needs */
const char *tnn_host_layer_io(void *handle);
void tnn_host_profile_start(void *handle, const char *only_type);
int tnn_host_profile_finish(void *handle, double *ms, int capacity);

#ifdef __cplusplus
}
#endif
#endif /* TNN_ROCM_HOST_H_ */
