"""ctypes front-end of the C++ host (tnn_amd/lib/libtnn_rocm_host.so): an engine Instance on DEVICE_ROCM created
from .tnnproto text + .tnnmodel bytes.  No fallback: a missing library or a failed call raises."""
import ctypes as C
import os

import numpy as np

from . import capi

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libtnn_rocm_host.so")

SIGNATURES = {
    "tnn_host_create": (C.c_void_p, [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.c_int, C.c_int, C.c_char_p,
                                     C.c_size_t]),
    "tnn_host_create_shaped": (C.c_void_p, [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.c_int, C.c_int, C.c_int,
                                            C.POINTER(C.c_char_p), C.POINTER(C.c_int), C.POINTER(C.c_int), C.c_char_p,
                                            C.c_size_t]),
    "tnn_host_reshape": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "tnn_host_plan": (C.c_int, [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_char_p),
                                C.POINTER(C.c_int), C.POINTER(C.c_int), C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]),
    "tnn_host_destroy": (None, [C.c_void_p]),
    "tnn_host_last_error": (C.c_char_p, [C.c_void_p]),
    "tnn_host_set_input": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int]),
    "tnn_host_time_loop_device": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_char_p, C.c_int, C.POINTER(C.c_double)]),
    "tnn_host_mat_copy_round_trip": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int, C.c_char_p,
                                               C.c_size_t]),
    "tnn_host_set_input_device": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int]),
    "tnn_host_get_output_device": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_int),
                                             C.POINTER(C.c_int)]),
    "tnn_host_input_blob_round_trip": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                                 C.c_void_p, C.c_int]),
    "tnn_host_forward": (C.c_int, [C.c_void_p]),
    "tnn_host_forward_async": (C.c_int, [C.c_void_p]),
    "tnn_host_sync": (C.c_int, [C.c_void_p]),
    "tnn_host_stream": (C.c_void_p, [C.c_void_p]),
    "tnn_host_forward_with_callback": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "tnn_host_share_command_queue": (C.c_int, [C.c_void_p, C.c_void_p]),
    "tnn_host_set_cpu_num_threads": (C.c_int, [C.c_void_p, C.c_int]),
    "tnn_host_get_output": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_int),
                                      C.POINTER(C.c_int)]),
    "tnn_host_get_output_as": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int, C.c_void_p, C.c_size_t, C.POINTER(C.c_int),
                                         C.POINTER(C.c_int)]),
    "tnn_host_time_loop": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_char_p, C.POINTER(C.c_double)]),
    "tnn_host_layer_count": (C.c_int, [C.c_void_p]),
    "tnn_host_layer_summary": (C.c_char_p, [C.c_void_p]),
    "tnn_host_layer_io": (C.c_char_p, [C.c_void_p]),
    "tnn_host_profile_start": (None, [C.c_void_p, C.c_char_p]),
    "tnn_host_profile_finish": (C.c_int, [C.c_void_p, C.POINTER(C.c_double), C.c_int]),
}
_lib = None


def load():
    global _lib
    if _lib is None:
        capi.load()  # the kernel library first: the host links against it
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError("%s not found: run `make -C tnn_amd/host`" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


# numpy type of the host array -> Mat type of the C API; bfloat16 has no numpy type: uint16 arrays carry its bit patterns
_MAT_CODE = {np.dtype(np.float32): 0, np.dtype(np.int32): 1, np.dtype(np.int8): 2, np.dtype(np.uint16): 3,
             np.dtype(np.float16): 4}


class HostError(RuntimeError):
    pass


def _shape_args(input_shapes):
    items = sorted(input_shapes.items())
    names = (C.c_char_p * len(items))(*[k.encode() for k, _ in items])
    ndims = (C.c_int * len(items))(*[len(v) for _, v in items])
    flat = [int(d) for _, v in items for d in v]
    dims = (C.c_int * max(len(flat), 1))(*flat)
    return len(items), names, ndims, dims


def _parse_io(lines, with_type):
    out = []
    for line in lines:
        if not line:
            continue
        f = line.split("|")
        t = f.pop(0) if with_type else None
        name, ins, outs, idims, odims = f

        def dims(sv):
            return [[int(x) for x in d.split(",") if x] for d in sv.split(";")] if sv else []

        entry = {"name": name, "inputs": [x for x in ins.split(",") if x], "outputs": [x for x in outs.split(",") if x],
                 "input_dims": dims(idims), "output_dims": dims(odims)}
        if with_type:
            entry["type"] = t
        out.append(entry)
    return out


def plan(graph_or_proto, model=None, precision="fp16", input_shapes=None):
    """The optimised graph (layer types, blobs, inferred shapes) of a model as an instance on DEVICE_ROCM would run it,
    computed on the host alone: no GPU is needed.  Raises HostError with the engine's status text."""
    lib = load()
    proto = graph_or_proto if model is not None else graph_or_proto.proto()
    model = model if model is not None else graph_or_proto.model()
    if isinstance(proto, str):
        proto = proto.encode()
    n, names, ndims, dims = _shape_args(input_shapes or {})
    out = C.create_string_buffer(1 << 22)
    err = C.create_string_buffer(1024)
    rc = lib.tnn_host_plan(proto, len(proto), model, len(model), {"fp32": 0, "fp16": 1, "bf16": 2}[precision], n, names,
                           ndims, dims, out, len(out), err, 1024)
    if rc != 0:
        raise HostError("plan failed (0x%x): %s" % (rc & 0xFFFFFFFF, err.value.decode(errors="replace")))
    return _parse_io(out.value.decode(errors="replace").splitlines(), True)


def mat_copy_round_trip(arr):
    """MatUtils::Copy host -> DEVICE_ROCM -> DEVICE_ROCM -> host of an array whose type names a Mat type"""
    a = np.ascontiguousarray(arr)
    out = np.empty_like(a)
    dims = (C.c_int * max(a.ndim, 1))(*a.shape)
    err = C.create_string_buffer(512)
    rc = load().tnn_host_mat_copy_round_trip(a.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), _MAT_CODE[a.dtype],
                                             dims, a.ndim, err, 512)
    if rc != 0:
        raise HostError("MatUtils::Copy failed (0x%x): %s" % (rc & 0xFFFFFFFF, err.value.decode(errors="replace")))
    return out


class RocmInstance:
    """precision: "fp32" (PRECISION_HIGH), "fp16" (PRECISION_AUTO: fp16 activations + fused kernels) or "bf16"
    (PRECISION_LOW: bf16 activations + fused kernels)."""

    def __init__(self, proto, model, precision="fp16", device_id=0, input_shapes=None):
        """input_shapes {name: dims}: create the instance at these shapes instead of the proto's (the engine's
        max_inputs_shape); reshape() later moves within or beyond them."""
        lib = load()
        if isinstance(proto, str):
            proto = proto.encode()
        err = C.create_string_buffer(1024)
        prec = {"fp32": 0, "fp16": 1, "bf16": 2}[precision]
        if input_shapes:
            n, names, ndims, dims = _shape_args(input_shapes)
            self._h = lib.tnn_host_create_shaped(proto, len(proto), model, len(model), device_id, prec, n, names, ndims,
                                                 dims, err, 1024)
        else:
            self._h = lib.tnn_host_create(proto, len(proto), model, len(model), device_id, prec, err, 1024)
        if not self._h:
            raise HostError("Instance::Init failed: " + err.value.decode(errors="replace"))
        self._keep = []

    @classmethod
    def from_graph(cls, graph, precision="fp16", input_shapes=None):
        return cls(graph.proto(), graph.model(), precision, input_shapes=input_shapes)

    def reshape(self, input_shapes):
        """Instance::Reshape: {input name: new dims}"""
        n, names, ndims, dims = _shape_args(input_shapes)
        self._check(load().tnn_host_reshape(self._h, n, names, ndims, dims), "Reshape")

    def _check(self, rc, what):
        if rc != 0:
            raise HostError("%s failed (0x%x): %s" % (what, rc & 0xFFFFFFFF, load().tnn_host_last_error(self._h).decode(errors="replace")))

    def set_input(self, name, arr):
        a = np.ascontiguousarray(arr)
        if a.dtype not in _MAT_CODE:
            raise TypeError("inputs are fp32 (NCHW_FLOAT), int32 (NC_INT32), int8 (RESERVED_INT8_TEST), float16 "
                            "(RESERVED_FP16_TEST) or uint16 holding bfloat16 bits (RESERVED_BFP16_TEST) host arrays")
        dims = (C.c_int * max(a.ndim, 1))(*a.shape)
        self._check(load().tnn_host_set_input(self._h, name.encode(), a.ctypes.data_as(C.c_void_p),
                                              _MAT_CODE[a.dtype], dims, a.ndim), "SetInputMat")

    def set_input_device(self, name, data_ptr, np_dtype, shape):
        """SetInputMat with a Mat in device memory (data_ptr: a device address holding `shape` elements of np_dtype, e.g. a
        torch tensor's data_ptr()); the memory must stay unchanged until the instance's stream has passed the copy"""
        dims = (C.c_int * max(len(shape), 1))(*shape)
        self._check(load().tnn_host_set_input_device(self._h, name.encode(), C.c_void_p(data_ptr), _MAT_CODE[np.dtype(np_dtype)],
                                                     dims, len(shape)), "SetInputMat (device mat)")

    def output_device(self, name, np_dtype):
        """GetOutputMat as a Mat in device memory the instance owns -> (device address, shape)"""
        ptr = C.c_void_p()
        dims = (C.c_int * 8)()
        nd = C.c_int(0)
        self._check(load().tnn_host_get_output_device(self._h, name.encode(), _MAT_CODE[np.dtype(np_dtype)], C.byref(ptr), dims,
                                                      C.byref(nd)), "GetOutputMat (device mat)")
        return ptr.value, [dims[i] for i in range(nd.value)]

    def input_blob_round_trip(self, name, arr, scale, bias, device_ptrs=None):
        """fp32 NCHW Mat -> the input blob (ConvertFromMat with per-channel scale, bias) -> fp32 NCHW Mat (ConvertToMat with
        the same scale, bias): the flow of the engine's blob-converter unit test.  device_ptrs = (in, out) device
        addresses: the same with DEVICE_ROCM Mats (arr is ignored, nothing is returned)."""
        sc, bi = np.ascontiguousarray(scale, np.float32), np.ascontiguousarray(bias, np.float32)
        assert sc.size == bi.size
        if device_ptrs is not None:
            self._check(load().tnn_host_input_blob_round_trip(self._h, name.encode(), C.c_void_p(device_ptrs[0]),
                                                              sc.ctypes.data_as(C.c_void_p), bi.ctypes.data_as(C.c_void_p),
                                                              int(sc.size), C.c_void_p(device_ptrs[1]), 1), "blob converter")
            return None
        a = np.ascontiguousarray(arr, np.float32)
        out = np.empty_like(a)
        self._check(load().tnn_host_input_blob_round_trip(self._h, name.encode(), a.ctypes.data_as(C.c_void_p),
                                                          sc.ctypes.data_as(C.c_void_p), bi.ctypes.data_as(C.c_void_p),
                                                          int(sc.size), out.ctypes.data_as(C.c_void_p), 0), "blob converter")
        return out

    def forward(self):
        self._check(load().tnn_host_forward(self._h), "Forward")

    def forward_async(self):
        self._check(load().tnn_host_forward_async(self._h), "ForwardAsync")

    def sync(self):
        self._check(load().tnn_host_sync(self._h), "Synchronize")

    def forward_with_callback(self, before=None, after=None):
        """Instance::ForwardWithCallback: before(layer_name, layer_type, [(blob, elements, data_type)]) with a layer's
        inputs, after(...) with its outputs once the layer has finished"""
        CB = C.CFUNCTYPE(None, C.c_void_p, C.c_char_p, C.c_char_p, C.c_int, C.c_int, C.POINTER(C.c_char_p),
                         C.POINTER(C.c_longlong), C.POINTER(C.c_int))

        def wrap(fn):
            if fn is None:
                return None
            return CB(lambda user, name, typ, is_out, n, names, counts, types: fn(
                name.decode(errors="replace"), typ.decode(errors="replace"), [(names[i].decode(errors="replace"), counts[i], types[i]) for i in range(n)]))
        b, a = wrap(before), wrap(after)
        self._check(load().tnn_host_forward_with_callback(self._h, C.cast(b, C.c_void_p) if b else None,
                                                          C.cast(a, C.c_void_p) if a else None, None), "ForwardWithCallback")

    def share_command_queue(self, other):
        """Instance::ShareCommandQueue: launch on `other`'s stream from now on (other must outlive this instance)"""
        self._check(load().tnn_host_share_command_queue(self._h, other._h), "ShareCommandQueue")

    def set_cpu_num_threads(self, n):
        self._check(load().tnn_host_set_cpu_num_threads(self._h, n), "SetCpuNumThreads")

    @property
    def stream(self):
        return load().tnn_host_stream(self._h)

    def output(self, name="", max_elems=1 << 25):
        buf = np.empty(max_elems, np.float32)
        dims = (C.c_int * 8)()
        nd = C.c_int(0)
        self._check(load().tnn_host_get_output(self._h, name.encode(), buf.ctypes.data_as(C.c_void_p), max_elems, dims,
                                               C.byref(nd)), "GetOutputMat")
        shape = [dims[i] for i in range(nd.value)]
        return buf[:int(np.prod(shape, dtype=np.int64))].reshape(shape).copy()

    def output_as(self, name, dtype, max_elems=1 << 25):
        """the output through a Mat of the given numpy type: float32, int32, int8 (an int8 blob's values as they are),
        float16, or uint16 (bfloat16 bit patterns)"""
        dtype = np.dtype(dtype)
        buf = np.empty(max_elems, dtype)
        dims = (C.c_int * 8)()
        nd = C.c_int(0)
        self._check(load().tnn_host_get_output_as(self._h, name.encode(), _MAT_CODE[dtype], buf.ctypes.data_as(C.c_void_p),
                                                  buf.nbytes, dims, C.byref(nd)), "GetOutputMat")
        shape = [dims[i] for i in range(nd.value)]
        return buf[:int(np.prod(shape, dtype=np.int64))].reshape(shape).copy()

    def time_loop(self, warmup, iters, out_name):
        """the engine benchmark tool's loop (SetInputMat for every input set so far + Forward + GetOutputMat per
        iteration), run natively -> (min, avg, max) seconds"""
        stats = (C.c_double * 3)()
        self._check(load().tnn_host_time_loop(self._h, warmup, iters, out_name.encode(), stats), "timing loop")
        return stats[0], stats[1], stats[2]

    def time_loop_device(self, warmup, iters, out_name, out_dtype=np.float32):
        """time_loop with the Mats in device memory (inputs: the device Mats last given to set_input_device; output: a
        device Mat of out_dtype) -> (min, avg, max) seconds"""
        stats = (C.c_double * 3)()
        self._check(load().tnn_host_time_loop_device(self._h, warmup, iters, out_name.encode(), _MAT_CODE[np.dtype(out_dtype)],
                                                     stats), "timing loop (device mats)")
        return stats[0], stats[1], stats[2]

    def layers(self):
        text = load().tnn_host_layer_summary(self._h).decode(errors="replace")
        return [tuple(line.split(" ", 1)) for line in text.splitlines() if line]

    def layer_io(self):
        """[{name, inputs, outputs, input_dims, output_dims}] for the layers of the optimised graph"""
        out = []
        for line in load().tnn_host_layer_io(self._h).decode(errors="replace").splitlines():
            name, ins, outs, din, dout = line.split("|")
            shape = lambda t: [[int(x) for x in b.split(",") if x] for b in t.split(";")] if t else []
            out.append({"name": name, "inputs": [x for x in ins.split(",") if x], "outputs": [x for x in outs.split(",") if x],
                        "input_dims": shape(din), "output_dims": shape(dout)})
        return out

    def profile_table(self, iters=10):
        """The engine's TNN_PROFILE report (source/tnn/core/profile.cc:111-201: per-layer table, the same sorted by cost,
        summary by op type, total) from hipEvent timings of `iters` eager forwards."""
        prof, io = self.profile(iters), self.layer_io()
        dims = lambda bl: " ".join("[" + ",".join(str(x) for x in d) + "]" for d in bl)
        rows = [(nm, t, ms, dims(i["input_dims"]), dims(i["output_dims"])) for (t, nm, ms), i in zip(prof, io)]

        def table(title, header, data):
            widths = [max(len(str(r[c])) for r in [header] + data) for c in range(len(header))]
            line = lambda r: "| " + " | ".join(str(v).ljust(w) for v, w in zip(r, widths)) + " |"
            bar = "-" * len(line(header))
            return "\n".join([title.center(len(bar), "="), line(header), bar] + [line(r) for r in data] + [bar, ""])

        header = ["name", "Op Type", "Kernel(ms)", "Input Dims", "Output Dims"]
        fmt = [[nm, t, "%.4f" % ms, di, do] for nm, t, ms, di, do in rows]
        by_cost = [[nm, t, "%.4f" % ms, di, do] for nm, t, ms, di, do in sorted(rows, key=lambda r: -r[2])]
        total = sum(r[2] for r in rows)
        per_type = {}
        for _, t, ms, _, _ in rows:
            per_type[t] = per_type.get(t, 0.0) + ms
        summary = [[t, "%.4f" % ms, "%.2f" % (100.0 * ms / total if total > 0 else 0.0)]
                   for t, ms in sorted(per_type.items(), key=lambda kv: -kv[1])]
        return (table("Profiling Data", header, fmt) + table("Profiling Data Sort by Cost time", header, by_cost) +
                table("Summary", ["Op Type", "Total Kernel Time(ms)", "Percent (%)"], summary) +
                "kernel runtime total: %.4f ms\n" % total)

    def profile_start(self, only_type=""):
        load().tnn_host_profile_start(self._h, only_type.encode())

    def profile_finish(self):
        """[(type, name, mean ms per forward)] since profile_start (hipEvents on the instance's stream)"""
        lib = load()
        n = lib.tnn_host_layer_count(self._h)
        ms = (C.c_double * n)()
        lib.tnn_host_profile_finish(self._h, ms, n)
        return [(t, nm, ms[i]) for i, (t, nm) in enumerate(self.layers())]

    def profile(self, iters=10):
        """per-layer mean milliseconds over `iters` forwards (hipEvent timing on the instance's stream)"""
        lib = load()
        lib.tnn_host_profile_start(self._h, b"")
        for _ in range(iters):
            self.forward()
        n = lib.tnn_host_layer_count(self._h)
        ms = (C.c_double * n)()
        lib.tnn_host_profile_finish(self._h, ms, n)
        return [(t, nm, ms[i]) for i, (t, nm) in enumerate(self.layers())]

    def close(self):
        if getattr(self, "_h", None):
            load().tnn_host_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
