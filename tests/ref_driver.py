"""ctypes front-end of oracle/_ref (the reference engine's own CPU paths, built from its sources).
Test infrastructure only; absent on machines where oracle/_ref was never built."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "oracle", "_ref", "libtnn_ref_driver.so")
_lib = None


def available():
    return os.path.exists(LIB)


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(LIB)
        _lib.tnn_ref_create.restype = C.c_void_p
        _lib.tnn_ref_create.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.c_char_p, C.c_int,
                                        C.c_char_p, C.c_size_t]
        _lib.tnn_ref_create_shaped.restype = C.c_void_p
        _lib.tnn_ref_create_shaped.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.c_char_p, C.c_int,
                                               C.c_char_p, C.c_char_p, C.c_char_p, C.c_size_t]
        _lib.tnn_ref_reshape.argtypes = [C.c_void_p, C.c_char_p]
        _lib.tnn_ref_destroy.argtypes = [C.c_void_p]
        _lib.tnn_ref_set_input.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int]
        _lib.tnn_ref_forward.argtypes = [C.c_void_p]
        _lib.tnn_ref_input_blob_round_trip.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                                       C.c_void_p, C.c_int]
        _lib.tnn_ref_mat_copy_round_trip.argtypes = [C.c_char_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_char_p,
                                                     C.c_size_t]
        _lib.tnn_ref_set_input_device.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_int, C.POINTER(C.c_int), C.c_int]
        _lib.tnn_ref_get_output_device.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int),
                                                   C.POINTER(C.c_int)]
        _lib.tnn_ref_forward_memory_size.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
        _lib.tnn_ref_set_forward_memory.argtypes = [C.c_void_p, C.c_void_p]
        _lib.tnn_ref_get_output.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_int),
                                            C.POINTER(C.c_int)]
        _lib.tnn_ref_get_output_as.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_void_p, C.c_size_t, C.POINTER(C.c_int),
                                               C.POINTER(C.c_int)]
        _lib.tnn_ref_output_data_type.argtypes = [C.c_void_p, C.c_char_p]
        _lib.tnn_ref_last_error.restype = C.c_char_p
        _lib.tnn_ref_last_error.argtypes = [C.c_void_p]
        _lib.tnn_ref_time_forward.restype = C.c_double
        _lib.tnn_ref_time_forward.argtypes = [C.c_void_p, C.c_int, C.c_int]
        _lib.tnn_ref_time_loop.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_char_p, C.POINTER(C.c_double)]
    return _lib


def _shape_spec(shapes):
    return ";".join("%s:%s" % (k, ",".join(str(int(d)) for d in v)) for k, v in (shapes or {}).items()).encode()


def mat_copy_round_trip(device, arr):
    """the reference's MatUtils::Copy host -> `device` -> `device` -> host of an fp32 array"""
    a = np.ascontiguousarray(arr, np.float32)
    out = np.empty_like(a)
    dims = (C.c_int * a.ndim)(*a.shape)
    err = C.create_string_buffer(512)
    rc = lib().tnn_ref_mat_copy_round_trip(device.encode(), a.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), dims,
                                           a.ndim, err, 512)
    if rc != 0:
        raise RuntimeError("MatUtils::Copy failed (0x%x): %s" % (rc & 0xFFFFFFFF, err.value.decode(errors="replace")))
    return out


class RefSession:
    def __init__(self, graph, device="NAIVE", threads=0, min_shapes=None, max_shapes=None):
        proto = graph.proto().encode()
        model = graph.model()
        err = C.create_string_buffer(512)
        self.h = lib().tnn_ref_create_shaped(proto, len(proto), model, len(model), device.encode(), threads,
                                             _shape_spec(min_shapes), _shape_spec(max_shapes), err, 512)
        if not self.h:
            raise RuntimeError("reference engine refused the model: " + err.value.decode())
        self._keep = []

    def _check(self, rc, what):
        if rc != 0:
            raise RuntimeError("%s failed (0x%x): %s" % (what, rc, lib().tnn_ref_last_error(self.h).decode()))

    def set_input(self, name, arr):
        a = np.ascontiguousarray(arr)
        assert a.dtype in (np.float32, np.int32, np.int8)   # int8: RESERVED_INT8_TEST, copied as it is into an int8 blob
        self._keep.append(a)
        dims = (C.c_int * a.ndim)(*a.shape)
        self._check(lib().tnn_ref_set_input(self.h, name.encode(), a.ctypes.data_as(C.c_void_p),
                                            {np.dtype(np.float32): 0, np.dtype(np.int32): 1, np.dtype(np.int8): 2}[a.dtype],
                                            dims, a.ndim), "SetInputMat")

    def input_blob_round_trip(self, name, arr, scale, bias, device_ptrs=None):
        """fp32 NCHW Mat -> the input blob (ConvertFromMat with per-channel scale, bias) -> fp32 NCHW Mat (ConvertToMat with
        the same scale, bias), through a BlobConverter of the blob's device.  device_ptrs = (in, out): Mats in the memory
        of the blob's device at these addresses instead of host Mats (arr is ignored, nothing is returned)."""
        sc, bi = np.ascontiguousarray(scale, np.float32), np.ascontiguousarray(bias, np.float32)
        assert sc.size == bi.size
        if device_ptrs is not None:
            self._check(lib().tnn_ref_input_blob_round_trip(self.h, name.encode(), C.c_void_p(device_ptrs[0]),
                                                            sc.ctypes.data_as(C.c_void_p), bi.ctypes.data_as(C.c_void_p),
                                                            int(sc.size), C.c_void_p(device_ptrs[1]), 1), "blob converter")
            return None
        a = np.ascontiguousarray(arr, np.float32)
        out = np.empty_like(a)
        self._check(lib().tnn_ref_input_blob_round_trip(self.h, name.encode(), a.ctypes.data_as(C.c_void_p),
                                                        sc.ctypes.data_as(C.c_void_p), bi.ctypes.data_as(C.c_void_p),
                                                        int(sc.size), out.ctypes.data_as(C.c_void_p), 0), "blob converter")
        return out

    def set_input_device(self, name, data_ptr, is_int32, shape):
        """SetInputMat with a Mat in the memory of the session's device at data_ptr (fp32, or int32 values)"""
        dims = (C.c_int * len(shape))(*shape)
        self._check(lib().tnn_ref_set_input_device(self.h, name.encode(), C.c_void_p(data_ptr), 1 if is_int32 else 0, dims,
                                                   len(shape)), "SetInputMat (device mat)")

    def output_device(self, name):
        """GetOutputMat as an fp32 Mat in the memory of the session's device -> (address, shape); the Mat stays with the
        session until the next call"""
        ptr = C.c_void_p()
        dims = (C.c_int * 8)()
        nd = C.c_int(0)
        self._check(lib().tnn_ref_get_output_device(self.h, name.encode(), C.byref(ptr), dims, C.byref(nd)),
                    "GetOutputMat (device mat)")
        return ptr.value, [dims[i] for i in range(nd.value)]

    def reshape(self, shapes):
        self._check(lib().tnn_ref_reshape(self.h, _shape_spec(shapes)), "Reshape")
        self._keep = []

    def forward(self):
        self._check(lib().tnn_ref_forward(self.h), "Forward")

    def forward_memory_size(self):
        n = C.c_int(0)
        self._check(lib().tnn_ref_forward_memory_size(self.h, C.byref(n)), "GetForwardMemorySize")
        return n.value

    def set_forward_memory(self, pointer):
        self._check(lib().tnn_ref_set_forward_memory(self.h, C.c_void_p(pointer)), "SetForwardMemory")

    def output(self, name, max_elems=1 << 26):
        buf = np.empty(max_elems, np.float32)
        dims = (C.c_int * 8)()
        nd = C.c_int(0)
        self._check(lib().tnn_ref_get_output(self.h, name.encode(), buf.ctypes.data_as(C.c_void_p), max_elems, dims,
                                             C.byref(nd)), "GetOutputMat")
        shape = [dims[i] for i in range(nd.value)]
        return buf[:int(np.prod(shape))].reshape(shape).copy()

    def output_data_type(self, name):
        """0 float, 1 half, 2 int8, 3 int32, 4 bf16: the output blob's type inside the network"""
        return lib().tnn_ref_output_data_type(self.h, name.encode())

    def output_as(self, name, dtype, max_elems=1 << 26):
        """the output through a Mat of the given numpy type (float32, int32, or int8 = RESERVED_INT8_TEST)"""
        dtype = np.dtype(dtype)
        buf = np.empty(max_elems, dtype)
        dims = (C.c_int * 8)()
        nd = C.c_int(0)
        code = {np.dtype(np.float32): 0, np.dtype(np.int32): 1, np.dtype(np.int8): 2}[dtype]
        self._check(lib().tnn_ref_get_output_as(self.h, name.encode(), code, buf.ctypes.data_as(C.c_void_p), buf.nbytes,
                                                dims, C.byref(nd)), "GetOutputMat")
        shape = [dims[i] for i in range(nd.value)]
        return buf[:int(np.prod(shape))].reshape(shape).copy()

    def time_forward(self, warmup, iters):
        t = lib().tnn_ref_time_forward(self.h, warmup, iters)
        if t < 0:
            raise RuntimeError("Forward failed while timing")
        return t

    def time_loop(self, warmup, iters, out_name):
        """the reference's own benchmark loop (test/test.cc:101-152): SetInputMat + Forward + GetOutputMat per
        iteration -> (min, avg, max) seconds"""
        stats = (C.c_double * 3)()
        self._check(lib().tnn_ref_time_loop(self.h, warmup, iters, out_name.encode(), stats), "timing loop")
        return stats[0], stats[1], stats[2]

    def close(self):
        if self.h:
            lib().tnn_ref_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()


def time_encoder(cfg, weights, ids, seg, mask, one_thread_seqs=1):
    """CPU baseline of the benchmark: the reference's DEVICE_X86 path on the same synthetic encoder, timed with the
    loop of the reference's own benchmark tool (test/test.cc:101-152: warm-up 5, 20 timed iterations of SetInputMat +
    Forward + GetOutputMat; min / avg / max) on all host cores, and again on ONE thread with a reduced loop (1 warm-up,
    2 timed iterations on `one_thread_seqs` sequences), which keeps the whole leg near half a minute."""
    from tnn_amd import tnnmodel
    B, S = ids.shape
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))

    def run(n_seq, n_threads, warmup, iters):
        g = tnnmodel.encoder_graph(cfg, weights, n_seq, S)
        s = RefSession(g, "X86", n_threads)
        s.set_input("input_ids", ids[:n_seq].astype(np.int32))
        s.set_input("token_type_ids", seg[:n_seq].astype(np.int32))
        s.set_input("attention_bias", mask[:n_seq].reshape(n_seq, 1, 1, S).astype(np.float32))
        mn, avg, mx = s.time_loop(warmup, iters, "last_hidden")
        s.close()
        return mn, avg, mx

    mn, avg, mx = run(B, threads, 5, 20)
    n1 = min(one_thread_seqs, B)
    mn1, avg1, mx1 = run(n1, 1, 1, 2)
    return {"value": B / avg, "unit": "sequences/s", "cores": threads, "kind": "reference",
            "ms_per_forward": {"min": mn * 1e3, "avg": avg * 1e3, "max": mx * 1e3},
            "one_thread": {"value": n1 / avg1, "unit": "sequences/s", "cores": 1,
                           "ms_per_forward": {"min": mn1 * 1e3, "avg": avg1 * 1e3, "max": mx1 * 1e3},
                           "sample": "%d sequence(s), 1 warm-up + 2 timed iterations" % n1},
            "sample": "%d sequences (S=%d) through all %d layers on the reference engine's DEVICE_X86 path (fp32, AVX2 + "
                      "OpenMP; its MatMul/Softmax/LayerNorm kernels are single-threaded), the reference benchmark "
                      "tool's loop: 5 warm-up + 20 timed iterations of SetInputMat + Forward + GetOutputMat" % (B, S, cfg.layers)}
