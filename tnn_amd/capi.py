"""ctypes binding of the C ABI declared in include/tnn_rocm.h.

The library is loaded from tnn_amd/lib/libtnn_rocm.so (built in-tree by `python -m tnn_amd.build`).
There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libtnn_rocm.so")

F32, F16, I8, I32, BF16 = 0, 1, 2, 3, 4
EPI_NONE, EPI_BIAS, EPI_GELU, EPI_RESIDUAL = 0, 1, 2, 4

_vp, _i, _l, _f, _sz = C.c_void_p, C.c_int, C.c_long, C.c_float, C.c_size_t
_ip = C.POINTER(C.c_int)

# name -> argtypes; every function returns int
SIGNATURES = {
    "tnn_rocm_device_count": [_ip],
    "tnn_rocm_set_device": [_i],
    "tnn_rocm_device_name": [_i, C.c_char_p, _sz],
    "tnn_rocm_malloc": [C.POINTER(_vp), _sz],
    "tnn_rocm_free": [_vp],
    "tnn_rocm_malloc_host": [C.POINTER(_vp), _sz],
    "tnn_rocm_free_host": [_vp],
    "tnn_rocm_memset": [_vp, _i, _sz, _vp],
    "tnn_rocm_memcpy_h2d": [_vp, _vp, _sz, _vp],
    "tnn_rocm_memcpy_d2h": [_vp, _vp, _sz, _vp],
    "tnn_rocm_memcpy_d2d": [_vp, _vp, _sz, _vp],
    "tnn_rocm_stream_create": [C.POINTER(_vp)],
    "tnn_rocm_stream_destroy": [_vp],
    "tnn_rocm_stream_sync": [_vp],
    "tnn_rocm_graph_begin_capture": [_vp],
    "tnn_rocm_graph_end_capture": [_vp, C.POINTER(_vp)],
    "tnn_rocm_graph_launch": [_vp, _vp],
    "tnn_rocm_graph_destroy": [_vp],
    "tnn_rocm_event_create": [C.POINTER(_vp)],
    "tnn_rocm_event_destroy": [_vp],
    "tnn_rocm_event_record": [_vp, _vp],
    "tnn_rocm_event_elapsed_ms": [_vp, _vp, C.POINTER(_f)],
    "tnn_rocm_gemm": [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i],
    "tnn_rocm_gemm_i8": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _i, _f],
    "tnn_rocm_gemm_i8_dequant_residual": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _i, _i, _f, _vp],
    "tnn_rocm_gemm_i8_qkv_split": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i],
    "tnn_rocm_attention": [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _l, _l, _l, _l, _l, _l, _l, _l, _l, _f,
                           _vp, _vp],
    "tnn_rocm_attention_vt": [_vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _l, _l, _l, _l, _l, _l, _l, _l, _l, _l, _l,
                              _l, _f, _vp, _vp],
    "tnn_rocm_attention_vt_q8": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _l, _l, _l, _l, _l, _l, _l, _l, _l,
                                 _l, _l, _l, _f, _vp, _vp, _i],
    "tnn_rocm_gemm_i8_lut": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "tnn_rocm_gemm_qkv_split": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i],
    "tnn_rocm_gemm_ln": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "tnn_rocm_gemm_qkv_split_ln": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i],
    "tnn_rocm_gemm_residual_ln": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp],
    "tnn_rocm_mask_to_kv_len": [_vp, _vp, _vp, _i, _i, _f],
    "tnn_rocm_mask_to_kv_len_flagged": [_vp, _vp, _vp, _i, _i, _f],
    "tnn_rocm_mask_prepare": [_vp, _i, _vp, _vp, _vp, _i, _i, _f],
    "tnn_rocm_mask_prepare_strided": [_vp, _i, _vp, _l, _vp, _vp, _i, _i, _f],
    "tnn_rocm_softmax": [_vp, _i, _vp, _vp, _i, _i, _i],
    "tnn_rocm_layernorm": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp, _f],
    "tnn_rocm_embed_layernorm": [_vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _i, _vp, _vp, _f, _vp, _i, _i, _vp],
    "tnn_rocm_embed_layernorm_pos": [_vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _vp, _vp, _f, _vp, _i, _i,
                                     _vp],
    "tnn_rocm_gelu": [_vp, _i, _vp, _vp, _sz],
    "tnn_rocm_tanh": [_vp, _i, _vp, _vp, _sz],
    "tnn_rocm_binary": [_vp, _i, _i, _vp, _ip, _i, _vp, _ip, _i, _vp, _ip, _i],
    "tnn_rocm_permute": [_vp, _i, _vp, _vp, _ip, _ip, _i],
    "tnn_rocm_gather": [_vp, _vp, _vp, _vp, _i, _i, _sz, _i, _vp],
    "tnn_rocm_cast": [_vp, _i, _vp, _i, _vp, _sz],
    "tnn_rocm_quantize": [_vp, _i, _vp, _f, _vp, _sz],
    "tnn_rocm_dequantize": [_vp, _vp, _f, _i, _vp, _sz],
    "tnn_rocm_quantize_per_channel": [_vp, _i, _vp, _vp, _vp, _sz, _i, _sz],
    "tnn_rocm_dequantize_per_channel": [_vp, _vp, _vp, _i, _vp, _sz, _i, _sz],
    "tnn_rocm_debug_set_gemm_config": [_i],
    "tnn_rocm_debug_set_gemm_tune": [C.c_char_p],
    "tnn_rocm_debug_set_gemm_group_m": [_i],
    "tnn_rocm_debug_set_ln_y_ahead": [_i],
    "tnn_rocm_debug_set_store_through": [_i],
    "tnn_rocm_debug_set_attention_dma": [_i],
    "tnn_rocm_add_i8": [_vp, _vp, _f, _vp, _f, _f, _vp, _sz, _i, _sz],
    "tnn_rocm_add_i8_per_channel": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _sz],
    "tnn_rocm_gelu_i8": [_vp, _vp, _f, _f, _vp, _sz],
}

_lib = None


class TnnRocmError(RuntimeError):
    def __init__(self, fn, code, msg):
        super().__init__("%s failed with code %d: %s" % (fn, code, msg))
        self.code = code


def load():
    """Load the shared library once and attach argument types; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            "%s not found: build it with `python -m tnn_amd.build` (no CPU fallback exists)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    lib.tnn_rocm_last_error.restype = C.c_char_p
    lib.tnn_rocm_last_error.argtypes = []
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.argtypes = args
        fn.restype = C.c_int
    _lib = lib
    return lib


def call(name, *args):
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise TnnRocmError(name, rc, lib.tnn_rocm_last_error().decode("utf-8", "replace"))
    return rc


def int_array(values):
    values = list(values)
    return (C.c_int * max(len(values), 1))(*values)
