"""ctypes binding of libhchip.so (the C ABI declared in include/hchip.h).

There is no fallback: if the library has not been built, importing this module raises.
"""
import ctypes
import os
from ctypes import (POINTER, Structure, c_char, c_char_p, c_float, c_int, c_int64, c_size_t,
                    c_uint32, c_uint64, c_void_p)

HERE = os.path.dirname(os.path.abspath(__file__))
# HCHIP_LIB points at an alternative build of the library (kernel experiments).
LIB_PATH = os.environ.get("HCHIP_LIB", os.path.join(HERE, "csrc", "libhchip.so"))

HC_MAX_DIMS = 8

HC_OK = 0
HC_ERR_INVALID = 1
HC_ERR_ALLOC = 2
HC_ERR_LOAD = 3
HC_ERR_UNSUPPORTED = 4
HC_ERR_TOO_LARGE = 5
HC_ERR_NO_DEVICE = 6
HC_ERR_HIP_BASE = 1000


class hc_strides(Structure):
    _fields_ = [
        ("ndim", c_uint32),
        ("reserved", c_uint32),
        ("shape", c_int64 * HC_MAX_DIMS),
        ("strides", c_int64 * HC_MAX_DIMS),
    ]


class hc_device_info(Structure):
    _fields_ = [
        ("name", c_char * 256),
        ("arch", c_char * 64),
        ("compute_units", c_int),
        ("clock_mhz", c_int),
        ("wavefront_size", c_int),
        ("lds_bytes_per_block", c_int),
        ("total_mem", c_size_t),
    ]


HOST_FN = ctypes.CFUNCTYPE(None, c_void_p)

_S = POINTER(hc_strides)
_P = c_void_p

# name -> (restype, argtypes); every symbol include/hchip.h declares.
PROTOTYPES = {
    "hc_init": (c_int, [c_int, POINTER(c_void_p)]),
    "hc_shutdown": (None, [_P]),
    "hc_last_error_string": (c_char_p, []),
    "hc_get_device_info": (c_int, [_P, POINTER(hc_device_info)]),
    "hc_debug_set": (c_int, [_P, c_char_p, c_char_p]),
    "hc_set_batching": (c_int, [_P, c_size_t, c_size_t]),
    "hc_flush": (c_int, [_P]),
    "hc_batching_stats": (c_int, [_P, POINTER(c_uint64), POINTER(c_uint64)]),
    "hc_malloc": (c_int, [_P, c_size_t, POINTER(c_void_p)]),
    "hc_free": (c_int, [_P, _P]),
    "hc_trim": (c_int, [_P]),
    "hc_mem_stats": (c_int, [_P, POINTER(c_size_t), POINTER(c_size_t)]),
    "hc_host_alloc": (c_int, [_P, c_size_t, POINTER(c_void_p)]),
    "hc_host_free": (c_int, [_P, _P]),
    "hc_memcpy_h2d": (c_int, [_P, _P, _P, c_size_t]),
    "hc_memcpy_d2h": (c_int, [_P, _P, _P, c_size_t]),
    "hc_memcpy_d2d": (c_int, [_P, _P, _P, c_size_t]),
    "hc_memcpy_h2d_async": (c_int, [_P, _P, _P, c_size_t]),
    "hc_memcpy_d2h_async": (c_int, [_P, _P, _P, c_size_t]),
    "hc_sync": (c_int, [_P]),
    "hc_event_create": (c_int, [_P, POINTER(c_void_p)]),
    "hc_event_record": (c_int, [_P, _P]),
    "hc_event_sync": (c_int, [_P]),
    "hc_event_query": (c_int, [_P]),
    "hc_event_elapsed_ms": (c_int, [_P, _P, POINTER(c_float)]),
    "hc_event_destroy": (c_int, [_P]),
    "hc_launch_host_func": (c_int, [_P, HOST_FN, _P]),
    "hc_capture_begin": (c_int, [_P]),
    "hc_capture_end": (c_int, [_P, POINTER(c_void_p)]),
    "hc_capture_abort": (c_int, [_P]),
    "hc_graph_launch": (c_int, [_P, _P]),
    "hc_graph_node_count": (c_int, [_P, POINTER(c_size_t)]),
    "hc_graph_destroy": (c_int, [_P, _P]),
    "hc_module_load": (c_int, [_P, _P, c_size_t, POINTER(c_void_p)]),
    "hc_module_unload": (c_int, [_P, _P]),
    "hc_module_get_function": (c_int, [_P, c_char_p, POINTER(c_void_p)]),
    "hc_launch": (c_int, [_P, _P, POINTER(c_uint32), POINTER(c_uint32), c_uint32, _P, c_size_t]),
    "hc_broadcast": (c_int, [_P, c_int, _P, _S, _P]),
    "hc_binary_op": (c_int, [_P, c_int, c_int, _P, _S, _P, _S, _P]),
    "hc_binary_op_scalar": (c_int, [_P, c_int, c_int, _P, c_float, c_int64, c_int, _P, c_size_t]),
    "hc_mul_add": (c_int, [_P, c_int, _P, _S, _P, _S, _P, _S, _P]),
    "hc_add_mul": (c_int, [_P, c_int, _P, _S, _P, _S, _P, _S, _P]),
    "hc_compare": (c_int, [_P, c_int, c_int, _P, _S, _P, _S, _P]),
    "hc_compare_scalar": (c_int, [_P, c_int, c_int, _P, c_float, c_int64, c_int, _P, c_size_t]),
    "hc_cast": (c_int, [_P, _P, c_int, _P, c_int, c_size_t]),
    "hc_pow": (c_int, [_P, c_int, _P, c_float, c_float, c_int64, c_int64, _P, _P, c_size_t]),
    "hc_elemwise": (c_int, [_P, c_int, c_int, _P, _P, _P, c_size_t]),
    "hc_reduce": (c_int, [_P, c_int, c_int, _P, _P, c_int64, c_int64, c_int64]),
    "hc_reduce_noalloc": (c_int, [_P, c_int, c_int, _P, _P, c_int64, c_int64, c_int64]),
    "hc_cumulative": (c_int, [_P, c_int, c_int, _P, _P, c_int64, c_int64, c_int64, c_int, c_int]),
    "hc_argsort": (c_int, [_P, c_int, _P, _P, c_int64, c_int64, c_int64, c_int]),
    "hc_log_softmax": (c_int, [_P, c_int, _P, _P, c_int64, c_int64, c_int64]),
    "hc_normalize": (c_int, [_P, c_int, _P, _P, c_int64, c_int64, c_int64, c_float]),
    "hc_gather": (c_int, [_P, c_int, _P, _P, _S, _P, c_int64, c_int64, c_int64, c_int64]),
    "hc_bitwise_op": (c_int, [_P, c_int, c_int, _P, _S, _P, _S, _P]),
    "hc_scatter": (c_int, [_P, c_int, _P, _P, _S, _P, c_int64, c_int64, c_int64, c_int64, c_int]),
    "hc_log_softmax_grad": (c_int, [_P, c_int, _P, _P, _P, c_int64, c_int64, c_int64]),
    "hc_clamp": (c_int, [_P, c_int, _P, _S, _P, _S, _P, _S, _P]),
    "hc_adamw": (c_int, [_P, c_int, _P, _P, _P, _P, c_float, c_float, c_float, c_float, c_float, c_float,
                         c_size_t, _P, _P, _P]),
    "hc_when": (c_int, [_P, c_int, _P, _S, _P, _S, _P, _S, _P]),
    "hc_matmul": (c_int, [_P, c_int, c_int64, _P, c_int, _P, c_int, c_int, c_int64, c_int64, c_int64, _P]),
    "hc_triangular": (c_int, [_P, c_int, _P, _P, c_int64, c_int64, c_int64, c_int, c_int64]),
    "hc_fill": (c_int, [_P, c_int, c_float, c_int64, _P, c_size_t]),
    "hc_axis_permutation": (c_int, [_P, POINTER(c_int64), POINTER(c_int64), c_int, _P]),
    "hc_permute": (c_int, [_P, c_int, _P, POINTER(c_int64), POINTER(c_int64), c_int, c_int64, _P]),
    "hc_concat": (c_int, [_P, c_int, POINTER(c_void_p), POINTER(c_int64), c_int, c_int64, _P]),
}


def load(path: str = LIB_PATH) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise ImportError(
            "%s is missing: build it with `python -m honeycrisp_amd.csrc.build` "
            "(there is no CPU fallback)" % path)
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def make_strides(shape, strides) -> hc_strides:
    if len(shape) > HC_MAX_DIMS:
        raise ValueError("at most %d axes are supported, got shape %s" % (HC_MAX_DIMS, list(shape)))
    s = hc_strides()
    s.ndim = len(shape)
    for i, (n, st) in enumerate(zip(shape, strides)):
        s.shape[i] = n
        s.strides[i] = st
    return s
