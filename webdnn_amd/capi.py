"""ctypes binding of libwebdnn_hip.so (the C ABI declared in include/webdnn_hip.h).

This is the Python counterpart of the N-API addon the Node.js host uses: a thin
1:1 mapping, no arithmetic.  The library is loaded from webdnn_amd/lib/ (built
in-tree by ``python -m webdnn_amd.build``); there is no CPU fallback — every
call fails loudly when the library or the GPU is missing.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# WEBDNN_HIP_LIB names another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("WEBDNN_HIP_LIB") or os.path.join(_HERE, "lib", "libwebdnn_hip.so")

# every symbol include/webdnn_hip.h declares, with its signature
c_buf = ctypes.c_int64
_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_u64p = ctypes.POINTER(ctypes.c_uint64)
_c = ctypes

SIGNATURES = {
    "wdh_init": (_c.c_int, [_c.c_int]),
    "wdh_shutdown": (None, []),
    "wdh_last_error": (_c.c_char_p, []),
    "wdh_device_info": (_c.c_int, [_c.c_char_p, _c.c_int, _c.POINTER(_c.c_int),
                                   _c.POINTER(_c.c_int), _u64p]),
    "wdh_set_option": (_c.c_int, [_c.c_char_p, _c.c_int]),
    "wdh_last_plan": (_c.c_int, [_c.POINTER(_c.c_int), _c.POINTER(_c.c_int), _i64p, _i64p,
                                 _c.POINTER(_c.c_int), _c.POINTER(_c.c_int)]),
    "wdh_alloc": (c_buf, [_c.c_size_t]),
    "wdh_free": (_c.c_int, [c_buf]),
    "wdh_write": (_c.c_int, [c_buf, _c.c_size_t, _c.c_void_p, _c.c_size_t]),
    "wdh_read": (_c.c_int, [c_buf, _c.c_size_t, _c.c_void_p, _c.c_size_t]),
    "wdh_copy": (_c.c_int, [c_buf, _c.c_size_t, c_buf, _c.c_size_t, _c.c_size_t]),
    "wdh_sync": (_c.c_int, []),
    "wdh_set_lane": (_c.c_int, [_c.c_int]),
    "wdh_branch_begin": (_c.c_int, []),
    "wdh_branch_end": (_c.c_int, []),
    "wdh_branch_join": (_c.c_int, []),
    "wdh_mem_stats": (_c.c_int, [_u64p, _u64p, _u64p]),
    "wdh_trim": (_c.c_int, [_c.c_size_t]),
    "wdh_graph_begin": (_c.c_int, []),
    "wdh_graph_end": (_c.c_int, [_c.POINTER(_c.c_int)]),
    "wdh_graph_launch": (_c.c_int, [_c.c_int]),
    "wdh_graph_destroy": (_c.c_int, [_c.c_int]),
    "wdh_event_record": (_c.c_int, [_c.c_int]),
    "wdh_event_elapsed_ms": (_c.c_int, [_c.c_int, _c.c_int, _c.POINTER(_c.c_float)]),
    "wdh_gemm": (_c.c_int, [c_buf, c_buf, c_buf, c_buf, _c.c_int, _c.c_int, _c.c_int, _c.c_int,
                            _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
                            _c.c_int64, _c.c_int64, _c.c_int64, _c.c_float, _c.c_float,
                            _c.c_int, c_buf]),
    "wdh_gemm_ex": (_c.c_int, [c_buf, c_buf, c_buf, c_buf, _c.c_int, _c.c_int, _c.c_int, _c.c_int,
                               _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
                               _c.c_int64, _c.c_int64, _c.c_int64, _c.c_float, _c.c_float,
                               _c.c_int, c_buf, _c.c_int64, _c.c_int64]),
    "wdh_gemm_static": (_c.c_int, [c_buf, c_buf, c_buf, c_buf, _c.c_int, _c.c_int, _c.c_int, _c.c_int,
                                   _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
                                   _c.c_int64, _c.c_int64, _c.c_int64, _c.c_float, _c.c_float,
                                   _c.c_int, c_buf]),
    "wdh_linear_group": (_c.c_int, [_c.c_int, _i64p, _i64p, _i64p, _i64p, _i32p, _i32p, _i32p, _c.c_int]),
    "wdh_conv2d": (_c.c_int, [c_buf, c_buf, c_buf, c_buf] + [_c.c_int] * 17 + [c_buf]),
    "wdh_conv2d_ex": (_c.c_int, [c_buf, c_buf, c_buf, c_buf] + [_c.c_int] * 17 + [c_buf, _c.c_int]),
    "wdh_binary": (_c.c_int, [_c.c_int, _c.c_int, c_buf, c_buf, c_buf, _c.c_int, _i32p, _i64p, _i64p]),
    "wdh_unary": (_c.c_int, [_c.c_int, _c.c_int, c_buf, c_buf, _c.c_size_t]),
    "wdh_softmax": (_c.c_int, [c_buf, c_buf, _c.c_int64, _c.c_int]),
    "wdh_attention": (_c.c_int, [c_buf, c_buf, c_buf, c_buf, _c.c_int, _c.c_int, _c.c_int, _c.c_int] +
                      [_c.c_int64] * 8 + [_c.c_float]),
    "wdh_layernorm": (_c.c_int, [c_buf, c_buf, c_buf, c_buf, _c.c_int64, _c.c_int, _c.c_float]),
    "wdh_layernorm_add": (_c.c_int, [c_buf, c_buf, c_buf, c_buf, c_buf, c_buf, _c.c_int64, _c.c_int, _c.c_float]),
    "wdh_reduce_mean": (_c.c_int, [c_buf, c_buf, _c.c_int64, _c.c_int]),
    "wdh_reduce_axis": (_c.c_int, [c_buf, c_buf, _c.c_int64, _c.c_int, _c.c_int64, _c.c_int64]),
    "wdh_maxpool2d": (_c.c_int, [c_buf, c_buf] + [_c.c_int] * 14),
    "wdh_global_avgpool": (_c.c_int, [c_buf, c_buf, _c.c_int64, _c.c_int]),
    "wdh_transpose": (_c.c_int, [c_buf, c_buf, _c.c_int, _i32p, _i64p]),
    "wdh_gather": (_c.c_int, [c_buf, c_buf, c_buf, _c.c_int64, _c.c_int, _c.c_int64, _c.c_int64]),
    "wdh_cast": (_c.c_int, [_c.c_int, _c.c_int, c_buf, c_buf, _c.c_size_t]),
    "wdh_strided_copy": (_c.c_int, [c_buf, _c.c_int64, c_buf, _c.c_int64, _c.c_int, _i32p, _i64p, _i64p]),
}


class HipError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, func, code, message):
        super().__init__("%s failed (%d): %s" % (func, code, message))
        self.func = func
        self.code = code


_lib = None


def load():
    """Loads the shared library and attaches signatures.  Does not touch the GPU."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipError("load", -5, "%s is missing: run `python -m webdnn_amd.build`" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error():
    return load().wdh_last_error().decode("utf-8", "replace")


def call(name, *args):
    """Calls an int-returning entry point; raises HipError on a negative status."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc < 0:
        raise HipError(name, rc, last_error())
    return rc
