"""ctypes binding of libgearhip.so (declared in include/gear_hip.h).

The library is the product's only compute path: if it is missing, loading raises; there is no
CPU or PyTorch fallback behind any of these calls.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libgearhip.so")

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_void_p = ctypes.c_void_p
c_size_t = ctypes.c_size_t
c_double = ctypes.c_double

MAX_COLUMNS = 16


class ColumnDesc(ctypes.Structure):
    """struct gear_hip_column_desc"""
    _fields_ = [("dst", c_void_p), ("mask_out", c_void_p), ("ofst", c_i64), ("span", c_i64),
                ("step_bytes", c_i64), ("col_base", c_i64), ("dst_stride", c_i64),
                ("pad_head", ctypes.c_int32), ("zero_fill", ctypes.c_int32)]


# name -> (restype, argtypes); one entry per function of include/gear_hip.h
SIGNATURES = {
    "gear_hip_abi_version": (c_int, []),
    "gear_hip_set_device": (c_int, [c_int]),
    "gear_hip_device_count": (c_int, [ctypes.POINTER(c_int)]),
    "gear_hip_error_string": (ctypes.c_char_p, [c_int]),
    "gear_hip_host_alloc": (c_int, [c_size_t, ctypes.POINTER(c_void_p), ctypes.POINTER(c_void_p)]),
    "gear_hip_host_free": (c_int, [c_void_p]),
    "gear_hip_device_alloc": (c_int, [c_size_t, ctypes.POINTER(c_void_p)]),
    "gear_hip_device_free": (c_int, [c_void_p]),
    "gear_hip_memcpy": (c_int, [c_void_p, c_void_p, c_size_t]),
    "gear_hip_host_register": (c_int, [c_void_p, c_size_t, ctypes.POINTER(c_void_p)]),
    "gear_hip_host_unregister": (c_int, [c_void_p]),
    "gear_hip_subcopy": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_int,
                                 c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_int, c_void_p,
                                 c_void_p]),
    "gear_hip_subcopy_multi": (c_int, [c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_i64,
                                       ctypes.POINTER(ColumnDesc), c_int, c_void_p]),
    "gear_hip_subcopy_multi_checked": (c_int, [c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_i64,
                                               c_i64, c_i64, ctypes.POINTER(ColumnDesc), c_int,
                                               c_void_p]),
    "gear_hip_vcopy": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_i64,
                               c_void_p]),
    "gear_hip_copy": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_i64, c_void_p]),
    "gear_hip_sub": (c_int, [c_i64, c_void_p, c_void_p, c_void_p, c_int, c_i64, c_i64, c_i64,
                             c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "gear_hip_split_step_index": (c_int, [c_void_p, c_i64, c_i64, c_i64, c_void_p, c_void_p,
                                          c_void_p, c_void_p]),
    "gear_hip_take_i64": (c_int, [c_void_p, c_i64, c_void_p, c_i64, c_i64, c_void_p, c_void_p]),
    "gear_hip_scan_workspace_bytes": (c_size_t, [c_i64]),
    "gear_hip_scan_f32_f64": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_size_t, c_void_p]),
    "gear_hip_scan_static_max_n": (c_i64, []),
    "gear_hip_scan_f32_f64_static": (c_int, [c_void_p, c_void_p, c_i64, c_void_p]),
    "gear_hip_rescan_f32_f64": (c_int, [c_void_p, c_void_p, c_i64, c_i64, c_void_p, c_size_t,
                                        c_void_p]),
    "gear_hip_scan_f32_f32": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_size_t, c_void_p]),
    "gear_hip_scan_i64": (c_int, [c_void_p, c_void_p, c_i64, c_void_p, c_size_t, c_void_p]),
    "gear_hip_sum_workspace_bytes": (c_size_t, [c_i64]),
    "gear_hip_sum_f32": (c_int, [c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_size_t,
                                 c_void_p]),
    "gear_hip_search_workspace_bytes": (c_size_t, [c_i64]),
    "gear_hip_upper_bound_f64": (c_int, [c_void_p, c_i64, c_void_p, c_i64, c_int, c_void_p,
                                         c_void_p, c_double, c_void_p, c_void_p, c_size_t,
                                         c_void_p]),
    "gear_hip_sample_workspace_bytes": (c_size_t, [c_i64]),
    "gear_hip_sample_sorted_f64": (c_int, [c_void_p, c_i64, c_void_p, c_i64, c_int, c_void_p, c_i64,
                                           c_i64, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                           c_void_p]),
    "gear_hip_sample_lookup_f64": (c_int, [c_void_p, c_i64, c_void_p, c_i64, c_int, c_void_p, c_i64,
                                           c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_size_t, c_void_p]),
    "gear_hip_sample_lookup_i64": (c_int, [c_void_p, c_i64, c_void_p, c_i64, c_int, c_void_p, c_i64,
                                           c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_i64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "gear_hip_sort_lookup_i64": (c_int, [c_void_p, c_i64, c_i64, c_void_p, c_i64, c_i64, c_void_p,
                                         c_i64, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                         c_void_p]),
    "gear_hip_lookup_i64": (c_int, [c_void_p, c_i64, c_void_p, c_i64, c_i64, c_void_p, c_i64,
                                    c_void_p, c_void_p, c_void_p, c_void_p]),
    "gear_hip_upper_bound_i64": (c_int, [c_void_p, c_i64, c_void_p, c_i64, c_int, c_void_p,
                                         c_void_p]),
    "gear_hip_sort_workspace_bytes": (c_size_t, [c_i64]),
    "gear_hip_sort_i64": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_int, c_void_p,
                                  c_size_t, c_void_p]),
    "gear_hip_topk_workspace_bytes": (c_size_t, [c_i64, c_i64]),
    "gear_hip_topk_f32": (c_int, [c_void_p, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p,
                                  c_size_t, c_void_p]),
    "gear_hip_topk_f32_warm": (c_int, [c_void_p, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p,
                                       c_size_t, c_void_p]),
    "gear_hip_scatter_workspace_bytes": (c_size_t, [c_i64]),
    "gear_hip_scatter_f32": (c_int, [c_void_p, c_i64, c_void_p, c_void_p, c_i64, c_int, c_void_p,
                                     c_size_t, c_void_p]),
    "gear_hip_scatter_i64": (c_int, [c_void_p, c_i64, c_void_p, c_void_p, c_i64, c_int, c_void_p,
                                     c_size_t, c_void_p]),
}

_lib = None


class GearHipError(RuntimeError):
    def __init__(self, fn, code, text):
        super().__init__("%s failed with code %d: %s" % (fn, code, text))
        self.code = code


def load():
    """dlopen libgearhip.so and attach the signatures; raises if the library is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "gear_amd: %s is missing; the HIP library is the only compute path. Build it with "
            "`python -c 'import __graft_entry__ as g; g.build()'`." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.gear_hip_abi_version() != 1:
        raise ImportError("gear_amd: libgearhip.so has an unexpected ABI version")
    _lib = lib
    return lib


def check(fn_name, code):
    if code != 0:
        text = load().gear_hip_error_string(code)
        raise GearHipError(fn_name, code, text.decode() if text else "?")


def call(fn_name, *args):
    """Call an int-returning entry point and raise GearHipError on a non-zero code."""
    code = getattr(load(), fn_name)(*args)
    check(fn_name, code)
