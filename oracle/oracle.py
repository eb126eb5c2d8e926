"""numpy-facing wrapper of liboracle.so (oracle/gear_oracle.c).  TEST INFRASTRUCTURE ONLY.

Every function takes and returns numpy arrays; see gear_oracle.c for the reference citations.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_i64p = ctypes.POINTER(ctypes.c_int64)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)


def build():
    """Compile oracle/gear_oracle.c into oracle/liboracle.so (gcc)."""
    subprocess.run(["make", "-s", "-B", "-C", _HERE, "liboracle.so"], check=True)


REFERENCE_ROOT = "/root/reference"
_REF = None


def build_ref():
    """Compile the reference's own table-spec sources (src/storage/specs.cc with its headers)
    behind oracle/ref_specs_glue.cc into oracle/_ref/libref_specs.so.  Needs the reference tree;
    returns False where it is absent (then a library built earlier is used if it is there)."""
    if not os.path.isdir(REFERENCE_ROOT):
        return False
    subprocess.run(["make", "-s", "-B", "-C", _HERE, "ref"], check=True)
    return True


def ref_specs():
    """ctypes handle of oracle/_ref/libref_specs.so, or None where it was never built."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, "_ref", "libref_specs.so")
        if not os.path.exists(path):
            return None
        _REF = ctypes.CDLL(path)
        for name in ("ref_sizeof_dtype", "ref_column_size", "ref_table_nbytes", "ref_table_index"):
            getattr(_REF, name).restype = ctypes.c_int64
    return _REF


def _ref_columns(columns):
    """columns: [(shape tuple, dtype code)] -> (flat shapes, ndims, dtypes) as ctypes arrays."""
    flat = [int(d) for shape, _ in columns for d in shape]
    shapes = (ctypes.c_int64 * max(1, len(flat)))(*flat)
    ndims = (ctypes.c_int * len(columns))(*[len(shape) for shape, _ in columns])
    dtypes = (ctypes.c_int * len(columns))(*[int(dt) for _, dt in columns])
    return shapes, ndims, dtypes


def ref_sizeof_dtype(code):
    return ref_specs().ref_sizeof_dtype(ctypes.c_int(int(code)))


def ref_column_size(shape, code):
    arr = (ctypes.c_int64 * max(1, len(shape)))(*[int(d) for d in shape])
    return ref_specs().ref_column_size(arr, ctypes.c_int(len(shape)), ctypes.c_int(int(code)))


def ref_table_nbytes(trajectory_length, capacity, columns):
    shapes, ndims, dtypes = _ref_columns(columns)
    return ref_specs().ref_table_nbytes(ctypes.c_int64(trajectory_length), ctypes.c_int64(capacity),
                                        ctypes.c_int(len(columns)), shapes, ndims, dtypes)


def ref_table_index(columns, name):
    shapes, ndims, dtypes = _ref_columns(columns)
    return ref_specs().ref_table_index(ctypes.c_int(len(columns)), shapes, ndims, dtypes,
                                       name.encode())


def lib():
    global _LIB
    if _LIB is None:
        path = os.environ.get("GEAR_ORACLE_LIB")  # another build of it (the sanitizer run)
        if not path:
            path = os.path.join(_HERE, "liboracle.so")
            if not os.path.exists(path):
                build()
        _LIB = ctypes.CDLL(path)
        _LIB.oracle_sub.restype = ctypes.c_int64
        _LIB.oracle_sum_f32.restype = ctypes.c_double
    return _LIB


def _p(a, t):
    return a.ctypes.data_as(t)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def layout(step_bytes, T, capacity):
    sb = _c(step_bytes, np.int64)
    accu = np.zeros(len(sb) + 1, np.int64)
    stride = ctypes.c_int64()
    total = ctypes.c_int64()
    lib().oracle_layout(ctypes.c_int64(len(sb)), _p(sb, _i64p), ctypes.c_int64(T),
                        ctypes.c_int64(capacity), _p(accu, _i64p), ctypes.byref(stride),
                        ctypes.byref(total))
    return accu, stride.value, total.value


def sub(idxs, tss, lens, pad_head, ofst, span, traj_stride, step_bytes, col_base):
    idxs, tss, lens = _c(idxs, np.int64), _c(tss, np.int64), _c(lens, np.int64)
    n = len(idxs)
    so, do, cl = (np.zeros(n, np.int64) for _ in range(3))
    exp = lib().oracle_sub(ctypes.c_int64(n), _p(idxs, _i64p), _p(tss, _i64p), _p(lens, _i64p),
                           ctypes.c_int(int(pad_head)), ctypes.c_int64(ofst),
                           ctypes.c_int64(span), ctypes.c_int64(traj_stride),
                           ctypes.c_int64(step_bytes), ctypes.c_int64(col_base),
                           _p(so, _i64p), _p(do, _i64p), _p(cl, _i64p))
    return so, do, cl, exp


def subcopy(table, idxs, tss, lens, pad_head, ofst, span, traj_stride, step_bytes, col_base,
            dst_stride=None, zero_fill=True, want_mask=False, dst=None, threads=1):
    """Returns (dst uint8[num, dst_stride], mask uint8[num, span] or None).  threads > 1 splits
    the windows over that many host threads (same result)."""
    table = _c(table, np.uint8)
    idxs, tss, lens = _c(idxs, np.int64), _c(tss, np.int64), _c(lens, np.int64)
    n = len(idxs)
    if dst_stride is None:
        dst_stride = span * step_bytes
    if dst is None:
        dst = np.zeros((n, dst_stride), np.uint8)
    mask = np.zeros((n, span), np.uint8) if want_mask else None
    args = [_p(table, _u8p), _p(dst, _u8p), ctypes.c_int64(n), _p(idxs, _i64p),
            _p(tss, _i64p), _p(lens, _i64p), ctypes.c_int(int(pad_head)),
            ctypes.c_int64(ofst), ctypes.c_int64(span),
            ctypes.c_int64(traj_stride), ctypes.c_int64(step_bytes),
            ctypes.c_int64(col_base), ctypes.c_int64(dst_stride),
            ctypes.c_int(int(zero_fill)),
            _p(mask, _u8p) if want_mask else None]
    if threads > 1:
        lib().oracle_subcopy_mt(*args, ctypes.c_int(int(threads)))
    else:
        lib().oracle_subcopy(*args)
    return dst, mask


def vcopy(src, dst, src_offsets, dst_offsets, strides):
    src = _c(src, np.uint8)
    so, do, st = _c(src_offsets, np.int64), _c(dst_offsets, np.int64), _c(strides, np.int64)
    lib().oracle_vcopy(_p(src, _u8p), _p(dst, _u8p), ctypes.c_int64(len(so)), _p(so, _i64p),
                       _p(do, _i64p), _p(st, _i64p))
    return dst


def copy(src, dst, src_offsets, dst_offsets, stride):
    src = _c(src, np.uint8)
    so, do = _c(src_offsets, np.int64), _c(dst_offsets, np.int64)
    lib().oracle_copy(_p(src, _u8p), _p(dst, _u8p), ctypes.c_int64(len(so)), _p(so, _i64p),
                      _p(do, _i64p), ctypes.c_int64(stride))
    return dst


def scan_f32_f64(p, threads=1):
    """threads > 1: two-level chunked scan over that many host threads (all-cores baseline);
    equal to the sequential result up to rounding, exactly on integer-valued input."""
    p = _c(p, np.float32)
    out = np.zeros(len(p), np.float64)
    if threads > 1:
        lib().oracle_scan_f32_f64_mt(_p(p, _f32p), _p(out, _f64p), ctypes.c_int64(len(p)),
                                     ctypes.c_int(int(threads)))
    else:
        lib().oracle_scan_f32_f64(_p(p, _f32p), _p(out, _f64p), ctypes.c_int64(len(p)))
    return out


def scan_i64(p):
    p = _c(p, np.int64)
    out = np.zeros(len(p), np.int64)
    lib().oracle_scan_i64(_p(p, _i64p), _p(out, _i64p), ctypes.c_int64(len(p)))
    return out


def sum_f32(p):
    p = _c(p, np.float32)
    return lib().oracle_sum_f32(_p(p, _f32p), ctypes.c_int64(len(p)))


def upper_bound_f64(prefix, u, unit_uniforms=False, threads=1):
    prefix, u = _c(prefix, np.float64), _c(u, np.float32)
    out = np.zeros(len(u), np.int64)
    args = [_p(prefix, _f64p), ctypes.c_int64(len(prefix)), _p(u, _f32p),
            ctypes.c_int64(len(u)), ctypes.c_int(int(unit_uniforms)), _p(out, _i64p)]
    if threads > 1:
        lib().oracle_upper_bound_f64_mt(*args, ctypes.c_int(int(threads)))
    else:
        lib().oracle_upper_bound_f64(*args)
    return out


def upper_bound_i64(prefix, u, unit_uniforms=False):
    prefix = _c(prefix, np.int64)
    u = _c(u, np.float64 if unit_uniforms else np.int64)
    out = np.zeros(len(u), np.int64)
    lib().oracle_upper_bound_i64(_p(prefix, _i64p), ctypes.c_int64(len(prefix)),
                                 ctypes.c_void_p(u.ctypes.data), ctypes.c_int64(len(u)),
                                 ctypes.c_int(int(unit_uniforms)), _p(out, _i64p))
    return out


def is_weights(priorities, total, idx, beta):
    priorities, idx = _c(priorities, np.float32), _c(idx, np.int64)
    out = np.zeros(len(idx), np.float32)
    lib().oracle_is_weights(_p(priorities, _f32p), ctypes.c_int64(len(priorities)),
                            ctypes.c_double(total), _p(idx, _i64p), ctypes.c_int64(len(idx)),
                            ctypes.c_double(beta), _p(out, _f32p))
    return out


def topk_f32(w, k, sorted_by_value=True, threads=1):
    """threads > 1: per-chunk selection over that many host threads, then a merge (all-cores
    baseline); identical result."""
    w = _c(w, np.float32)
    vals = np.zeros(k, np.float32)
    idx = np.zeros(k, np.int64)
    args = [_p(w, _f32p), ctypes.c_int64(len(w)), ctypes.c_int64(k),
            ctypes.c_int(int(sorted_by_value)), _p(vals, _f32p), _p(idx, _i64p)]
    if threads > 1:
        lib().oracle_topk_f32_mt(*args, ctypes.c_int(int(threads)))
    else:
        lib().oracle_topk_f32(*args)
    return vals, idx


def sort_i64(keys, vals=None):
    keys = _c(keys, np.int64)
    ko = np.zeros(len(keys), np.int64)
    if vals is not None:
        vals = _c(vals, np.int64)
        vo = np.zeros(len(keys), np.int64)
    lib().oracle_sort_i64(_p(keys, _i64p), _p(ko, _i64p),
                          _p(vals, _i64p) if vals is not None else None,
                          _p(vo, _i64p) if vals is not None else None,
                          ctypes.c_int64(len(keys)))
    return (ko, vo) if vals is not None else ko


def scatter_f32(weights, idx, values):
    """In place on `weights` (float32 array); returns it."""
    assert weights.dtype == np.float32 and weights.flags.c_contiguous
    idx, values = _c(idx, np.int64), _c(values, np.float32)
    lib().oracle_scatter_f32(_p(weights, _f32p), ctypes.c_int64(len(weights)), _p(idx, _i64p),
                             _p(values, _f32p), ctypes.c_int64(len(idx)))
    return weights
