"""Tensor-level entry points over the C ABI (include/gear_hip.h).

torch tensors are used for what they are here: handles to device memory plus the current HIP
stream.  All arithmetic happens in libgearhip.so; nothing in this module computes on tensors and
nothing falls back to torch or to the CPU.
"""
import ctypes
import functools

import torch

from . import _cabi
from ._cabi import ColumnDesc, call, load


# torch's C accessor for the raw current stream (a fraction of the cost of
# torch.cuda.current_stream(), which builds a Stream object through several Python layers)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_cur_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream_value(device=None):
    if _raw_stream is not None and _cur_device is not None:
        index = device.index if (device is not None and device.index is not None) \
            else _cur_device()
        return _raw_stream(index)
    return torch.cuda.current_stream(device).cuda_stream


def _stream():
    # (plain integers: ctypes converts them for the void* parameters itself, and building a
    # c_void_p object per argument is a measurable part of a small step)
    return _stream_value()


def _ptr(t):
    if t is None:
        return None
    return t.data_ptr()


def _need(t, dtype, name, device=True):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor" % name)
    if t.dtype != dtype:
        raise TypeError("%s must have dtype %s, got %s" % (name, dtype, t.dtype))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if device and not t.is_cuda:
        raise ValueError("%s must live on the GPU" % name)
    return t


def _src_ptr(src):
    """Table base: an int address (MemoryPtr-style), or a tensor (device, or pinned host)."""
    if isinstance(src, int):
        return src
    if isinstance(src, torch.Tensor):
        return src.data_ptr()
    if hasattr(src, "address"):
        return int(src.address)
    raise TypeError("unsupported table source %r" % type(src))


@functools.lru_cache(maxsize=512)
def _ws_bytes(query, *sizes):
    """Result of a *_workspace_bytes query of the library (a pure function of the sizes)."""
    return getattr(load(), query)(*[int(v) for v in sizes])


class _Workspace:
    """Scratch tensors per (purpose, device, stream), grown on demand and reused: no allocation
    in steady state, and calls enqueued on different streams never share a workspace."""

    def __init__(self):
        self._bufs = {}

    def get(self, tag, nbytes, device):
        key = (tag, device, _stream_value(device))
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
            self._bufs[key] = buf
        return buf


_ws = _Workspace()


def set_device(device_id):
    call("gear_hip_set_device", int(device_id))


def subcopy(src, dst, idxs, tss, lens, *, pad_head, ofst, span, traj_stride, step_bytes,
            col_base, zero_fill=True, mask_out=None, dst_stride=None):
    """One column of windows -> dst[num, span, ...]; see gear_hip_subcopy."""
    _need(idxs, torch.int64, "idxs")
    _need(tss, torch.int64, "tss")
    _need(lens, torch.int64, "lens")
    num = idxs.numel()
    if tss.numel() != num or lens.numel() != num:
        raise ValueError("idxs, tss and lens must have the same number of elements")
    if not dst.is_cuda or not dst.is_contiguous():
        raise ValueError("dst must be a contiguous GPU tensor")
    if dst_stride is None:
        dst_stride = span * step_bytes
    if dst.numel() * dst.element_size() < num * dst_stride:
        raise ValueError("dst is smaller than num * dst_stride bytes")
    if mask_out is not None:
        _need(mask_out, torch.uint8, "mask_out")
        if mask_out.numel() < num * span:
            raise ValueError("mask_out is smaller than num * span")
    call("gear_hip_subcopy", _src_ptr(src), _ptr(dst), num, _ptr(idxs), _ptr(tss), _ptr(lens),
         int(bool(pad_head)), int(ofst), int(span), int(traj_stride), int(step_bytes),
         int(col_base), int(dst_stride), int(bool(zero_fill)), _ptr(mask_out), _stream())
    return dst


def subcopy_multi(src, idxs, tss, lens, traj_stride, columns, capacity=0, trajectory_length=0):
    """All columns of one batch in one launch.

    columns: list of dicts with keys dst, ofst, span, step_bytes, col_base, pad_head and
    optionally zero_fill (default True), mask_out, dst_stride.
    capacity / trajectory_length > 0: the kernel checks every window against the table (an index
    outside [0, capacity) gathers nothing, lens are clamped to trajectory_length).
    """
    _need(idxs, torch.int64, "idxs")
    _need(tss, torch.int64, "tss")
    _need(lens, torch.int64, "lens")
    num = idxs.numel()
    n = len(columns)
    if n > _cabi.MAX_COLUMNS:
        raise ValueError("at most %d columns per launch" % _cabi.MAX_COLUMNS)
    descs = (ColumnDesc * max(n, 1))()
    for i, c in enumerate(columns):
        dst = c["dst"]
        stride = c.get("dst_stride", c["span"] * c["step_bytes"])
        if not dst.is_cuda or not dst.is_contiguous():
            raise ValueError("column %d: dst must be a contiguous GPU tensor" % i)
        if dst.numel() * dst.element_size() < num * stride:
            raise ValueError("column %d: dst is smaller than num * dst_stride bytes" % i)
        m = c.get("mask_out")
        if m is not None and m.numel() < num * c["span"]:
            raise ValueError("column %d: mask_out is smaller than num * span" % i)
        descs[i].dst = dst.data_ptr()
        descs[i].mask_out = m.data_ptr() if m is not None else None
        descs[i].ofst = int(c["ofst"])
        descs[i].span = int(c["span"])
        descs[i].step_bytes = int(c["step_bytes"])
        descs[i].col_base = int(c["col_base"])
        descs[i].dst_stride = int(stride)
        descs[i].pad_head = int(bool(c["pad_head"]))
        descs[i].zero_fill = int(bool(c.get("zero_fill", True)))
    call("gear_hip_subcopy_multi_checked", _src_ptr(src), num, _ptr(idxs), _ptr(tss), _ptr(lens),
         int(traj_stride), int(capacity), int(trajectory_length), descs, n, _stream())


class GatherPlan:
    """subcopy_multi for a loop that gathers into the same batch tensors every step: the column
    descriptors and every argument that does not change are marshalled once, run() is one call
    into the library with the three index tensors of the step."""

    def __init__(self, src, traj_stride, columns, num, capacity=0, trajectory_length=0):
        n = len(columns)
        if n > _cabi.MAX_COLUMNS:
            raise ValueError("at most %d columns per launch" % _cabi.MAX_COLUMNS)
        self._descs = (ColumnDesc * max(n, 1))()
        self._keep = []
        for i, c in enumerate(columns):
            dst = c["dst"]
            stride = c.get("dst_stride", c["span"] * c["step_bytes"])
            if not dst.is_cuda or not dst.is_contiguous():
                raise ValueError("column %d: dst must be a contiguous GPU tensor" % i)
            if dst.numel() * dst.element_size() < num * stride:
                raise ValueError("column %d: dst is smaller than num * dst_stride bytes" % i)
            m = c.get("mask_out")
            if m is not None and m.numel() < num * c["span"]:
                raise ValueError("column %d: mask_out is smaller than num * span" % i)
            d = self._descs[i]
            d.dst = dst.data_ptr()
            d.mask_out = m.data_ptr() if m is not None else None
            d.ofst, d.span = int(c["ofst"]), int(c["span"])
            d.step_bytes, d.col_base, d.dst_stride = int(c["step_bytes"]), int(c["col_base"]), int(stride)
            d.pad_head = int(bool(c["pad_head"]))
            d.zero_fill = int(bool(c.get("zero_fill", True)))
            self._keep.append((dst, m))
        self._keep.append(src)
        self._fn = load().gear_hip_subcopy_multi_checked
        self._num = int(num)
        self._head = (_src_ptr(src), self._num)
        self._tail = (int(traj_stride), int(capacity), int(trajectory_length), self._descs, n)

    def run(self, idxs, tss, lens):
        if idxs.numel() != self._num or tss.numel() != self._num or lens.numel() != self._num:
            raise ValueError("the plan was made for %d windows" % self._num)
        if idxs.dtype != torch.int64 or tss.dtype != torch.int64 or lens.dtype != torch.int64:
            raise TypeError("idxs, tss and lens must be int64 tensors")
        code = self._fn(*self._head, idxs.data_ptr(), tss.data_ptr(), lens.data_ptr(), *self._tail,
                        _stream_value(idxs.device))
        if code != 0:
            _cabi.check("gear_hip_subcopy_multi_checked", code)


def vcopy(src, dst, src_offsets, dst_offsets, strides, max_stride):
    _need(src_offsets, torch.int64, "src_offsets")
    _need(dst_offsets, torch.int64, "dst_offsets")
    _need(strides, torch.int64, "strides")
    num = min(src_offsets.numel(), dst_offsets.numel(), strides.numel())
    call("gear_hip_vcopy", _src_ptr(src), _ptr(dst), num, _ptr(src_offsets), _ptr(dst_offsets),
         _ptr(strides), int(max_stride), _stream())
    return dst


def copy(src, dst, src_offsets, dst_offsets, stride):
    _need(src_offsets, torch.int64, "src_offsets")
    _need(dst_offsets, torch.int64, "dst_offsets")
    num = min(src_offsets.numel(), dst_offsets.numel())
    call("gear_hip_copy", _src_ptr(src), _ptr(dst), num, _ptr(src_offsets), _ptr(dst_offsets),
         int(stride), _stream())
    return dst


def sub(idxs, tss, lens, *, pad_head, ofst, span, traj_stride, step_bytes, col_base,
        src_offsets=None, dst_offsets=None, copy_lens=None):
    _need(idxs, torch.int64, "idxs")
    _need(tss, torch.int64, "tss")
    _need(lens, torch.int64, "lens")
    num = idxs.numel()
    outs = []
    for t in (src_offsets, dst_offsets, copy_lens):
        outs.append(t if t is not None else torch.empty(num, dtype=torch.int64,
                                                        device=idxs.device))
    call("gear_hip_sub", num, _ptr(idxs), _ptr(tss), _ptr(lens), int(bool(pad_head)), int(ofst),
         int(span), int(traj_stride), int(step_bytes), int(col_base), _ptr(outs[0]),
         _ptr(outs[1]), _ptr(outs[2]), _stream())
    return outs[0], outs[1], outs[2], span * step_bytes


def split_step_index(flat, trajectory_length, modulo=0, idxs=None, tss=None, lens=None):
    """flat step indices -> (trajectory, timestep, length = timestep + 1) on the device."""
    _need(flat, torch.int64, "flat")
    num = flat.numel()
    outs = [t if t is not None else torch.empty(num, dtype=torch.int64, device=flat.device)
            for t in (idxs, tss, lens)]
    call("gear_hip_split_step_index", _ptr(flat), num, int(trajectory_length), int(modulo),
         _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), _stream())
    return outs[0], outs[1], outs[2]


def take_i64(table, idx, add=0, out=None):
    """out[j] = table[idx[j]] + add (int64, device)."""
    _need(table, torch.int64, "table")
    _need(idx, torch.int64, "idx")
    if out is None:
        out = torch.empty(idx.numel(), dtype=torch.int64, device=idx.device)
    call("gear_hip_take_i64", _ptr(table), table.numel(), _ptr(idx), idx.numel(), int(add),
         _ptr(out), _stream())
    return out


def prefix_sum(priorities, out=None):
    """fp32[n] -> inclusive fp64 prefix[n] (gear_hip_scan_f32_f64)."""
    _need(priorities, torch.float32, "priorities")
    n = priorities.numel()
    if out is None:
        out = torch.empty(n, dtype=torch.float64, device=priorities.device)
    else:
        _need(out, torch.float64, "out")
        if out.numel() < n:
            raise ValueError("out is too small")
    nbytes = _ws_bytes("gear_hip_scan_workspace_bytes", n)
    ws = _ws.get("scan", nbytes, priorities.device)
    call("gear_hip_scan_f32_f64", _ptr(priorities), _ptr(out), n, _ptr(ws), ws.numel(), _stream())
    return out


def prefix_sum_static(priorities, out):
    """fp32[n] -> fp64 prefix[n] into the caller's `out` with no allocation anywhere: the range
    sums live in the library's static device array (gear_hip_scan_f32_f64_static).  Calls that
    overlap on one GPU share that array and race."""
    _need(priorities, torch.float32, "priorities")
    _need(out, torch.float64, "out")
    n = priorities.numel()
    if out.numel() < n:
        raise ValueError("out is too small")
    call("gear_hip_scan_f32_f64_static", _ptr(priorities), _ptr(out), n, _stream())
    return out


class PrefixState:
    """The fp64 prefix of ONE priority array together with a workspace of its own, so that the
    range sums of the last scan survive other scans and a rescan can start at the first changed
    priority (gear_hip_rescan_f32_f64).  All calls must be enqueued on the same stream."""

    def __init__(self):
        self.out = None
        self._ws = None
        self._n = -1
        self._src = None
        self._valid = False

    def scan(self, priorities, first_changed=0):
        """first_changed = 0: full scan; k > 0: only priorities[k:] changed since the last call;
        k >= n: nothing changed (no launch).  Returns the fp64 prefix (the same tensor each call)."""
        _need(priorities, torch.float32, "priorities")
        n = priorities.numel()
        if self.out is None or self._n != n or self.out.device != priorities.device:
            self.out = torch.empty(n, dtype=torch.float64, device=priorities.device)
            nbytes = _ws_bytes("gear_hip_scan_workspace_bytes", n)
            self._ws = torch.empty(max(int(nbytes), 256), dtype=torch.uint8,
                                   device=priorities.device)
            self._n = n
            self._valid = False
        if self._src != priorities.data_ptr():
            self._valid = False
        if not self._valid or first_changed <= 0:
            call("gear_hip_scan_f32_f64", _ptr(priorities), _ptr(self.out), n, _ptr(self._ws),
                 self._ws.numel(), _stream())
        else:
            call("gear_hip_rescan_f32_f64", _ptr(priorities), _ptr(self.out), n,
                 int(first_changed), _ptr(self._ws), self._ws.numel(), _stream())
        self._src = priorities.data_ptr()
        self._valid = True
        return self.out


def prefix_sum_i64(weights, out=None):
    _need(weights, torch.int64, "weights")
    n = weights.numel()
    if out is None:
        out = torch.empty(n, dtype=torch.int64, device=weights.device)
    else:
        _need(out, torch.int64, "out")
    nbytes = _ws_bytes("gear_hip_scan_workspace_bytes", n)
    ws = _ws.get("scan", nbytes, weights.device)
    call("gear_hip_scan_i64", _ptr(weights), _ptr(out), n, _ptr(ws), ws.numel(), _stream())
    return out


def sum_f32(values, out=None, out_f64=None):
    _need(values, torch.float32, "values")
    n = values.numel()
    if out is None:
        out = torch.empty(1, dtype=torch.float32, device=values.device)
    nbytes = _ws_bytes("gear_hip_sum_workspace_bytes", n)
    ws = _ws.get("sum", nbytes, values.device)
    call("gear_hip_sum_f32", _ptr(values), n, _ptr(out), _ptr(out_f64), _ptr(ws), ws.numel(),
         _stream())
    return out


def upper_bound(prefix, u, *, unit_uniforms=False, idx_out=None, priorities=None, beta=0.4,
                weights_out=None):
    """Batched search of draws in an fp64 prefix array; optionally importance weights."""
    _need(prefix, torch.float64, "prefix")
    _need(u, torch.float32, "u")
    num = u.numel()
    if idx_out is None:
        idx_out = torch.empty(num, dtype=torch.int64, device=u.device)
    else:
        _need(idx_out, torch.int64, "idx_out")
    ws = None
    if priorities is not None:
        _need(priorities, torch.float32, "priorities")
        if priorities.numel() != prefix.numel():
            raise ValueError("priorities and prefix differ in length")
        if weights_out is None:
            weights_out = torch.empty(num, dtype=torch.float32, device=u.device)
        nbytes = _ws_bytes("gear_hip_search_workspace_bytes", num)
        ws = _ws.get("search", nbytes, u.device)
    call("gear_hip_upper_bound_f64", _ptr(prefix), prefix.numel(), _ptr(u), num,
         int(bool(unit_uniforms)), _ptr(idx_out), _ptr(priorities), float(beta),
         _ptr(weights_out) if priorities is not None else None, _ptr(ws),
         ws.numel() if ws is not None else 0, _stream())
    if priorities is not None:
        return idx_out, weights_out
    return idx_out


def sample_sorted(prefix, u, *, unit_uniforms=True, sorted_out=None, trajectory_length=0,
                  modulo=0, idxs=None, tss=None, lens=None):
    """Search + ascending sort (+ split into window arguments) of one batch of draws."""
    _need(prefix, torch.float64, "prefix")
    _need(u, torch.float32, "u")
    num = u.numel()
    dev = u.device
    if sorted_out is None:
        sorted_out = torch.empty(num, dtype=torch.int64, device=dev)
    if trajectory_length > 0:
        idxs = idxs if idxs is not None else torch.empty(num, dtype=torch.int64, device=dev)
        tss = tss if tss is not None else torch.empty(num, dtype=torch.int64, device=dev)
        lens = lens if lens is not None else torch.empty(num, dtype=torch.int64, device=dev)
    nbytes = _ws_bytes("gear_hip_sample_workspace_bytes", num)
    ws = _ws.get("sample", nbytes, dev)
    call("gear_hip_sample_sorted_f64", _ptr(prefix), prefix.numel(), _ptr(u), num,
         int(bool(unit_uniforms)), _ptr(sorted_out), int(trajectory_length), int(modulo),
         _ptr(idxs), _ptr(tss), _ptr(lens), _ptr(ws), ws.numel(), _stream())
    if trajectory_length > 0:
        return sorted_out, idxs, tss, lens
    return sorted_out


def _lookup_outputs(num, dev, lengths_table, sampled_out, local_out, lens_out):
    empty = lambda: torch.empty(num, dtype=torch.int64, device=dev)
    sampled = sampled_out if sampled_out is not None else empty()
    local = local_out if local_out is not None else empty()
    lens = lens_out if lens_out is not None else (empty() if lengths_table is not None else None)
    return sampled, local, lens


def sample_lookup(prefix, u, *, unit_uniforms=True, index_table=None, index_offset=0,
                  lengths_table=None, sampled_out=None, local_out=None, lens_out=None,
                  start_uniforms=None, window=0, starts_out=None):
    """Weighted draws, sorted, with the loader's look-ups in the same call: positions of the
    draws in the prefix, ascending -> (sampled = index_table[position], local = sampled -
    index_offset, lens = lengths_table[local]).  An fp64 prefix takes float32 draws
    (gear_hip_sample_lookup_f64), an int64 prefix -- a sampler over lengths -- float64 uniforms
    or int64 targets (gear_hip_sample_lookup_i64); there, `start_uniforms` (float64 in [0, 1), one
    per draw) and `window` add a fourth result: starts = floor(start_uniforms * (lens - window + 1)),
    where a window of that many steps begins inside each drawn entry."""
    if start_uniforms is not None and prefix.dtype != torch.int64:
        raise ValueError("window starts come with an int64 prefix only")
    if prefix.dtype == torch.int64:
        _need(prefix, torch.int64, "prefix")
        if unit_uniforms:
            _need(u, torch.float64, "u")
        else:
            _need(u, torch.int64, "u")
        entry = "gear_hip_sample_lookup_i64"
    else:
        _need(prefix, torch.float64, "prefix")
        _need(u, torch.float32, "u")
        entry = "gear_hip_sample_lookup_f64"
    num, dev = u.numel(), u.device
    if index_table is not None:
        _need(index_table, torch.int64, "index_table")
        if index_table.numel() != prefix.numel():
            raise ValueError("index_table and prefix differ in length")
    if lengths_table is not None:
        _need(lengths_table, torch.int64, "lengths_table")
    sampled, local, lens = _lookup_outputs(num, dev, lengths_table, sampled_out, local_out, lens_out)
    ws = _ws.get("sample", _ws_bytes("gear_hip_sample_workspace_bytes", num), dev)
    args = [_ptr(prefix), prefix.numel(), _ptr(u), num, int(bool(unit_uniforms)), _ptr(index_table),
            int(index_offset), _ptr(lengths_table),
            lengths_table.numel() if lengths_table is not None else 0, _ptr(sampled), _ptr(local),
            _ptr(lens)]
    starts = None
    if prefix.dtype == torch.int64:
        if start_uniforms is not None:
            _need(start_uniforms, torch.float64, "start_uniforms")
            if start_uniforms.numel() != num or lengths_table is None or window < 1:
                raise ValueError("window starts need a uniform per draw, lengths_table and window >= 1")
            starts = starts_out if starts_out is not None else torch.empty(
                num, dtype=torch.int64, device=dev)
        args += [_ptr(start_uniforms), int(window), _ptr(starts)]
    call(entry, *args, _ptr(ws), ws.numel(), _stream())
    if starts is not None:
        return sampled, local, lens, starts
    return sampled, local, lens


def sort_lookup(positions, bound, *, index_table=None, index_offset=0, lengths_table=None,
                sampled_out=None, local_out=None, lens_out=None):
    """Given positions (each in [0, bound)): ascending sort, then the same look-ups
    (gear_hip_sort_lookup_i64)."""
    _need(positions, torch.int64, "positions")
    num, dev = positions.numel(), positions.device
    if index_table is not None:
        _need(index_table, torch.int64, "index_table")
    if lengths_table is not None:
        _need(lengths_table, torch.int64, "lengths_table")
    sampled, local, lens = _lookup_outputs(num, dev, lengths_table, sampled_out, local_out, lens_out)
    ws = _ws.get("sample", _ws_bytes("gear_hip_sample_workspace_bytes", num), dev)
    call("gear_hip_sort_lookup_i64", _ptr(positions), num, int(bound), _ptr(index_table),
         index_table.numel() if index_table is not None else 0, int(index_offset),
         _ptr(lengths_table), lengths_table.numel() if lengths_table is not None else 0,
         _ptr(sampled), _ptr(local), _ptr(lens), _ptr(ws), ws.numel(), _stream())
    return sampled, local, lens


def lookup(positions, *, index_table=None, index_offset=0, lengths_table=None, sampled_out=None,
           local_out=None, lens_out=None):
    """The look-ups alone, for positions that are already in the wanted order
    (gear_hip_lookup_i64)."""
    _need(positions, torch.int64, "positions")
    num, dev = positions.numel(), positions.device
    if index_table is not None:
        _need(index_table, torch.int64, "index_table")
    if lengths_table is not None:
        _need(lengths_table, torch.int64, "lengths_table")
    sampled, local, lens = _lookup_outputs(num, dev, lengths_table, sampled_out, local_out, lens_out)
    call("gear_hip_lookup_i64", _ptr(positions), num, _ptr(index_table),
         index_table.numel() if index_table is not None else 0, int(index_offset),
         _ptr(lengths_table), lengths_table.numel() if lengths_table is not None else 0,
         _ptr(sampled), _ptr(local), _ptr(lens), _stream())
    return sampled, local, lens


def upper_bound_i64(prefix, u, *, unit_uniforms=True, idx_out=None):
    _need(prefix, torch.int64, "prefix")
    _need(u, torch.float64 if unit_uniforms else torch.int64, "u")
    num = u.numel()
    if idx_out is None:
        idx_out = torch.empty(num, dtype=torch.int64, device=u.device)
    call("gear_hip_upper_bound_i64", _ptr(prefix), prefix.numel(), _ptr(u), num,
         int(bool(unit_uniforms)), _ptr(idx_out), _stream())
    return idx_out


def sort_i64(keys, vals=None, key_bits=63):
    _need(keys, torch.int64, "keys")
    num = keys.numel()
    keys_out = torch.empty_like(keys)
    vals_out = None
    if vals is not None:
        _need(vals, torch.int64, "vals")
        vals_out = torch.empty_like(vals)
    nbytes = _ws_bytes("gear_hip_sort_workspace_bytes", num)
    ws = _ws.get("sort", nbytes, keys.device)
    call("gear_hip_sort_i64", _ptr(keys), _ptr(keys_out), _ptr(vals), _ptr(vals_out), num,
         int(key_bits), _ptr(ws), ws.numel(), _stream())
    return (keys_out, vals_out) if vals is not None else keys_out


def topk(priorities, k, *, sorted_by_value=True, want_values=True, warm=False, workspace=None):
    """Top-k of fp32 priorities (values, indices), by value descending or by index ascending.
    warm=True: the call may start from the bound that the last call on `workspace` (same n, k and
    order) left there instead of sampling the array; the result is the same either way."""
    _need(priorities, torch.float32, "priorities")
    n = priorities.numel()
    idx = torch.empty(k, dtype=torch.int64, device=priorities.device)
    vals = torch.empty(k, dtype=torch.float32, device=priorities.device) if want_values else None
    nbytes = _ws_bytes("gear_hip_topk_workspace_bytes", n, k)
    ws = workspace if workspace is not None else _ws.get("topk", nbytes, priorities.device)
    if ws.numel() < nbytes:
        raise ValueError("top-k workspace holds %d bytes, %d needed" % (ws.numel(), nbytes))
    call("gear_hip_topk_f32_warm" if warm else "gear_hip_topk_f32", _ptr(priorities), n, int(k),
         int(bool(sorted_by_value)), _ptr(vals), _ptr(idx), _ptr(ws), ws.numel(), _stream())
    return vals, idx


class TopKState:
    """A top-k selection that is repeated on one slowly changing priority array (the priority
    maintenance of a replay buffer): owns the workspace, so that every call after the first can
    take up the bound the call before it left (gear_hip_topk_f32_warm)."""

    def __init__(self):
        self._ws = None
        self._shape = None

    def select(self, priorities, k, *, sorted_by_value=True, want_values=True):
        n = priorities.numel()
        shape = (n, int(k), bool(sorted_by_value), priorities.device)
        nbytes = _ws_bytes("gear_hip_topk_workspace_bytes", n, k)
        warm = self._shape == shape
        if self._ws is None or self._ws.numel() < nbytes or self._ws.device != priorities.device:
            self._ws = torch.empty(max(int(nbytes), 256), dtype=torch.uint8,
                                   device=priorities.device)
            warm = False
        self._shape = shape
        return topk(priorities, k, sorted_by_value=sorted_by_value, want_values=want_values,
                    warm=warm, workspace=self._ws)


def scatter(weights, idx, values, *, unique_indices=False):
    """weights[idx[j]] = values[j]; duplicates: last one wins.  fp32 or int64 tables."""
    if weights.dtype not in (torch.float32, torch.int64):
        raise TypeError("scatter works on float32 or int64 tables")
    _need(weights, weights.dtype, "weights")
    _need(idx, torch.int64, "idx")
    _need(values, weights.dtype, "values")
    num = idx.numel()
    if values.numel() != num:
        raise ValueError("idx and values differ in length")
    ws = None
    if not unique_indices:
        nbytes = _ws_bytes("gear_hip_scatter_workspace_bytes", num)
        ws = _ws.get("scatter", nbytes, weights.device)
    fn = "gear_hip_scatter_f32" if weights.dtype == torch.float32 else "gear_hip_scatter_i64"
    call(fn, _ptr(weights), weights.numel(), _ptr(idx), _ptr(values), num,
         int(bool(unique_indices)), _ptr(ws), ws.numel() if ws is not None else 0, _stream())
    return weights
