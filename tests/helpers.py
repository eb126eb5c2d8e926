"""Synthetic tables in GEAR's byte layout, built with numpy only (independent of the oracle).

Layout (reference src/storage/table.cc:8-25, src/storage/handler.cc:93-96,223-229):
    address(i, c, t) = i*S + A_c*T + t*s_c,  S = T*sum(s_c),  A_c = sum_{j<c} s_j
"""
import numpy as np

NP_DTYPES = {"float32": np.float32, "int32": np.int32, "uint8": np.uint8, "int64": np.int64,
             "float64": np.float64, "int16": np.int16, "bool": np.bool_, "int8": np.int8}


class Schema:
    def __init__(self, columns, T, capacity):
        """columns: list of (name, dtype-name, shape tuple)"""
        self.columns = columns
        self.T = T
        self.capacity = capacity
        self.step_bytes = [int(np.dtype(NP_DTYPES[d]).itemsize * int(np.prod(s, dtype=np.int64)))
                           for _, d, s in columns]
        self.accu = [0]
        for b in self.step_bytes:
            self.accu.append(self.accu[-1] + b)
        self.traj_stride = self.accu[-1] * T
        self.nbytes = self.traj_stride * capacity

    def col_base(self, c):
        return self.accu[c] * self.T

    def column_view(self, table, c):
        """numpy view [capacity, T, *shape] of column c inside the uint8 table (no copy)."""
        name, d, shape = self.columns[c]
        dt = np.dtype(NP_DTYPES[d])
        sb = self.step_bytes[c]
        rows = np.lib.stride_tricks.as_strided(
            table[self.col_base(c):], shape=(self.capacity, self.T * sb),
            strides=(self.traj_stride, 1), writeable=True)
        return rows, dt, shape


def fill_random(schema, seed):
    """uint8 table with random payload in every column (raw random bytes: every bit pattern)."""
    rng = np.random.default_rng(seed)
    return rng.integers(0, 256, size=schema.nbytes, dtype=np.uint8)


def numpy_window_gather(schema, table, c, idxs, tss, lens, ofst, span, pad_head):
    """Independent statement of the window gather with numpy slicing; returns (dst, mask)."""
    sb = schema.step_bytes[c]
    n = len(idxs)
    dst = np.zeros((n, span * sb), np.uint8)
    mask = np.zeros((n, span), np.uint8)
    for g in range(n):
        start = max(int(tss[g]) + ofst, 0)
        end = min(start + span, int(lens[g]))
        steps = max(end - start, 0)
        if steps == 0:
            continue
        a = int(idxs[g]) * schema.traj_stride + schema.col_base(c) + start * sb
        chunk = table[a:a + steps * sb]
        if pad_head:
            dst[g, span * sb - steps * sb:] = chunk
            mask[g, span - steps:] = 1
        else:
            dst[g, :steps * sb] = chunk
            mask[g, :steps] = 1
    return dst, mask
