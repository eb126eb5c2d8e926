"""The host layer's and the oracle's layout arithmetic against the reference's OWN object code:
oracle/_ref/libref_specs.so is src/storage/specs.cc with include/storage/specs.h and
include/common/dtypes.h of the reference, compiled as they lie (oracle/Makefile, target `ref`).
Skipped where that library was never built (it is built wherever the reference tree is present)."""
import numpy as np
import pytest

from gear_amd.libgear import core as glibc

NAMES = ["bool", "int8", "uint8", "int16", "int32", "int64", "float16", "float32", "float64"]
# What the reference's C++ receives for a dtype is the integer of the Python-visible enumerator
# (src/common/pybind.cc:50-75 binds "int8" to kByte = 1 and "uint8" to kChar = 2); this module's
# enumerators carry the same integers, so they are passed to the reference's code as they are.
REF_CODE = {name: int(getattr(glibc, name)) for name in NAMES}


@pytest.fixture(scope="module")
def ref(oracle):
    if oracle.ref_specs() is None:
        pytest.skip("oracle/_ref/libref_specs.so not built (make -C oracle ref needs the reference tree)")
    return oracle


def test_sizeof_dtype_equals_the_reference(ref):
    for name in NAMES:
        want = ref.ref_sizeof_dtype(REF_CODE[name])
        if want < 0:                                  # the reference throws (float16)
            with pytest.raises(RuntimeError, match="Unsupported type"):
                glibc.sizeof_dtype(getattr(glibc, name))
        else:
            assert glibc.sizeof_dtype(getattr(glibc, name)) == want, name
    assert ref.ref_sizeof_dtype(REF_CODE["float16"]) == -1
    assert ref.ref_sizeof_dtype(99) == -1


def test_column_and_table_sizes_equal_the_reference(ref):
    rng = np.random.default_rng(11)
    usable = [n for n in NAMES if n != "float16"]
    for _ in range(200):
        ncols = int(rng.integers(1, 7))
        cols = []
        for _c in range(ncols):
            shape = [int(d) for d in rng.integers(1, 9, size=int(rng.integers(1, 4)))]
            cols.append((shape, usable[int(rng.integers(0, len(usable)))]))
        T, cap = int(rng.integers(1, 1200)), int(rng.integers(1, 5000))
        specs = [glibc.ColumnSpec(shape, getattr(glibc, dt), "col%d" % i)
                 for i, (shape, dt) in enumerate(cols)]
        for spec, (shape, dt) in zip(specs, cols):
            assert spec.size() == ref.ref_column_size(shape, REF_CODE[dt])
        table = glibc.TableSpec(0, 1, T, cap, ncols, specs)
        rcols = [(shape, REF_CODE[dt]) for shape, dt in cols]
        assert table.size() == ref.ref_table_nbytes(T, cap, rcols)
        # the oracle's layout of the same table
        _, stride, total = ref.layout([s.size() for s in specs], T, cap)
        assert total == ref.ref_table_nbytes(T, cap, rcols) and stride * cap == total
        pick = int(rng.integers(0, ncols))
        assert table.index("col%d" % pick) == ref.ref_table_index(rcols, "col%d" % pick) == pick
        assert table.index("nope") == ref.ref_table_index(rcols, "nope") == -1


def test_baseline_tables_equal_the_reference(ref):
    """The five benchmark tables' byte sizes from the reference's TableSpec."""
    atari = [([4, 84, 84], REF_CODE["uint8"]), ([1], REF_CODE["int32"]), ([1], REF_CODE["float32"]),
             ([1], REF_CODE["uint8"])]
    assert ref.ref_table_nbytes(1000, 1000, atari) == 28_233_000_000
    assert ref.ref_table_nbytes(1000, 2000, atari) == 56_466_000_000
    mujoco = [([17], REF_CODE["float32"]), ([6], REF_CODE["float32"]), ([1], REF_CODE["float32"]),
              ([1], REF_CODE["uint8"])]
    assert ref.ref_table_nbytes(64, 4096, mujoco) == 97 * 64 * 4096
