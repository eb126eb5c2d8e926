"""CPU tests of the boundary: libgearhip.so loads without a GPU, exports every function that
include/gear_hip.h declares, the ctypes table covers exactly those, and argument errors are
reported by return code before any device work."""
import ctypes
import os
import re

from gear_amd import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "gear_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gear_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_functions_are_exported_and_bound():
    names = _declared()
    assert len(names) >= 30
    lib = _cabi.load()
    for n in names:
        assert getattr(lib, n) is not None, n
    assert sorted(_cabi.SIGNATURES) == names


def test_every_declaration_cites_the_reference_or_says_it_has_no_counterpart():
    text = open(os.path.join(ROOT, "include", "gear_hip.h")).read()
    for cite in ("src/cuda/copy.cu", "src/storage/handler.cc", "src/cuda/one_dim_prefix_sum.cu",
                 "src/cuda/one_dim_sum.cu", "gear/sampler/global_sampler.py", "src/cuda/init.cu",
                 "include/index/set.h", "src/index/request.cc", "src/memory/shared_memory.cc"):
        assert cite in text, cite


def test_error_paths_without_gpu():
    lib = _cabi.load()
    assert lib.gear_hip_abi_version() == 1
    assert lib.gear_hip_error_string(0) == b"success"
    assert b"workspace" in lib.gear_hip_error_string(-2)
    n = ctypes.c_int(-5)
    assert lib.gear_hip_device_count(ctypes.byref(n)) == 0 or n.value == 0
    # negative sizes / null pointers are refused on the host
    assert lib.gear_hip_subcopy(None, None, -1, None, None, None, 0, 0, 1, 1, 1, 0, 1, 1, None,
                                None) == -1
    assert lib.gear_hip_subcopy(None, None, 4, None, None, None, 0, 0, 1, 1, 1, 0, 1, 1, None,
                                None) == -1
    assert lib.gear_hip_vcopy(None, None, 3, None, None, None, 16, None) == -1
    assert lib.gear_hip_scan_f32_f64(None, None, 10, None, 0, None) == -1
    assert lib.gear_hip_scan_f32_f64(None, None, -1, None, 0, None) == -1
    assert lib.gear_hip_topk_f32(None, 10, 11, 1, None, None, None, 0, None) == -1
    assert lib.gear_hip_sort_i64(None, None, None, None, 5, 70, None, 0, None) == -1
    # zero-sized work succeeds without touching the device
    assert lib.gear_hip_subcopy(None, None, 0, None, None, None, 0, 0, 1, 1, 1, 0, 1, 1, None,
                                None) == 0
    assert lib.gear_hip_scan_f32_f64(None, None, 0, None, 0, None) == 0
    # the allocation-free scan checks its size limit before it touches the device
    assert lib.gear_hip_scan_static_max_n() == 1 << 27
    assert lib.gear_hip_scan_f32_f64_static(None, None, (1 << 27) + 1, None) == -3
    assert lib.gear_hip_scan_f32_f64_static(None, None, -1, None) == -1
    assert lib.gear_hip_scan_f32_f64_static(None, None, 0, None) == 0
    # workspace queries are pure host arithmetic
    assert lib.gear_hip_scan_workspace_bytes(1_000_000) >= 256 + 16 * 245
    assert lib.gear_hip_topk_workspace_bytes(10_000_000, 65_536) > 6 * 4 * 65_536
    assert lib.gear_hip_sort_workspace_bytes(4096) >= 2 * 8 * 4096


def test_missing_library_is_loud(tmp_path, monkeypatch):
    import pytest
    monkeypatch.setattr(_cabi, "_lib", None)
    monkeypatch.setattr(_cabi, "LIB_PATH", str(tmp_path / "libgearhip.so"))
    with pytest.raises(ImportError):
        _cabi.load()


def test_header_is_plain_c(tmp_path):
    """include/gear_hip.h is the boundary a C, Go (cgo) or Rust binding would consume: it must
    compile as C99 on its own."""
    import shutil
    import subprocess

    import pytest
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include "gear_hip.h"\nint main(void) { return GEAR_HIP_ABI_VERSION < 0; }\n')
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, "-c",
                    str(src), "-o", str(tmp_path / "use_header.o")], check=True)
