"""The allocation-free scan entry point (gear_hip_scan_f32_f64_static) against the workspace
form it is a variant of (gear_hip_scan_f32_f64): bit-identical prefixes, through the C ABI, on
calls in a row that share the library's static device array."""
import ctypes

import numpy as np
import pytest
import torch

from gear_amd import _cabi
from tests.conftest import announce

pytestmark = pytest.mark.gpu


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _scan_workspace(lib, pri):
    n = pri.numel()
    out = torch.empty(n, dtype=torch.float64, device="cuda")
    nbytes = lib.gear_hip_scan_workspace_bytes(n)
    ws = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device="cuda")
    rc = lib.gear_hip_scan_f32_f64(_p(pri), _p(out), n, _p(ws), ws.numel(), _stream())
    assert rc == 0, rc
    return out


def _scan_static(lib, pri, out):
    rc = lib.gear_hip_scan_f32_f64_static(_p(pri), _p(out), pri.numel(), _stream())
    assert rc == 0, rc
    return out


def test_static_scan_equals_workspace_scan_on_consecutive_calls(oracle):
    lib = _cabi.load()
    assert lib.gear_hip_set_device(0) == 0
    rng = np.random.default_rng(77)
    # second call smaller than the first, third larger again, last one a single ragged range:
    # every call finds the previous call's range sums in the shared array
    sizes = [3_000_001, 70_001, 10_000_000, 777]
    outs = {n: torch.empty(n, dtype=torch.float64, device="cuda") for n in sizes}
    for n in sizes:
        announce("static scan n=%d" % n)
        host = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
        pri = torch.from_numpy(host).cuda()
        torch.cuda.synchronize()
        # free device memory as the driver reports it (hipMemGetInfo): a hipMalloc or hipFree
        # inside the library would show here, torch's own allocator statistics would not
        free_before = torch.cuda.mem_get_info()[0]
        got = _scan_static(lib, pri, outs[n])
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        exp = _scan_workspace(lib, pri)
        torch.cuda.synchronize()
        assert torch.equal(got, exp), n
        if n <= 70_001:
            ref = oracle.scan_f32_f64(host)
            assert np.max(np.abs(got.cpu().numpy() - ref) / ref) <= 1e-12
    # integer-valued priorities: exact in any summation order, so the oracle pins every bit
    host = rng.integers(0, 1000, size=1_234_567).astype(np.float32)
    pri = torch.from_numpy(host).cuda()
    got = _scan_static(lib, pri, torch.empty(host.size, dtype=torch.float64, device="cuda"))
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), oracle.scan_f32_f64(host))


def test_static_scans_from_two_streams_are_ordered_by_the_library():
    """Two streams issue static scans one right after the other, with nothing between them but
    the library's own event: the second call's kernels wait for the first call's, so neither
    finds the other's range sums in the shared array."""
    lib = _cabi.load()
    assert lib.gear_hip_set_device(0) == 0
    rng = np.random.default_rng(78)
    hosts = [(rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
             for n in (9_000_001, 2_500_000, 6_000_000, 300_000)]
    pris = [torch.from_numpy(h).cuda() for h in hosts]
    outs = [torch.empty(h.size, dtype=torch.float64, device="cuda") for h in hosts]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    announce("static scans alternating between two streams")
    for i, (pri, out) in enumerate(zip(pris, outs)):
        st = ctypes.c_void_p(streams[i % 2].cuda_stream)
        assert lib.gear_hip_scan_f32_f64_static(_p(pri), _p(out), pri.numel(), st) == 0
    torch.cuda.synchronize()
    for pri, out in zip(pris, outs):
        assert torch.equal(out, _scan_workspace(lib, pri)), pri.numel()


def test_static_scan_rejects_what_it_cannot_hold():
    lib = _cabi.load()
    max_n = lib.gear_hip_scan_static_max_n()
    assert max_n == 1 << 27
    x = torch.zeros(16, dtype=torch.float32, device="cuda")
    o = torch.zeros(16, dtype=torch.float64, device="cuda")
    assert lib.gear_hip_scan_f32_f64_static(_p(x), _p(o), max_n + 1, _stream()) == -3
    assert lib.gear_hip_scan_f32_f64_static(_p(x), _p(o), -1, _stream()) == -1
    assert lib.gear_hip_scan_f32_f64_static(None, None, 0, _stream()) == 0
    assert b"range" in lib.gear_hip_error_string(-3)
