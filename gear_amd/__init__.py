"""gear_amd: the replay-sampling hot path of GEAR, rebuilt for one AMD Instinct MI355X (gfx950).

Layers (bottom up):
  gear_amd/csrc/*.hip      hand-written HIP kernels behind the C ABI of include/gear_hip.h
  gear_amd/libgearhip.so   that C ABI (built by gear_amd._build / __graft_entry__.build)
  gear_amd._cabi           ctypes binding of the C ABI
  gear_amd.ops             tensor-level calls (torch tensors only carry device memory + stream)
"""
__version__ = "0.1.0"
