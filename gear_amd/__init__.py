"""gear_amd: the replay-sampling hot path of GEAR, rebuilt for one AMD Instinct MI355X (gfx950).

Layers (bottom up):
  gear_amd/csrc/*.hip      hand-written HIP kernels behind the C ABI of include/gear_hip.h
  gear_amd/libgearhip.so   that C ABI (built by gear_amd._build / __graft_entry__.build)
  gear_amd._cabi           ctypes binding of the C ABI
  gear_amd.ops             tensor-level calls (torch tensors only carry device memory + stream)
  gear_amd/csrc/host       host C++ (specs, table layout, patterns, handler, index set, memory)
  gear_amd.libgear         pybind11 module with the reference's `libgear.core` names
  gear_amd.{specs,dtypes,sampler,loader,dataset,mpu}   the reference's `gear` Python API
"""
__version__ = "0.1.0"


def init(device_id=None):
    """Select the GPU of this process (reference gear/__init__.py:8-24: LOCAL_RANK or 0)."""
    import os
    from .libgear import core as glibc
    if device_id is None:
        device_id = int(os.environ.get("LOCAL_RANK", 0))
    glibc.init(device_id)


def check_visible_device():
    from .libgear import core as glibc
    glibc.print_environ()


def install_as_gear():
    """Register this package under the reference's module names, so that code written against
    the reference (`import gear`, `import libgear.core as glibc`) runs unchanged."""
    import importlib
    import sys
    me = sys.modules[__name__]
    from . import libgear
    sys.modules.setdefault("libgear", libgear)
    sys.modules.setdefault("libgear.core", libgear.core)
    sys.modules.setdefault("libgear.comm", libgear.comm)
    sys.modules.setdefault("gear", me)
    for sub in ("config", "errors", "dtypes", "specs", "utils", "mpu", "sampler", "dataset",
                "loader"):
        mod = importlib.import_module(__name__ + "." + sub)
        sys.modules.setdefault("gear." + sub, mod)
        setattr(me, sub, mod)
    # modules that pickled objects of the reference name (SharedDatasetMeta, IndexMeta)
    for sub in ("dataset.shared_dataset", "sampler.global_sampler", "loader.offline_loader"):
        sys.modules.setdefault("gear." + sub, importlib.import_module(__name__ + "." + sub))
    # BasicLoader lives beside OfflineLoader here
    sys.modules.setdefault("gear.loader.basic_loader",
                           importlib.import_module(__name__ + ".loader.offline_loader"))
    return me
