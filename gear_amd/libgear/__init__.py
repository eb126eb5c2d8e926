"""`libgear`: the host library of GEAR (C++/pybind11) over the MI355X kernels.

`gear_amd.libgear.core` carries the names of the reference's `libgear.core`
(src/pybind.cc:75-109 of bigrl-team/gear): specs, TrajectoryTable, SubscribePattern,
get_cpu_handler / CpuTrajectoryStorageHandler, Indexset, the Memory classes, the *Span views,
DataType and the kernel launchers init / copy / vcopy / copy_debug / sum / prefix_sum.
"""
import os as _os
import sys as _sys

try:
    _alt = _os.environ.get("GEAR_LIBGEAR_MODULE")
    if _alt:
        # another build of the same module (the host-sanitizer run of tests/host_sanitizers.py)
        import importlib.machinery as _mach
        import importlib.util as _util
        _loader = _mach.ExtensionFileLoader(__name__ + "._libgear", _alt)
        _spec = _util.spec_from_file_location(__name__ + "._libgear", _alt, loader=_loader)
        _libgear = _util.module_from_spec(_spec)
        _loader.exec_module(_libgear)
        _sys.modules[__name__ + "._libgear"] = _libgear
    else:
        from . import _libgear
except ImportError as _e:  # pragma: no cover - only without a build
    raise ImportError(
        "gear_amd.libgear: the native module is not built; run "
        "`python -c 'import __graft_entry__ as g; g.build()'` in the repository root"
    ) from _e

core = _libgear.core
comm = _libgear.comm
_sys.modules[__name__ + ".core"] = core
_sys.modules[__name__ + ".comm"] = comm

# Pickles written by the reference name its classes `libgear.core.<Class>`
# (src/storage/pybind.cc:28-40,53-69,85-99,178-204; src/index/pybind.cc:299-306).  The classes here
# carry the same module path and the same state tuples, so checkpoints travel in both directions;
# the names `libgear`, `libgear.core` resolve to this package unless a real `libgear` is installed.
for _name in dir(core):
    _obj = getattr(core, _name)
    if isinstance(_obj, type):
        try:
            _obj.__module__ = "libgear.core"
        except (AttributeError, TypeError):
            pass
        for _inner in vars(_obj).values():
            if isinstance(_inner, type):
                try:
                    _inner.__module__ = "libgear.core"
                except (AttributeError, TypeError):
                    pass
_sys.modules.setdefault("libgear", _sys.modules[__name__])
_sys.modules.setdefault("libgear.core", core)
_sys.modules.setdefault("libgear.comm", comm)

__all__ = ["core", "comm"]
