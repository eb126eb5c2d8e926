"""`libgear`: the host library of GEAR (C++/pybind11) over the MI355X kernels.

`gear_amd.libgear.core` carries the names of the reference's `libgear.core`
(src/pybind.cc:75-109 of bigrl-team/gear): specs, TrajectoryTable, SubscribePattern,
get_cpu_handler / CpuTrajectoryStorageHandler, Indexset, the Memory classes, the *Span views,
DataType and the kernel launchers init / copy / vcopy / copy_debug / sum / prefix_sum.
"""
import os as _os
import sys as _sys

try:
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

__all__ = ["core", "comm"]
