"""Build steps for the native parts of gear_amd (hipcc for gfx950, g++ for host code)."""
import os
import subprocess
import sys
import sysconfig

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
CSRC = os.path.join(_PKG, "csrc")
INCLUDE = os.path.join(_ROOT, "include")

HIP_SOURCES = ["runtime.hip", "gather.hip", "scan.hip", "search.hip", "sort.hip", "topk.hip",
               "scatter.hip"]
LIBGEARHIP = os.path.join(_PKG, "libgearhip.so")

# -packed-fp32-ops is switched off on purpose: hipcc -O3 otherwise forms v_pk_*_f32 from plain
# float code.  The host pass of hipcc warns that it does not know the feature; harmless.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


def _run(cmd, cwd=None):
    r = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def build_libgearhip(verbose=False):
    """Compile every HIP source into gear_amd/libgearhip.so (the C-ABI library)."""
    objs = []
    procs = []
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    for src in HIP_SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            raise RuntimeError("missing HIP source %s" % path)
        obj = os.path.join(CSRC, "build", src.replace(".hip", ".o"))
        cmd = [hipcc()] + HIPCC_FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c", path, "-o", obj]
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                            stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out.strip():
            print(out)
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIBGEARHIP] + objs)
    return LIBGEARHIP


def libgear_ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(_PKG, "libgear", "_libgear" + suffix)


def build_libgear_ext():
    """Compile the host C++ layer + pybind11 module (gear_amd/libgear/_libgear*.so)."""
    import pybind11
    host = os.path.join(CSRC, "host")
    srcs = sorted(os.path.join(host, f) for f in os.listdir(host) if f.endswith(".cc"))
    out = libgear_ext_path()
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-I", INCLUDE, "-I", host, "-I", pybind11.get_include(),
           "-I", sysconfig.get_paths()["include"]] + srcs + [
               "-o", out, "-L", _PKG, "-lgearhip", "-Wl,-rpath,$ORIGIN/..", "-ldl", "-lpthread"]
    _run(cmd)
    return out


SANITIZE_FLAGS = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                  "-fno-omit-frame-pointer", "-O1", "-g"]


def build_sanitized(outdir):
    """The host C++ layer (pybind module) and the CPU oracle compiled with AddressSanitizer and
    UndefinedBehaviorSanitizer into `outdir`: host code only, for tests/host_sanitizers.py.  The
    HIP library is linked as it is (never a sanitized GPU build).  Returns the two paths."""
    import pybind11
    os.makedirs(outdir, exist_ok=True)
    host = os.path.join(CSRC, "host")
    srcs = sorted(os.path.join(host, f) for f in os.listdir(host) if f.endswith(".cc"))
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    module = os.path.join(outdir, "_libgear" + suffix)
    _run(["g++", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden"] + SANITIZE_FLAGS +
         ["-I", INCLUDE, "-I", host, "-I", pybind11.get_include(),
          "-I", sysconfig.get_paths()["include"]] + srcs +
         ["-o", module, "-L", _PKG, "-lgearhip", "-Wl,-rpath," + _PKG, "-ldl", "-lpthread"])
    oracle = os.path.join(outdir, "liboracle.so")
    _run(["gcc", "-std=c11", "-fPIC", "-shared", "-fvisibility=hidden", "-fopenmp", "-Wall",
          "-Wextra"] + SANITIZE_FLAGS +
         [os.path.join(_ROOT, "oracle", "gear_oracle.c"), "-o", oracle, "-lm"])
    return module, oracle


def build_all(verbose=False):
    build_libgearhip(verbose)
    if os.path.isdir(os.path.join(CSRC, "host")):
        build_libgear_ext()


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", LIBGEARHIP)
