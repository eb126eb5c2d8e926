"""Host-side sanitizer run: `python tests/host_sanitizers.py [pytest args]`.

Builds the host C++ layer (gear_amd/csrc/host/*.cc, the pybind module) and the CPU oracle
(oracle/gear_oracle.c) with AddressSanitizer + UndefinedBehaviorSanitizer and runs the CPU tests
that exercise them (table layout, spans, pickles, handler.sub, request arrays, every oracle
function) in a child pytest process whose native modules are the sanitized builds.  Host code
only: the HIP library is linked as built, and nothing here runs on a GPU.  Exit code = the
child's; any sanitizer report aborts the child (halt_on_error)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TESTS = ["tests/test_host_layer.py", "tests/test_oracle_sampler.py", "tests/test_oracle_storage.py",
         "tests/test_ref_specs.py"]


def main(argv):
    sys.path.insert(0, ROOT)
    from gear_amd import _build
    module, oracle = _build.build_sanitized(os.path.join(ROOT, "gear_amd", "csrc", "build", "san"))
    def gcc_file(name):
        return subprocess.run(["gcc", "-print-file-name=" + name], stdout=subprocess.PIPE,
                              text=True, check=True).stdout.strip()

    env = dict(os.environ)
    # The sanitizer runtime has to come first among the preloaded libraries, and the C++ runtime
    # has to be there when it starts (the interpreter does not link it, and the interceptor of
    # __cxa_throw looks the real one up once, at start); whatever is preloaded already stays
    # behind them.
    env["LD_PRELOAD"] = ":".join([gcc_file("libasan.so"), gcc_file("libstdc++.so.6")] +
                                 ([env["LD_PRELOAD"]] if env.get("LD_PRELOAD") else []))
    # (the interpreter and torch are not instrumented: their exit-time leaks are not the subject)
    env["ASAN_OPTIONS"] = "detect_leaks=0:halt_on_error=1:abort_on_error=1"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    env["GEAR_LIBGEAR_MODULE"] = module
    env["GEAR_ORACLE_LIB"] = oracle
    cmd = [sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] \
        + (argv or TESTS)
    print("host sanitizers: " + " ".join(cmd), flush=True)
    return subprocess.run(cmd, cwd=ROOT, env=env).returncode


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
