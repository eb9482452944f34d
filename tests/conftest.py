import glob
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _newest(patterns):
    times = [os.path.getmtime(p) for pat in patterns for p in glob.glob(os.path.join(ROOT, pat))]
    return max(times) if times else 0.0


def _stale(target, sources):
    """True when `target` is missing or older than any of its sources (a source edit without a rebuild would
    otherwise leave the suites testing a stale binary).  Where hipcc is absent (a GPU box that received the built
    files) what is there is used as it is; the library's own source digest check still guards the pairing."""
    path = os.path.join(ROOT, target)
    if not os.path.exists(path):
        return True
    return os.path.getmtime(path) + 1.0 < _newest(sources)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # Tests load what is built; what is missing or older than its sources is built first (hipcc cross-compiles
    # without a GPU).
    lib_sources = ["multimesh-jax_amd/csrc/*", "include/*.h"]
    have_hipcc = subprocess.call(["bash", "-c", "command -v hipcc >/dev/null"]) == 0
    if _stale("multimesh-jax_amd/libmmreshard.so", lib_sources) and (have_hipcc or not os.path.exists(
            os.path.join(ROOT, "multimesh-jax_amd", "libmmreshard.so"))):
        subprocess.check_call(["bash", os.path.join(ROOT, "multimesh-jax_amd", "csrc", "build.sh")])
    if _stale("oracle/libreshard_oracle.so", ["oracle/reshard_cpu.c"]):
        subprocess.check_call(["make", "-s", "-B", "-C", os.path.join(ROOT, "oracle")])
    cpp = ["tests/cpp/*.cc", "tests/cpp/build.sh"] + lib_sources
    # the sanitizer binary is host-only and does not travel to a GPU box: a GPU-only run does not ask for it
    gpu_only = config.getoption("markexpr", "").strip() == "gpu"
    if (_stale("tests/cpp/libmmr_emulation.so", cpp) or _stale("tests/cpp/hip_execute_context_test", cpp)
            or _stale("tests/cpp/libmmr_emulation_span_options.so", cpp)
            or _stale("tests/cpp/context_bench", cpp)
            or (not gpu_only and _stale("tests/cpp/sanitize_sweep", cpp))) and (have_hipcc or not os.path.exists(
                os.path.join(ROOT, "tests", "cpp", "libmmr_emulation.so"))):
        subprocess.check_call(["bash", os.path.join(ROOT, "tests", "cpp", "build.sh")])


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "sharding_golden.json")) as f:
        return json.load(f)
