import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # Tests load what is built; only when nothing is built do they build it (hipcc cross-compiles without a GPU).
    import subprocess
    if not os.path.exists(os.path.join(ROOT, "multimesh-jax_amd", "libmmreshard.so")):
        subprocess.check_call(["bash", os.path.join(ROOT, "multimesh-jax_amd", "csrc", "build.sh")])
    if not os.path.exists(os.path.join(ROOT, "oracle", "libreshard_oracle.so")):
        subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle")])
    if not (os.path.exists(os.path.join(ROOT, "tests", "cpp", "libmmr_emulation.so"))
            and os.path.exists(os.path.join(ROOT, "tests", "cpp", "hip_execute_context_test"))
            and os.path.exists(os.path.join(ROOT, "tests", "cpp", "sanitize_sweep"))):
        subprocess.check_call(["bash", os.path.join(ROOT, "tests", "cpp", "build.sh")])


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "sharding_golden.json")) as f:
        return json.load(f)
