import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
for p in (HERE, ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a GPU (runs the HIP path through the C ABI)")


@pytest.fixture(scope="session")
def oracle_lib():
    """The CPU restatement; built on demand (a 10 s g++ compile) when the .so is not there yet."""
    import cpu_ref
    if not os.path.exists(cpu_ref.ORACLE_PATH):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "oracle"])
    return cpu_ref.load_oracle()


@pytest.fixture(scope="session")
def reference_lib():
    """The compiled reference (oracle/_ref), or skip when it was not built."""
    import cpu_ref
    lib = cpu_ref.load_reference()
    if lib is None:
        pytest.skip("oracle/_ref/libnd4j_ref.so not built (needs the reference tree)")
    return lib


@pytest.fixture(scope="session")
def cpu_checker():
    """Best available CPU checker for GPU parity: the compiled reference when present, else the restatement."""
    import cpu_ref
    lib = cpu_ref.load_reference()
    if lib is None:
        if not os.path.exists(cpu_ref.ORACLE_PATH):
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "oracle"])
        lib = cpu_ref.load_oracle()
    return lib


@pytest.fixture(scope="session")
def gpu():
    import backends
    return backends.GpuBackend()
