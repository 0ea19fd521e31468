import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# CATGRAD_ORACLE_LIB: another build of the oracle (the sanitizer build of `make -C oracle SAN=1 san-test`)
ORACLE_LIB = os.environ.get("CATGRAD_ORACLE_LIB") or os.path.join(ROOT, "oracle", "liboracle.so")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def cg():
    return importlib.import_module("catgrad-rs_amd")


@pytest.fixture(scope="session")
def oracle_lib(cg):
    if not os.path.exists(ORACLE_LIB):
        import subprocess
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    return cg.load_library(ORACLE_LIB)


@pytest.fixture(scope="session")
def oracle(cg, oracle_lib):
    """The CPU restatement of NdArrayBackend: the checker."""
    return cg.Backend(oracle_lib)


@pytest.fixture(scope="session")
def hip_lib(cg):
    return cg.load_library()


@pytest.fixture(scope="session")
def hip(cg, hip_lib):
    """The product: deferred (fusing) mode, f32."""
    return cg.Backend(hip_lib)


@pytest.fixture(scope="session")
def hip_eager(cg, hip_lib):
    return cg.Backend(hip_lib, flags=cg.FLAG_EAGER)


@pytest.fixture(scope="session")
def hip_bf16(cg, hip_lib):
    return cg.Backend(hip_lib, flags=cg.FLAG_BF16)


@pytest.fixture(scope="session")
def hip_nopat(cg, hip_lib):
    """Deferred mode with the hand-written pattern kernels switched off (generic programs only)."""
    return cg.Backend(hip_lib, flags=4)
