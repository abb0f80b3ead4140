import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


# a tuning store on the machine must not change what the tests launch (the reference's
# test main does the same: tests/test_main.cpp:21-26)
os.environ["VKERNELS_TUNING_CACHE"] = "off"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle
    oracle.lib()  # builds liboracle.so with gcc when it is not there yet
    return oracle


@pytest.fixture(scope="session")
def hip_lib():
    """The built device library; GPU tests fail loudly when it is missing."""
    from vkernels_amd import vllm_experts as ve
    path = ve.find_libvkernels_hip()
    if path is None:
        from vkernels_amd import build
        build.build()
    return ve.load_libvkernels_hip()
