import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load what is built; in a tree where nothing has been built yet (a fresh checkout) they build the host
    library, the oracle and the stand-alone runner first (the product itself never does: it fails loudly without its
    library).  Kernels are compiled on demand through the library either way."""
    import subprocess
    from codegendemo_amd import _native
    if not os.path.exists(_native.LIB_PATH):
        _native.build_library(verbose=False)
    if not os.path.exists(os.path.join(ROOT, "oracle", "liboracle.so")):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    if not os.path.exists(os.path.join(ROOT, "codegendemo_amd", "kcg_runner")) and os.path.exists("/opt/rocm/bin/hipcc"):
        subprocess.run(["make", "-C", _native.CSRC_DIR, "runner"], check=True, capture_output=True)


@pytest.fixture(scope="session")
def oracle():
    from tests import oracle_binding
    return oracle_binding.load()
