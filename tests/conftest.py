import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # The native libraries are built in-tree by `python -m decx_amd.build` (hipcc cross-compiles
    # without a GPU) and travel with the tree.  A fresh checkout has none: build once, here.
    lib = os.path.join(ROOT, "decx_amd", "lib")
    needed = [os.path.join(lib, "libdecx_hip.so"), os.path.join(lib, "libDECX_BLAS_HIP.so"),
              os.path.join(ROOT, "tests", "cpp", "de_api_test")]
    if not all(os.path.exists(p) for p in needed):
        from decx_amd import build as native
        native.build_all()


@pytest.fixture(scope="session")
def oracle():
    from oracle import binding
    binding.lib()
    return binding
