import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # the tests load what is built; only when nothing is built yet do they build (hipcc cross-compiles without a GPU)
    lib = os.path.join(ROOT, "flashoptim_amd", "lib", "libflashoptim_hip.so")
    if not os.path.exists(lib):
        import subprocess

        subprocess.run(["make", "-j", "8", "-C", os.path.join(ROOT, "flashoptim_amd", "csrc")], check=True,
                       capture_output=True)


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, on a machine without a device, unless -m gpu asked for them."""
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
