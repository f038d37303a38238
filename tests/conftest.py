import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ko():
    """The product library on a GPU box.  No fallback: a missing library or device is an error."""
    import kernel_optimization_amd as ko_mod
    ko_mod.lib()
    info = ko_mod.device_info()  # raises KoError(KO_ERR_NO_DEVICE) without a GPU
    assert "gfx950" in info["arch"], "libko.so is built for gfx950 only, found %s" % info["arch"]
    return ko_mod
