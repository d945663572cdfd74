import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _ensure_built():
    """Tests load what is already built; they build only if nothing is there."""
    oracle_so = os.path.join(ROOT, "oracle", "libkhan_oracle.so")
    if not os.path.exists(oracle_so):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "all"], check=True)
    datagen_so = os.path.join(ROOT, "khan_amd", "csrc", "libkhan_datagen.so")
    aev_so = os.path.join(ROOT, "khan_amd", "csrc", "libkhan_aev.so")
    host_so = os.path.join(ROOT, "khan_amd", "csrc", "libkhan_host.so")
    if not os.path.exists(datagen_so) or not os.path.exists(aev_so) or not os.path.exists(host_so):
        from khan_amd import build
        if not os.path.exists(datagen_so):
            build.build_datagen()
        if not os.path.exists(host_so):
            build.build_host()
        if not os.path.exists(aev_so):
            build.build_hip()


_ensure_built()


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")
