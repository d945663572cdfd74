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
    """Tests load what is already built.  They build what is missing, and they build libkhan_aev.so again when the
    stamp beside it (the digest of the sources and flags it was built from) does not match the sources in the tree:
    a library from other sources would pass or fail for the wrong code.  Without hipcc a stale library is an error."""
    oracle_so = os.path.join(ROOT, "oracle", "libkhan_oracle.so")
    if not os.path.exists(oracle_so):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "all"], check=True)
    from khan_amd import build
    datagen_so = os.path.join(ROOT, "khan_amd", "csrc", "libkhan_datagen.so")
    host_so = os.path.join(ROOT, "khan_amd", "csrc", "libkhan_host.so")
    if not os.path.exists(datagen_so):
        build.build_datagen()
    if not os.path.exists(host_so):
        build.build_host()
    stale = [name for name, lib, defines in (("default", build.LIBRARY, ()), ("check", build.CHECK_LIBRARY, build.CHECK_DEFINES))
             if not build.library_is_current(lib, defines)]
    if stale:
        import shutil
        if not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")):
            raise RuntimeError("libkhan_aev.so (%s build) is missing or was built from other sources than the tree's "
                               "(stamp %s, sources %s), and there is no hipcc here to build it"
                               % (", ".join(stale), build.library_stamp(), build.sources_digest()))
        if "default" in stale:
            build.build_hip()
        build.build_check_variant()       # takes the default build's objects


_ensure_built()


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")
