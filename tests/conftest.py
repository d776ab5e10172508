import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _ensure_built():
    """The tests load what is built; only when nothing is (a fresh checkout) do they run the
    same makefiles __graft_entry__.build() runs.  hipcc cross-compiles without a GPU."""
    lib = os.path.join(ROOT, "deers_amd", "libdeers_rocm.so")
    host = os.path.join(ROOT, "deers_amd", "host", "host_test")
    if not os.path.exists(lib) and shutil.which("hipcc"):
        subprocess.run(["make", "-C", os.path.join(ROOT, "deers_amd", "csrc"), "-j8"], check=True,
                       capture_output=True)
    if not os.path.exists(host) and os.path.exists(lib) and shutil.which("g++"):
        subprocess.run(["make", "-C", os.path.join(ROOT, "deers_amd", "host")], check=True,
                       capture_output=True)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    _ensure_built()
