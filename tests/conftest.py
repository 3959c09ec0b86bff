import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # load what is built; build only if nothing is (hipcc cross-compiles gfx950 without a GPU)
    import subprocess
    if not os.path.exists(os.path.join(ROOT, "libtbvcoll_amd", "libtbvcoll.so")):
        subprocess.run(["make", "-C", os.path.join(ROOT, "libtbvcoll_amd", "csrc")], check=True, stdout=subprocess.DEVNULL)
    if not (os.path.exists(os.path.join(ROOT, "oracle", "liborc.so")) and os.path.exists(os.path.join(ROOT, "oracle", "libhiphdr.so"))):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, stdout=subprocess.DEVNULL)


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.lib()
    return oracle
