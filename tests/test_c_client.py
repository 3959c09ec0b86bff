"""A plain C program against include/tbvcoll.h and libtbvcoll.so: the header is valid C,
every symbol it uses links (CPU), and the program's all-reduces are exact (GPU)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_abi_client.c")
LIBDIR = os.path.join(ROOT, "libtbvcoll_amd")


def build(out):
    cmd = ["gcc", "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"),
           "-I", "/opt/rocm/include", SRC, "-o", out, "-L", LIBDIR, "-ltbvcoll", "-L", "/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath," + LIBDIR, "-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(cmd, check=True)


def test_header_is_c_and_client_links(tmp_path):
    exe = str(tmp_path / "c_client")
    build(exe)
    assert os.path.exists(exe)


@pytest.mark.gpu
def test_c_client_runs_exact(tmp_path):
    exe = str(tmp_path / "c_client")
    build(exe)
    env = dict(os.environ, TBV_NSLOT="4", TBV_WDOG="5")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    print(r.stdout, r.stderr)
    assert r.returncode == 0 and "C client OK" in r.stdout and "MISMATCH" not in r.stdout
