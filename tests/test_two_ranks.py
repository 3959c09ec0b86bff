"""Two processes on one GPU: the rendezvous (CPU, sockets only) and reference-shape RANK=0/1 drivers that never hand
the library a peer payload (-m gpu).  With TBV_PEER=tcp the library meets its peer the way the reference does (rank 0
listens, rank 1 connects with retries, step4/libtbvcoll.cpp:371-385) and each rail's connection carries its fragments."""
import ctypes
import json
import os
import socket
import subprocess
import sys
import threading

import pytest

from libtbvcoll_amd import tbvcoll

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def free_port():
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    p = s.getsockname()[1]
    s.close()
    return p


RENDEZVOUS_CHILD = r"""
import ctypes, os, sys
sys.path.insert(0, {root!r})
from libtbvcoll_amd import tbvcoll
lib = tbvcoll.load()
lib.tbv_emu_rendezvous.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.c_double]
rank, port, rails, cap, timeout = int(sys.argv[1]), int(sys.argv[2]), int(sys.argv[3]), int(sys.argv[4]), float(sys.argv[5])
assert lib.tbv_emu_configure(",".join("r%d" % i for i in range(rails)).encode(), cap) == 0
rc = lib.tbv_emu_rendezvous(rank, b"127.0.0.1" if rank == 1 else b"", port, timeout)
print("RC", rc, flush=True)
"""


def rendezvous_pair(port, a, b, env_a=None, env_b=None, delay_b=0.0):
    """Run the rendezvous of rank 0 with settings a = (rails, cap) and rank 1 with b in two processes; return their codes."""
    code = RENDEZVOUS_CHILD.format(root=ROOT)
    out = {}

    def run(rank, cfg, env, delay):
        import time
        time.sleep(delay)
        e = dict(os.environ)
        for k in list(e):
            if k.startswith("TBV_"):
                del e[k]
        e.update(env or {})
        p = subprocess.run([sys.executable, "-c", code, str(rank), str(port), str(cfg[0]), str(cfg[1]), str(cfg[2])],
                           capture_output=True, text=True, timeout=60, env=e)
        rc = [ln for ln in p.stdout.splitlines() if ln.startswith("RC ")]
        out[rank] = (int(rc[-1].split()[1]) if rc else None, p.stderr)

    t0 = threading.Thread(target=run, args=(0, a, env_a, 0.0)); t1 = threading.Thread(target=run, args=(1, b, env_b, delay_b))
    t0.start(); t1.start(); t0.join(); t1.join()
    return out


def test_rendezvous_meets_and_compares_settings():
    # both ranks agree: two rails, same cap; rank 1 starts late and finds rank 0 by retrying
    out = rendezvous_pair(free_port(), (2, 1 << 20, 20.0), (2, 1 << 20, 20.0))
    assert out[0][0] == 0 and out[1][0] == 0, out
    out = rendezvous_pair(free_port(), (1, 8192, 20.0), (1, 8192, 20.0), delay_b=1.0)
    assert out[0][0] == 0 and out[1][0] == 0, out
    # rank 1 first: it retries until rank 0 listens
    out = rendezvous_pair(free_port(), (2, 4096, 20.0), (2, 4096, 20.0), delay_b=-0.0)
    assert out[0][0] == 0 and out[1][0] == 0, out


def test_rendezvous_refuses_ranks_that_disagree():
    out = rendezvous_pair(free_port(), (2, 1 << 20, 10.0), (2, 2 << 20, 10.0))                  # different caps
    assert out[0][0] == -1 and out[1][0] == -1, out
    assert "disagree" in out[0][1] + out[1][1]
    out = rendezvous_pair(free_port(), (2, 1 << 20, 10.0), (2, 1 << 20, 10.0), env_b={"TBV_NSLOT": "4"})   # different rings
    assert out[0][0] == -1 and out[1][0] == -1, out
    out = rendezvous_pair(free_port(), (2, 1 << 20, 10.0), (2, 1 << 20, 10.0), env_a={"TBV_TAG": "1"})     # one side tags
    assert out[0][0] == -1 and out[1][0] == -1, out


def test_rendezvous_gives_up_without_a_peer():
    lib = tbvcoll.load()
    lib.tbv_emu_rendezvous.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.c_double]
    lib.tbv_emu_shutdown()
    assert lib.tbv_emu_rendezvous(0, b"", free_port(), 0.5) == -1           # not configured
    assert lib.tbv_emu_configure(b"rail0", 4096) == 0
    assert lib.tbv_emu_rendezvous(0, b"", free_port(), 0.5) == -1           # nobody connects
    assert lib.tbv_emu_rendezvous(1, b"127.0.0.1", free_port(), 0.5) == -1  # nobody listens
    assert lib.tbv_emu_rendezvous(1, b"", free_port(), 0.5) == -1           # rank 1 without rank 0's address
    lib.tbv_emu_shutdown()


def run_two_ranks(env_common, timeout=240):
    port = free_port()
    procs = []
    for rank in (0, 1):
        e = dict(os.environ)
        for k in list(e):
            if k.startswith("TBV_"):
                del e[k]
        e.update({"RANK": str(rank), "PORT": str(port), "TBV_PEER": "tcp", "TBV_WDOG": "20", "TBV_NSLOT": "4",
                  "PYTHONPATH": os.path.join(ROOT, "libtbvcoll_amd") + os.pathsep + e.get("PYTHONPATH", "")})
        if rank == 1:
            e["PEER_IP"] = "127.0.0.1"
        e.update({k: str(v) for k, v in env_common.items()})
        procs.append(subprocess.Popen([sys.executable, "-u", os.path.join(ROOT, "tests", "two_rank_driver.py")], env=e,
                                      stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True))
    results = []
    for rank, p in enumerate(procs):
        try:
            so, se = p.communicate(timeout=timeout)
        except subprocess.TimeoutExpired:
            for q in procs:
                q.kill()                       # exactly the two processes started above
            so, se = p.communicate()
            pytest.fail(f"rank {rank} did not finish: {se[-2000:]}")
        line = [ln for ln in so.splitlines() if ln.startswith("RESULT ")]
        assert line, (rank, p.returncode, so[-1000:], se[-3000:])
        results.append((p.returncode, json.loads(line[-1][7:]), se))
    return results


@pytest.mark.gpu
@pytest.mark.parametrize("env", [{}, {"TBV_ASYNC": 0}, {"TBV_STAGEDMERGE": 0, "TBV_ONEKERNEL": 0, "TBV_FUSEWAIT": 0}, {"TBV_TAG": 1},
                                 {"TBV_RAILSUM": 1}, {"TBV_WIRE": "host"}, {"TBV_CHUNK": 65536, "TBV_UNCACHED": 1}, {"DEVS": "a,b,c"}])
def test_two_processes_exact(env):
    """The counterpart of step4/test_exact.py as two processes on the one GPU: 9 dtype x size cells, both references."""
    from gpu_util import say
    say("two ranks exact", env)
    for rc, res, se in run_two_ranks(dict(MODE="exact", **env)):
        assert rc == 0 and res["ok"], (res, se[-2000:])
        assert len(res["cells"]) == 9 and all(c["same_dt"] and c["same_f32"] for c in res["cells"])
        assert "peer = a second process" in se


@pytest.mark.gpu
@pytest.mark.parametrize("dt,nb,iters,env", [("bf16", 57344, 600, {}), ("f16", 229376, 300, {}), ("f32", 8192, 600, {"DEVS": "rail0"}),
                                             ("bf16", 4 << 20, 60, {}), ("bf16", 1 << 20, 100, {"TBV_CODEC": 1, "TBV_CODEC_MIN": 1 << 30})])
def test_two_processes_stress(dt, nb, iters, env):
    """The counterpart of step4/test_stress.py: back-to-back calls without synchronisation, all checked at the end."""
    from gpu_util import say
    say("two ranks stress", dt, nb, iters, env)
    for rc, res, se in run_two_ranks(dict(MODE="stress", DT=dt, BYTES=nb, ITERS=iters, **env)):
        assert rc == 0 and res["ok"] and res["bad"] == 0 and res["async"], (res, se[-2000:])
