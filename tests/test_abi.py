"""CPU-only checks of the drop-in boundary: the shared library loads, exports every
symbol the header declares, and its host-side planning logic agrees with the oracle.
No compute call is made here (there is no GPU on this box)."""
import ctypes
import os
import re

import pytest

from libtbvcoll_amd import tbvcoll

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tbvcoll.h")             # the boundary and the entry points added to it
HEADER_EMU = os.path.join(ROOT, "include", "tbvcoll_emu.h")     # the emulated peer, test hooks, measurement aids
REFERENCE_SYMBOLS = ["tbv_ar_init", "tbv_ar_allreduce", "tbv_ar_stats", "tbv_ar_stats4", "tbv_ar_stats5", "tbv_ar_cap",
                     "tbv_ar_async", "tbv_ar_err", "tbv_ar_rails", "tbv_ar_hist", "tbv_ar_fini"]


def declared_symbols(header=None):
    names = []
    for h in ([header] if header else [HEADER, HEADER_EMU]):
        txt = open(h).read()
        txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
        names += re.findall(r"\b(tbv_(?:ar|emu|step)_\w+)\s*\(", txt)
    return names


def test_library_exports_every_declared_symbol():
    lib = tbvcoll.load()
    names = declared_symbols()
    assert len(names) >= 30
    for n in REFERENCE_SYMBOLS:                      # the eleven the reference's binding uses (step4/tbvcoll.py:19-30)
        assert n in names
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/ but not exported"
    # the boundary header holds no test hook: nothing of the emulated peer is declared there
    main = declared_symbols(HEADER)
    assert not [n for n in main if n.startswith("tbv_emu_")], main
    assert set(REFERENCE_SYMBOLS) <= set(main) and "tbv_step_noalloc" in main
    # and the Python binding binds exactly what the two headers declare
    assert set(tbvcoll._SIGNATURES) == set(names)


def test_calls_before_init_fail_cleanly():
    lib = tbvcoll.load()
    assert lib.tbv_ar_cap() == 0 and lib.tbv_ar_err() == 0
    assert lib.tbv_ar_allreduce(None, None, 16, 0, None) == -1       # not initialised
    assert lib.tbv_ar_allreduce_chunked(None, None, 16, 0, None) == -1
    a, n = ctypes.c_double(-1.0), ctypes.c_ulonglong(99)
    lib.tbv_ar_stats(ctypes.byref(a), ctypes.byref(n))
    assert a.value == 0.0 and n.value == 0
    lib.tbv_ar_stats(None, None); lib.tbv_ar_stats4(None, None, None, None, None)   # NULL-tolerant
    lib.tbv_ar_stats5(None, None, None, None, None, None)
    lib.tbv_ar_fini()                                                 # harmless when nothing runs
    import torch
    assert tbvcoll.all_reduce(torch.zeros(4)) is False                # binding not initialised: caller falls back


def test_missing_library_is_loud(tmp_path):
    with pytest.raises(RuntimeError, match="no fallback"):
        tbvcoll.load(str(tmp_path / "libtbvcoll.so"))


@pytest.mark.parametrize("rails,env", [(2, {}), (2, {"TBV_TAG": "1"}), (3, {}), (4, {"TBV_RAIL1MAX": "4096"}), (1, {})])
def test_rail_plan_against_oracle(orc, rails, env):
    """Slot/rail arithmetic of the shipped engine vs the oracle's restatement of
    step4/libtbvcoll.cpp:173-177,430-431.  They must agree wherever the reference's
    split covers the transfer; where the reference leaves a tail without an owner
    the engine must still cover every byte."""
    lib = tbvcoll.load()
    lib.tbv_emu_shutdown()
    keys = ("TBV_TAG", "TBV_RAIL1MAX", "TBV_NSLOT")
    for k in keys:
        os.environ.pop(k, None)
    os.environ.update(env)
    try:
        assert lib.tbv_emu_configure(",".join("r%d" % i for i in range(rails)).encode(), 16 << 20) == 0
        tag = int(env.get("TBV_TAG", "0"))
        rail1max = int(env.get("TBV_RAIL1MAX", "98304"))
        off = (ctypes.c_size_t * 4)(); ln = (ctypes.c_size_t * 4)()
        for nb in (2, 8192, 57344, 98304, 98306, 110594, 229376, 917504, 1048576, 4 << 20, (16 << 20) - 2, 16 << 20):
            R = lib.tbv_emu_plan(nb, off, ln)
            assert R == orc.lib().orc_rails_for(nb, rail1max, rails)
            xb = orc.lib().orc_xbytes(nb, tag)
            cover = 0
            for r in range(R):
                if ln[r]:
                    assert off[r] == cover and off[r] % 4096 == 0
                    cover += ln[r]
            assert cover == xb                                        # every byte has an owner
            q = xb // R
            if not (q % 4096 == 0 and xb % R):                        # the reference's split is complete here
                for r in range(R):
                    fr = orc.fragment(xb, R, r)
                    assert (fr or (xb, 0)) == (off[r], ln[r]) or (fr is None and ln[r] == 0)
        assert lib.tbv_emu_nslot() == 8                               # default ring depth (step4/libtbvcoll.cpp:287)
    finally:
        for k in keys:
            os.environ.pop(k, None)
        lib.tbv_emu_shutdown()


def test_failed_init_returns_minus_one_and_leaves_nothing_behind():
    lib = tbvcoll.load()
    lib.tbv_emu_shutdown()
    assert lib.tbv_ar_init(0, b"a,b,c,d,e", b"", 18995, 4096) == -1           # five rails: refused before any allocation
    assert lib.tbv_ar_cap() >= 0 and lib.tbv_ar_err() == 0
    assert lib.tbv_ar_allreduce(None, None, 16, 0, None) == -1               # still not initialised
    lib.tbv_emu_shutdown()


def test_configure_rejects_bad_rail_counts():
    lib = tbvcoll.load()
    lib.tbv_emu_shutdown()
    assert lib.tbv_emu_configure(b"a,b,c,d,e", 4096) == -1            # more than four rails (step4/libtbvcoll.cpp:350)
    lib.tbv_emu_shutdown()


def test_configure_bounds_the_cap_by_what_tbv_ar_cap_can_report():
    """tbv_ar_cap returns an int (step4/libtbvcoll.cpp:537): the largest cap is 2 GiB - 4 KiB, rounded like any other."""
    lib = tbvcoll.load()
    lib.tbv_emu_shutdown()
    assert lib.tbv_emu_configure(b"a,b", (1 << 31) - 4096) == 0 and lib.tbv_ar_cap() == (1 << 31) - 4096
    lib.tbv_emu_shutdown()
    assert lib.tbv_emu_configure(b"a,b", (1 << 31) - 4095) == -1
    lib.tbv_emu_shutdown()
    assert lib.tbv_emu_configure(b"a,b", 1 << 40) == -1
    lib.tbv_emu_shutdown()


def test_binding_surface_matches_reference_module():
    for name in ("init", "all_reduce", "is_async", "err", "rails", "hist", "raw_fn", "cap", "stats", "stats3", "stats4",
                 "stats5"):
        assert callable(getattr(tbvcoll, name)), name
    import inspect
    sig = inspect.signature(tbvcoll.init)
    assert list(sig.parameters)[:5] == ["rank", "devs", "peer_ip", "port", "cap_bytes"]
    assert sig.parameters["port"].default == 18995 and sig.parameters["cap_bytes"].default == 8 << 20
    assert list(inspect.signature(tbvcoll.all_reduce).parameters) == ["t", "out"]
