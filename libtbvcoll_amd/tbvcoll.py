"""tbvcoll -- ctypes binding of libtbvcoll.so (MI355X build).

Same module surface as the reference binding (step4/tbvcoll.py:14-111): `init`,
`all_reduce`, `is_async`, `err`, `rails`, `hist`, `raw_fn`, `cap`, `stats`,
`stats3`, `stats4`, `stats5`, with the same guards and return conventions, so a
caller written against the reference (an exact/stress driver, a vLLM
`GroupCoordinator.all_reduce` intercept) runs unchanged.

    import tbvcoll
    tbvcoll.init(rank, "rail0,rail1", "", cap_bytes=8 << 20)
    tbvcoll.all_reduce(t)              # in-place SUM; False -> caller falls back

Additions (no counterpart in the reference) drive the emulated peer that
replaces the wire: `stage_peer`, `stage_peer_repeat`, `peer_resident`,
`arrival_script`, `withhold`, `latency_probe`, `latencies`, `arrival_log`,
`all_reduce_chunked`, `shutdown`, `lib`.

There is no CPU fallback: if the shared library is missing, `init` raises.
"""
import ctypes
import os

import torch

_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_lib = None
_cap = 0
_DEFAULT_SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtbvcoll.so")


def _bind(so):
    l = ctypes.CDLL(so)
    vp, sz, ci, dp, up = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.POINTER(ctypes.c_double), \
        ctypes.POINTER(ctypes.c_ulonglong)
    l.tbv_ar_init.argtypes = [ci, ctypes.c_char_p, ctypes.c_char_p, ci, sz]; l.tbv_ar_init.restype = ci
    l.tbv_ar_allreduce.argtypes = [vp, vp, sz, ci, vp]; l.tbv_ar_allreduce.restype = ci
    l.tbv_ar_stats.argtypes = [dp, up]; l.tbv_ar_stats.restype = None
    l.tbv_ar_stats4.argtypes = [dp] * 4 + [up]; l.tbv_ar_stats4.restype = None
    l.tbv_ar_stats5.argtypes = [dp] * 5 + [up]; l.tbv_ar_stats5.restype = None
    for name in ("tbv_ar_async", "tbv_ar_err", "tbv_ar_cap"):
        getattr(l, name).argtypes = []; getattr(l, name).restype = ci
    for name in ("tbv_ar_rails", "tbv_ar_hist", "tbv_ar_fini", "tbv_emu_shutdown"):
        getattr(l, name).argtypes = []; getattr(l, name).restype = None
    # emulated peer
    l.tbv_emu_stage_peer.argtypes = [vp, sz]; l.tbv_emu_stage_peer.restype = ci
    l.tbv_emu_stage_peer_repeat.argtypes = [vp, sz]; l.tbv_emu_stage_peer_repeat.restype = ci
    l.tbv_emu_peer_resident.argtypes = [vp, sz]; l.tbv_emu_peer_resident.restype = ci
    l.tbv_emu_arrival_script.argtypes = [ctypes.POINTER(ci), sz]; l.tbv_emu_arrival_script.restype = ci
    l.tbv_emu_withhold.argtypes = [ctypes.c_ulonglong, ci]; l.tbv_emu_withhold.restype = ci
    l.tbv_emu_seq.argtypes = []; l.tbv_emu_seq.restype = ctypes.c_ulonglong
    l.tbv_emu_plan.argtypes = [sz, ctypes.POINTER(sz), ctypes.POINTER(sz)]; l.tbv_emu_plan.restype = ci
    l.tbv_emu_configure.argtypes = [ctypes.c_char_p, sz]; l.tbv_emu_configure.restype = ci
    l.tbv_emu_nslot.argtypes = []; l.tbv_emu_nslot.restype = ci
    l.tbv_emu_stride.argtypes = []; l.tbv_emu_stride.restype = sz
    l.tbv_emu_send_slot.argtypes = [ci]; l.tbv_emu_send_slot.restype = vp
    l.tbv_emu_recv_slot.argtypes = [ci]; l.tbv_emu_recv_slot.restype = vp
    l.tbv_emu_arrival_log.argtypes = [up, ctypes.POINTER(ci), sz]; l.tbv_emu_arrival_log.restype = sz
    l.tbv_emu_latency_probe.argtypes = [ci]; l.tbv_emu_latency_probe.restype = ci
    l.tbv_emu_latencies.argtypes = [dp, sz]; l.tbv_emu_latencies.restype = sz
    l.tbv_emu_kernel_timing.argtypes = [ci]; l.tbv_emu_kernel_timing.restype = ci
    l.tbv_emu_kernel_times.argtypes = [ci, dp, dp]; l.tbv_emu_kernel_times.restype = sz
    l.tbv_emu_footprints.argtypes = [ctypes.POINTER(ctypes.c_ulonglong)]; l.tbv_emu_footprints.restype = None
    l.tbv_emu_tag_counts.argtypes = [up, up, up]; l.tbv_emu_tag_counts.restype = None
    l.tbv_ar_allreduce_chunked.argtypes = [vp, vp, sz, ci, vp]; l.tbv_ar_allreduce_chunked.restype = ci
    l.tbv_emu_run_pack.argtypes = [vp, sz, ci, vp]; l.tbv_emu_run_pack.restype = ci
    l.tbv_emu_run_sum.argtypes = [vp, vp, vp, sz, ci, vp]; l.tbv_emu_run_sum.restype = ci
    l.tbv_step_noalloc.argtypes = [vp, vp, vp, vp, ci, sz, ci, vp, vp, ctypes.c_ulonglong, vp]; l.tbv_step_noalloc.restype = ci
    l.tbv_emu_hbm_probe.argtypes = [ci, sz, sz, ci, dp, dp]; l.tbv_emu_hbm_probe.restype = ci
    l.tbv_emu_launch_floor.argtypes = [ci, dp]; l.tbv_emu_launch_floor.restype = ci
    return l


def load(so=_DEFAULT_SO):
    """Load and bind the shared library without initialising it (no GPU needed)."""
    if not os.path.exists(so):
        raise RuntimeError(f"{so} is missing: build it with `make -C libtbvcoll_amd/csrc` "
                           "(there is no fallback path)")
    return _bind(so)


def init(rank, devs, peer_ip, port=18995, cap_bytes=8 << 20, so=_DEFAULT_SO):
    global _lib, _cap
    if _lib is not None:
        return
    l = load(so)
    rc = l.tbv_ar_init(rank, devs.encode(), (peer_ip or "").encode(), port, cap_bytes)
    if rc != 0:
        raise RuntimeError(f"tbv_ar_init failed rc={rc}")
    _lib, _cap = l, l.tbv_ar_cap()


def all_reduce(t: torch.Tensor, out: torch.Tensor = None) -> bool:
    """SUM with the peer.  out=None means in place.  False means "not handled
    here, use your own collective" (step4/tbvcoll.py:35-58)."""
    if _lib is None or not t.is_cuda or not t.is_contiguous():
        return False
    if out is not None and (not out.is_contiguous() or out.dtype is not t.dtype or out.numel() != t.numel()):
        return False
    dt = _DT.get(t.dtype)
    if dt is None:
        return False
    nb = t.numel() * t.element_size()
    if nb == 0:
        return True
    if nb > _cap:
        return False
    # the current stream is read on every call: a cached handle goes stale when the caller switches streams
    st = torch.cuda.current_stream().cuda_stream
    rc = _lib.tbv_ar_allreduce(ctypes.c_void_p(t.data_ptr()),
                               ctypes.c_void_p(out.data_ptr()) if out is not None else None,
                               nb, dt, ctypes.c_void_p(st))
    if rc == -2:
        return False
    if rc != 0:
        raise RuntimeError(f"tbv_ar_allreduce failed rc={rc}")
    return True


def is_async():
    return bool(_lib.tbv_ar_async())


def err():
    return bool(_lib.tbv_ar_err())


def rails():
    """Dump per-rail post / arrival averages to stderr (resets them)."""
    _lib.tbv_ar_rails()


def hist():
    """Dump the transfer histogram by size to stderr (resets it)."""
    _lib.tbv_ar_hist()


def raw_fn():
    """The bound C function for hot callers: (in_ptr, out_ptr, nbytes, dtype, stream) -> rc.
    The caller checks dtype, size and contiguity itself."""
    return _lib.tbv_ar_allreduce


def cap():
    return _cap


def stats5():
    """(pre, xfer, post, enq, drain, count), microseconds per call; reading resets."""
    a, b, c, d, e = (ctypes.c_double() for _ in range(5))
    n = ctypes.c_ulonglong()
    _lib.tbv_ar_stats5(*[ctypes.byref(x) for x in (a, b, c, d, e)], ctypes.byref(n))
    return a.value, b.value, c.value, d.value, e.value, n.value


def stats4():
    """(pre_us, xfer_us, post_us, enq_us, count)."""
    a, b, c, d = (ctypes.c_double() for _ in range(4))
    n = ctypes.c_ulonglong()
    _lib.tbv_ar_stats4(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c), ctypes.byref(d), ctypes.byref(n))
    return a.value, b.value, c.value, d.value, n.value


def stats3():
    pre, xf, post, enq, n = stats4()
    return pre, xf, post, n


def stats():
    """(mean transfer us, calls); reading resets."""
    a, c = ctypes.c_double(), ctypes.c_ulonglong()
    _lib.tbv_ar_stats(ctypes.byref(a), ctypes.byref(c))
    return a.value, c.value


# ------------------------------------------------------------------ emulated peer (additive)

def lib():
    """The bound library after `init` (None before)."""
    return _lib


def _nbytes(t):
    return t.numel() * t.element_size()


def stage_peer(t: torch.Tensor):
    """Queue `t` as the peer's payload of the next call that has none.  Keep `t`
    alive until that call's result is complete."""
    assert t.is_contiguous()
    rc = _lib.tbv_emu_stage_peer(ctypes.c_void_p(t.data_ptr()), _nbytes(t))
    if rc != 0:
        raise RuntimeError(f"tbv_emu_stage_peer failed rc={rc}")


def stage_peer_repeat(t):
    if t is None:
        _lib.tbv_emu_stage_peer_repeat(None, 0)
    else:
        assert t.is_contiguous()
        _lib.tbv_emu_stage_peer_repeat(ctypes.c_void_p(t.data_ptr()), _nbytes(t))


def peer_resident(t):
    rc = _lib.tbv_emu_peer_resident(None, 0) if t is None else \
        _lib.tbv_emu_peer_resident(ctypes.c_void_p(t.data_ptr()), _nbytes(t))
    if rc != 0:
        raise RuntimeError(f"tbv_emu_peer_resident failed rc={rc}")


def arrival_script(rails_list):
    n = len(rails_list)
    arr = (ctypes.c_int * max(n, 1))(*rails_list)
    rc = _lib.tbv_emu_arrival_script(arr, n)
    if rc != 0:
        raise RuntimeError(f"tbv_emu_arrival_script failed rc={rc}")


def withhold(seq, rail=0):
    _lib.tbv_emu_withhold(seq, rail)


def seq():
    return _lib.tbv_emu_seq()


def latency_probe(on=True):
    rc = _lib.tbv_emu_latency_probe(1 if on else 0)
    if rc != 0:
        raise RuntimeError("tbv_emu_latency_probe failed")


def latencies(max_n=1 << 20):
    buf = (ctypes.c_double * max_n)()
    n = _lib.tbv_emu_latencies(buf, max_n)
    return list(buf[:n])


def arrival_log(max_n=1 << 16):
    s = (ctypes.c_ulonglong * max_n)()
    r = (ctypes.c_int * max_n)()
    n = _lib.tbv_emu_arrival_log(s, r, max_n)
    return [(s[i], r[i]) for i in range(n)]


def kernel_timing(on=True):
    _lib.tbv_emu_kernel_timing(1 if on else 0)


def kernel_times(which):
    """(count, mean_us, min_us) of the recorded pack (0) or sum (1) launches; clears them."""
    m, mn = ctypes.c_double(), ctypes.c_double()
    n = _lib.tbv_emu_kernel_times(which, ctypes.byref(m), ctypes.byref(mn))
    return n, m.value, mn.value


def hbm_probe(kind, nbytes, pool_bytes, reps, so=_DEFAULT_SO):
    """(mean_us, min_us) of a plain streaming kernel: kind 0 read, 1 write, 2 non-temporal copy, 3 plain copy."""
    l = _lib or load(so)
    m, mn = ctypes.c_double(), ctypes.c_double()
    if l.tbv_emu_hbm_probe(kind, nbytes, pool_bytes, reps, ctypes.byref(m), ctypes.byref(mn)) != 0:
        raise RuntimeError("tbv_emu_hbm_probe failed")
    return m.value, mn.value


def launch_floor(reps=2000, so=_DEFAULT_SO):
    """Launch-to-launch microseconds of an empty kernel in one stream."""
    l = _lib or load(so)
    v = ctypes.c_double()
    if l.tbv_emu_launch_floor(reps, ctypes.byref(v)) != 0:
        raise RuntimeError("tbv_emu_launch_floor failed")
    return v.value


def footprints():
    """[wait entered, wait passed, pack started, sum done, wait timed out] sequence numbers (TBV_KWAIT=1)."""
    buf = (ctypes.c_ulonglong * 5)()
    _lib.tbv_emu_footprints(buf)
    return list(buf)


def tag_counts():
    a, b, c = (ctypes.c_ulonglong() for _ in range(3))
    _lib.tbv_emu_tag_counts(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return a.value, b.value, c.value


def all_reduce_chunked(t: torch.Tensor, out: torch.Tensor = None) -> bool:
    """Pipelined SUM of a tensor of any size as cap-sized chunks."""
    if _lib is None or not t.is_cuda or not t.is_contiguous():
        return False
    if out is not None and (not out.is_contiguous() or out.dtype is not t.dtype or out.numel() != t.numel()):
        return False
    dt = _DT.get(t.dtype)
    if dt is None:
        return False
    st = torch.cuda.current_stream().cuda_stream
    rc = _lib.tbv_ar_allreduce_chunked(ctypes.c_void_p(t.data_ptr()),
                                       ctypes.c_void_p(out.data_ptr()) if out is not None else None,
                                       _nbytes(t), dt, ctypes.c_void_p(st))
    if rc != 0:
        raise RuntimeError(f"tbv_ar_allreduce_chunked failed rc={rc}")
    return True


def shutdown():
    """Tear the library down so that `init` can run again with other settings."""
    global _lib, _cap
    if _lib is not None:
        _lib.tbv_emu_shutdown()
    _lib, _cap = None, 0
