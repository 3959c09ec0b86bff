"""tbvcoll -- ctypes binding of libtbvcoll.so (MI355X build).

The module keeps the surface of the reference binding (step4/tbvcoll.py:14-111): `init`,
`all_reduce`, `is_async`, `err`, `rails`, `hist`, `raw_fn`, `cap`, `stats`, `stats3`,
`stats4`, `stats5`, with the same guards and return conventions, so a caller written
against the reference (a vLLM `GroupCoordinator.all_reduce` intercept, code that uses the
C function through `raw_fn`) binds without changes.  On one GPU the peer is emulated: a
two-rank exact/stress driver additionally has to hand over the peer's payload with
`stage_peer` before each call (without one the peer echoes this rank's own payload).

    import tbvcoll
    tbvcoll.init(rank, "rail0,rail1", "", cap_bytes=8 << 20)
    tbvcoll.stage_peer(peer_tensor)    # this build only: what the other rank would have sent
    tbvcoll.all_reduce(t)              # in-place SUM; False -> caller falls back

Additions (no counterpart in the reference): the emulated peer (`stage_peer`,
`stage_peer_repeat`, `peer_resident`, `arrival_script`, `hold_rail`, `withhold`,
`arrival_log`), measurement (`latency_probe`, `latencies`, `kernel_timing`, `kernel_times`,
`hbm_probe`, `launch_floor`), `all_reduce_chunked`, `shutdown`, `lib`.

There is no CPU fallback: if the shared library is missing, `init` raises.
"""
import ctypes
import os

import torch

_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
_lib = None
_cap = 0
_DEFAULT_SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtbvcoll.so")

_VP, _SZ, _I, _U64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_ulonglong
_PD, _PU, _PI, _PSZ = (ctypes.POINTER(t) for t in (ctypes.c_double, ctypes.c_ulonglong, ctypes.c_int, ctypes.c_size_t))

# symbol -> (restype, argtypes): everything include/tbvcoll.h and include/tbvcoll_emu.h declare
_SIGNATURES = {
    "tbv_ar_init": (_I, [_I, ctypes.c_char_p, ctypes.c_char_p, _I, _SZ]),
    "tbv_ar_allreduce": (_I, [_VP, _VP, _SZ, _I, _VP]),
    "tbv_ar_stats": (None, [_PD, _PU]),
    "tbv_ar_stats4": (None, [_PD] * 4 + [_PU]),
    "tbv_ar_stats5": (None, [_PD] * 5 + [_PU]),
    "tbv_ar_cap": (_I, []), "tbv_ar_async": (_I, []), "tbv_ar_err": (_I, []),
    "tbv_ar_rails": (None, []), "tbv_ar_hist": (None, []), "tbv_ar_fini": (None, []),
    "tbv_emu_shutdown": (None, []),
    "tbv_emu_stage_peer": (_I, [_VP, _SZ]), "tbv_emu_stage_peer_repeat": (_I, [_VP, _SZ]), "tbv_emu_peer_resident": (_I, [_VP, _SZ]),
    "tbv_emu_arrival_script": (_I, [_PI, _SZ]), "tbv_emu_withhold": (_I, [_U64, _I]), "tbv_emu_hold_rail": (_I, [_I, _I]),
    "tbv_emu_seq": (_U64, []), "tbv_emu_plan": (_I, [_SZ, _PSZ, _PSZ]), "tbv_emu_configure": (_I, [ctypes.c_char_p, _SZ]),
    "tbv_emu_rendezvous": (_I, [_I, ctypes.c_char_p, _I, ctypes.c_double]),
    "tbv_emu_nslot": (_I, []), "tbv_emu_stride": (_SZ, []), "tbv_emu_send_slot": (_VP, [_I]), "tbv_emu_recv_slot": (_VP, [_I]),
    "tbv_emu_arrival_log": (_SZ, [_PU, _PI, _SZ]),
    "tbv_emu_latency_probe": (_I, [_I]), "tbv_emu_latencies": (_SZ, [_PD, _SZ]),
    "tbv_emu_kernel_timing": (_I, [_I]), "tbv_emu_kernel_times": (_SZ, [_I, _PD, _PD]),
    "tbv_emu_kernel_timeline": (_SZ, [_I, _PD, _PD, _SZ]),
    "tbv_emu_footprints": (None, [_PU]), "tbv_emu_tag_counts": (None, [_PU, _PU, _PU]),
    "tbv_ar_allreduce_chunked": (_I, [_VP, _VP, _SZ, _I, _VP]),
    "tbv_emu_run_pack": (_I, [_VP, _SZ, _I, _VP]), "tbv_emu_run_sum": (_I, [_VP, _VP, _VP, _SZ, _I, _VP]),
    "tbv_step_noalloc": (_I, [_VP, _VP, _VP, _VP, _I, _SZ, _I, _VP, _VP, _U64, _VP]),
    "tbv_emu_hbm_probe": (_I, [_I, _SZ, _SZ, _I, _PD, _PD]), "tbv_emu_launch_floor": (_I, [_I, _PD]),
    "tbv_emu_step_floor": (_I, [_SZ, _I, _PD]),
    "tbv_ar_allreduce_rmsnorm": (_I, [_VP, _VP, _VP, _VP, ctypes.c_float, _SZ, _SZ, _I, _VP]),
    "tbv_emu_run_sum_norm": (_I, [_I, _VP, _VP, _VP, _VP, _VP, ctypes.c_float, _SZ, _SZ, _I, _VP]),
    "tbv_emu_codec_image_bytes": (_SZ, [_SZ, _I]),
    "tbv_emu_run_quant": (_I, [_VP, _VP, _SZ, _I, _VP]), "tbv_emu_run_sum_quant": (_I, [_VP, _VP, _VP, _SZ, _I, _VP]),
}


def _bind(so):
    l = ctypes.CDLL(so)
    for name, (res, args) in _SIGNATURES.items():
        f = getattr(l, name)                   # AttributeError names the missing symbol
        f.restype, f.argtypes = res, args
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


def _call_args(t, out):
    """(in_ptr, out_ptr, nbytes, dtype code) of a tensor pair the library can take, or None: not initialised,
    not on the GPU, not contiguous, mismatched output, unsupported dtype (the guards of step4/tbvcoll.py:38-47)."""
    if _lib is None or not t.is_cuda or not t.is_contiguous():
        return None
    if out is not None and (not out.is_contiguous() or out.dtype is not t.dtype or out.numel() != t.numel()):
        return None
    code = _DT.get(t.dtype)
    if code is None:
        return None
    return _VP(t.data_ptr()), (_VP(out.data_ptr()) if out is not None else None), t.numel() * t.element_size(), code


def _stream():
    # read on every call: a cached handle goes stale when the caller switches streams
    return _VP(torch.cuda.current_stream().cuda_stream)


def all_reduce(t: torch.Tensor, out: torch.Tensor = None) -> bool:
    """SUM with the peer.  out=None means in place.  False means "not handled
    here, use your own collective" (step4/tbvcoll.py:35-58)."""
    a = _call_args(t, out)
    if a is None:
        return False
    pin, pout, nb, code = a
    if nb == 0:
        return True
    if nb > _cap:
        return False
    rc = _lib.tbv_ar_allreduce(pin, pout, nb, code, _stream())
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


def _read_stats(fn, ndoubles):
    vals = [ctypes.c_double() for _ in range(ndoubles)]
    n = ctypes.c_ulonglong()
    fn(*[ctypes.byref(v) for v in vals], ctypes.byref(n))
    return tuple(v.value for v in vals) + (n.value,)


def stats5():
    """(pre, xfer, post, enq, drain, count), microseconds per call; reading resets."""
    return _read_stats(_lib.tbv_ar_stats5, 5)


def stats4():
    """(pre_us, xfer_us, post_us, enq_us, count)."""
    return _read_stats(_lib.tbv_ar_stats4, 4)


def stats3():
    pre, xf, post, _, n = stats4()
    return pre, xf, post, n


def stats():
    """(mean transfer us, calls); reading resets."""
    return _read_stats(_lib.tbv_ar_stats, 1)


# ------------------------------------------------------------------ emulated peer (additive)

def lib():
    """The bound library after `init` (None before)."""
    return _lib


def _nbytes(t):
    return t.numel() * t.element_size()


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed rc={rc}")


def stage_peer(t: torch.Tensor):
    """Queue `t` as the peer's payload of the next call that has none.  Keep `t`
    alive until that call's result is complete."""
    assert t.is_contiguous()
    _check(_lib.tbv_emu_stage_peer(_VP(t.data_ptr()), _nbytes(t)), "tbv_emu_stage_peer")


def stage_peer_repeat(t):
    if t is None:
        _lib.tbv_emu_stage_peer_repeat(None, 0)
    else:
        assert t.is_contiguous()
        _lib.tbv_emu_stage_peer_repeat(_VP(t.data_ptr()), _nbytes(t))


def peer_resident(t):
    _check(_lib.tbv_emu_peer_resident(None, 0) if t is None else _lib.tbv_emu_peer_resident(_VP(t.data_ptr()), _nbytes(t)),
           "tbv_emu_peer_resident")


def arrival_script(rails_list):
    n = len(rails_list)
    _check(_lib.tbv_emu_arrival_script((ctypes.c_int * max(n, 1))(*rails_list), n), "tbv_emu_arrival_script")


def withhold(seq, rail=0):
    _lib.tbv_emu_withhold(seq, rail)


def hold_rail(rail, hold=True):
    _check(_lib.tbv_emu_hold_rail(rail, 1 if hold else 0), "tbv_emu_hold_rail")


def seq():
    return _lib.tbv_emu_seq()


def latency_probe(on=True):
    _check(_lib.tbv_emu_latency_probe(1 if on else 0), "tbv_emu_latency_probe")


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


def kernel_timeline(which, max_n=4096):
    """[(start_us, stop_us)] of the recorded launches, relative to the start of the first; keeps the samples."""
    a, b = (ctypes.c_double * max_n)(), (ctypes.c_double * max_n)()
    n = _lib.tbv_emu_kernel_timeline(which, a, b, max_n)
    return [(a[i], b[i]) for i in range(n)]


def hbm_probe(kind, nbytes, pool_bytes, reps, so=_DEFAULT_SO):
    """(mean_us, min_us) of a plain streaming kernel: kind 0 read, 1 write, 2 non-temporal copy, 3 plain copy."""
    l = _lib or load(so)
    m, mn = ctypes.c_double(), ctypes.c_double()
    _check(l.tbv_emu_hbm_probe(kind, nbytes, pool_bytes, reps, ctypes.byref(m), ctypes.byref(mn)), "tbv_emu_hbm_probe")
    return m.value, mn.value


def launch_floor(reps=2000, so=_DEFAULT_SO):
    """Launch-to-launch microseconds of an empty kernel in one stream."""
    l = _lib or load(so)
    v = ctypes.c_double()
    _check(l.tbv_emu_launch_floor(reps, ctypes.byref(v)), "tbv_emu_launch_floor")
    return v.value


def step_floor(nbytes, reps=480, so=_DEFAULT_SO):
    """Microseconds per launch of a kernel that only moves the four streams of one bf16 step of `nbytes`
    (no counting, no signal, no gate) over rotating cache-cold buffers: the floor under every form of the step."""
    l = _lib or load(so)
    v = ctypes.c_double()
    _check(l.tbv_emu_step_floor(nbytes, reps, ctypes.byref(v)), "tbv_emu_step_floor")
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
    a = _call_args(t, out)
    if a is None:
        return False
    pin, pout, nb, code = a
    _check(_lib.tbv_ar_allreduce_chunked(pin, pout, nb, code, _stream()), "tbv_ar_allreduce_chunked")
    return True


def all_reduce_rmsnorm(t: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor = None, normed: torch.Tensor = None):
    """SUM with the peer fused with the RMSNorm of the result over the last dimension:
    out = t + peer (in place when out is None), normed = rmsnorm(out) * weight.  Returns `normed`
    (allocated when not given), or None when the library does not take the call (not initialised,
    unsupported layout, over the cap): the caller then runs its own all-reduce and norm."""
    a = _call_args(t, out)
    if a is None or t.dim() < 1 or weight.dtype is not t.dtype or not weight.is_contiguous() or weight.numel() != t.shape[-1]:
        return None
    pin, pout, nb, code = a
    if nb == 0 or nb > _cap:
        return None
    hidden = t.shape[-1]
    # what the row kernel takes: rows of whole 16-byte vectors, at most 64 KiB each, every buffer 16-byte aligned.
    # Anything else is declined here (the caller falls back) rather than turned into an error by the library.
    row_bytes = hidden * t.element_size()
    if row_bytes % 16 or row_bytes > 65536:
        return None
    if normed is not None and (not normed.is_contiguous() or normed.dtype is not t.dtype or normed.numel() != t.numel()):
        return None
    ptrs = [t.data_ptr(), weight.data_ptr()] + [x.data_ptr() for x in (out, normed) if x is not None]
    if any(p % 16 for p in ptrs):
        return None
    if normed is None:
        normed = torch.empty_like(t)
    rc = _lib.tbv_ar_allreduce_rmsnorm(pin, pout, _VP(normed.data_ptr()), _VP(weight.data_ptr()), eps,
                                       t.numel() // hidden, hidden, code, _stream())
    if rc == -2:
        return None
    _check(rc, "tbv_ar_allreduce_rmsnorm")
    return normed


def shutdown():
    """Tear the library down so that `init` can run again with other settings."""
    global _lib, _cap
    if _lib is not None:
        _lib.tbv_emu_shutdown()
    _lib, _cap = None, 0
