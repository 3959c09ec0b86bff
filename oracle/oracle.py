"""ctypes face of the CPU oracle (oracle/tbv_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
bench's cpu_baseline leg.  The shipped package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None
_hdr = None

DT_F32, DT_F16, DT_BF16 = 0, 1, 2          # step4/libtbvcoll.cpp:416
_NP = {DT_F32: np.float32, DT_F16: np.uint16, DT_BF16: np.uint16}


def build(force=False):
    """(Re)build liborc.so / libhiphdr.so with the Makefile beside this file."""
    args = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        so = os.path.join(_HERE, "liborc.so")
        if not os.path.exists(so):
            build()
        l = ctypes.CDLL(so)
        vp, sz, u64, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_int
        l.orc_sum.argtypes = [ci, vp, vp, vp, sz]; l.orc_sum.restype = ci
        l.orc_pack.argtypes = [vp, vp, sz, ci, u64]; l.orc_pack.restype = None
        l.orc_tag_offset.argtypes = [sz]; l.orc_tag_offset.restype = sz
        l.orc_cap_round.argtypes = [sz]; l.orc_cap_round.restype = sz
        l.orc_stride.argtypes = [sz, ci]; l.orc_stride.restype = sz
        l.orc_xbytes.argtypes = [sz, ci]; l.orc_xbytes.restype = sz
        l.orc_rails_for.argtypes = [sz, sz, ci]; l.orc_rails_for.restype = ci
        l.orc_slot.argtypes = [u64, ci]; l.orc_slot.restype = ci
        l.orc_nslot_clamp.argtypes = [ci]; l.orc_nslot_clamp.restype = ci
        l.orc_fragment.argtypes = [sz, ci, ci, ctypes.POINTER(sz), ctypes.POINTER(sz)]; l.orc_fragment.restype = ci
        l.orc_wr_hwm.argtypes = [ci, sz, sz]; l.orc_wr_hwm.restype = ci
        l.orc_pack_grid.argtypes = [sz]; l.orc_pack_grid.restype = ci
        l.orc_sum_grid.argtypes = [sz]; l.orc_sum_grid.restype = ci
        l.orc_hist_bucket.argtypes = [sz]; l.orc_hist_bucket.restype = ci
        l.orc_sum1_bf16.argtypes = [ctypes.c_uint16, ctypes.c_uint16]; l.orc_sum1_bf16.restype = ctypes.c_uint16
        l.orc_sum1_f16.argtypes = [ctypes.c_uint16, ctypes.c_uint16]; l.orc_sum1_f16.restype = ctypes.c_uint16
        l.orc_f32bits_to_bf16.argtypes = [ctypes.c_uint32]; l.orc_f32bits_to_bf16.restype = ctypes.c_uint16
        l.orc_f32bits_to_f16.argtypes = [ctypes.c_uint32]; l.orc_f32bits_to_f16.restype = ctypes.c_uint16
        l.orc_f16_to_f32bits.argtypes = [ctypes.c_uint16]; l.orc_f16_to_f32bits.restype = ctypes.c_uint32
        l.orc_bf16_to_f32bits.argtypes = [ctypes.c_uint16]; l.orc_bf16_to_f32bits.restype = ctypes.c_uint32
        l.orc_ring_model.argtypes = [ctypes.POINTER(sz), sz, ctypes.POINTER(ci), sz, ci, ci, sz, ci,
                                     ctypes.POINTER(u64), ctypes.POINTER(ci), ctypes.POINTER(ci)]
        l.orc_ring_model.restype = ctypes.c_long
        l.orc_ring_model2.argtypes = [ctypes.POINTER(sz), sz, ctypes.POINTER(ci), sz, ci, ci, sz, ci, ci,
                                      ctypes.POINTER(u64), ctypes.POINTER(ci), ctypes.POINTER(ci), ctypes.POINTER(ctypes.c_long)]
        l.orc_ring_model2.restype = ctypes.c_long
        l.orc_rmsnorm_rows.argtypes = [ci, vp, vp, vp, sz, sz, ctypes.c_float]; l.orc_rmsnorm_rows.restype = ci
        l.orc_sum_rmsnorm.argtypes = [ci, vp, vp, vp, vp, vp, sz, sz, ctypes.c_float]; l.orc_sum_rmsnorm.restype = ci
        l.orc_q8_image_bytes.argtypes = [sz]; l.orc_q8_image_bytes.restype = sz
        l.orc_q8_encode.argtypes = [ci, vp, sz, vp]; l.orc_q8_encode.restype = ci
        l.orc_q8_decode.argtypes = [vp, sz, vp]; l.orc_q8_decode.restype = None
        l.orc_q8_sum.argtypes = [ci, vp, vp, sz, vp]; l.orc_q8_sum.restype = ci
        l.orc_reduce_copy.argtypes = [ci, vp, vp, vp, vp, sz, ci]; l.orc_reduce_copy.restype = ci
        l.orc_time_reduce_copy.argtypes = [ci, vp, vp, vp, vp, sz, ci, ci, ci]; l.orc_time_reduce_copy.restype = ctypes.c_double
        _lib = l
    return _lib


def hdr():
    """Host build of the HIP headers' operator+ (third-party arithmetic)."""
    global _hdr
    if _hdr is None:
        so = os.path.join(_HERE, "libhiphdr.so")
        if not os.path.exists(so):
            build()
        l = ctypes.CDLL(so)
        for f in (l.hdr_sum_bf16, l.hdr_sum_f16):
            f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
            f.restype = None
        _hdr = l
    return _hdr


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def sum_bits(dtype, a, b):
    """Element-wise reference sum.  a, b: contiguous numpy arrays holding the raw
    storage (float32 for dtype 0, uint16 bit patterns for fp16/bf16)."""
    a = np.ascontiguousarray(a, dtype=_NP[dtype]); b = np.ascontiguousarray(b, dtype=_NP[dtype])
    assert a.shape == b.shape
    out = np.empty_like(a)
    rc = lib().orc_sum(dtype, _p(a), _p(b), _p(out), a.size)
    assert rc == 0
    return out


def pack(src_bytes, tag=False, seq=0, slot_bytes=None):
    """Bounce-slot image after the pack copy: payload bytes, then (tag) the 64-bit seq at align8(n)."""
    src = np.ascontiguousarray(src_bytes, dtype=np.uint8)
    n = src.size
    need = int(lib().orc_tag_offset(n)) + 8 if tag else n
    dst = np.zeros(slot_bytes if slot_bytes is not None else need, dtype=np.uint8)
    lib().orc_pack(_p(dst), _p(src), n, int(bool(tag)), seq)
    return dst


def fragment(xbytes, R, idx):
    off, ln = ctypes.c_size_t(), ctypes.c_size_t()
    ok = lib().orc_fragment(xbytes, R, idx, ctypes.byref(off), ctypes.byref(ln))
    return (off.value, ln.value) if ok else None


def ring_model(call_nbytes, script, nslot, nrails, rail1max=98304, depth=1):
    n, m = len(call_nbytes), len(script)
    calls = (ctypes.c_size_t * max(n, 1))(*call_nbytes)
    scr = (ctypes.c_int * max(m, 1))(*script)
    rel = (ctypes.c_uint64 * max(m, 1))()
    slots = (ctypes.c_int * max(n, 1))()
    rails = (ctypes.c_int * max(n, 1))()
    k = lib().orc_ring_model(calls, n, scr, m, nslot, nrails, rail1max, depth, rel, slots, rails)
    return k, list(rel)[:max(k, 0)], list(slots)[:n], list(rails)[:n]


def ring_model2(call_nbytes, script, nslot, nrails, rail1max=98304, depth=1, slot_guard=1):
    """As ring_model, with the caller optionally holding a call back until its slot's previous user has
    been released; also returns how many calls were issued into a slot still owned by an unreleased call."""
    n, m = len(call_nbytes), len(script)
    calls = (ctypes.c_size_t * max(n, 1))(*call_nbytes)
    scr = (ctypes.c_int * max(m, 1))(*script)
    rel = (ctypes.c_uint64 * max(m, 1))()
    slots = (ctypes.c_int * max(n, 1))()
    rails = (ctypes.c_int * max(n, 1))()
    shared = ctypes.c_long(0)
    k = lib().orc_ring_model2(calls, n, scr, m, nslot, nrails, rail1max, depth, slot_guard, rel, slots, rails, ctypes.byref(shared))
    return k, list(rel)[:max(k, 0)], list(slots)[:n], list(rails)[:n], shared.value


def rmsnorm_rows(dtype, x, w, hidden, eps):
    """normed = T(float(x) * s) * w per row of `hidden` elements, s = 1/sqrt(mean(x^2) + eps); storage-bit arrays."""
    x = np.ascontiguousarray(x, dtype=_NP[dtype]).reshape(-1); w = np.ascontiguousarray(w, dtype=_NP[dtype]).reshape(-1)
    assert w.size == hidden and x.size % hidden == 0
    out = np.empty_like(x)
    rc = lib().orc_rmsnorm_rows(dtype, _p(x), _p(w), _p(out), x.size // hidden, hidden, eps)
    assert rc == 0
    return out


def sum_rmsnorm(dtype, a, b, w, hidden, eps):
    """(out, normed) of the fused step: out = a + b in the storage type, normed = rmsnorm(out) * w."""
    a = np.ascontiguousarray(a, dtype=_NP[dtype]).reshape(-1); b = np.ascontiguousarray(b, dtype=_NP[dtype]).reshape(-1)
    w = np.ascontiguousarray(w, dtype=_NP[dtype]).reshape(-1)
    assert a.size == b.size and w.size == hidden and a.size % hidden == 0
    out = np.empty_like(a); normed = np.empty_like(a)
    rc = lib().orc_sum_rmsnorm(dtype, _p(a), _p(b), _p(w), _p(out), _p(normed), a.size // hidden, hidden, eps)
    assert rc == 0
    return out, normed


def q8_encode(dtype, x):
    """int8 codec image (uint8 array) of the storage-bit array x."""
    x = np.ascontiguousarray(x, dtype=_NP[dtype]).reshape(-1)
    img = np.zeros(int(lib().orc_q8_image_bytes(x.size)), dtype=np.uint8)
    assert lib().orc_q8_encode(dtype, _p(x), x.size, _p(img)) == 0
    return img


def q8_decode(img, n):
    out = np.empty(n, dtype=np.float32)
    lib().orc_q8_decode(_p(np.ascontiguousarray(img, dtype=np.uint8)), n, _p(out))
    return out


def q8_sum(dtype, own_img, recv_img, n):
    """out = T(decode(own) + decode(received)) as storage bits."""
    out = np.empty(n, dtype=_NP[dtype])
    assert lib().orc_q8_sum(dtype, _p(np.ascontiguousarray(own_img, dtype=np.uint8)), _p(np.ascontiguousarray(recv_img, dtype=np.uint8)), n, _p(out)) == 0
    return out


def reduce_copy(dtype, local, peer, nthreads=1):
    """One whole step on the host: returns (bounce image, out)."""
    local = np.ascontiguousarray(local); peer = np.ascontiguousarray(peer)
    bounce = np.empty_like(local); out = np.empty_like(local)
    rc = lib().orc_reduce_copy(dtype, _p(local), _p(peer), _p(bounce), _p(out), local.nbytes, nthreads)
    assert rc == 0
    return bounce, out


def time_reduce_copy(dtype, local, peer, nthreads, warm, reps):
    """Median seconds per whole step (pack + sum) on `nthreads` host threads."""
    local = np.ascontiguousarray(local); peer = np.ascontiguousarray(peer)
    bounce = np.empty_like(local); out = np.empty_like(local)
    return lib().orc_time_reduce_copy(dtype, _p(local), _p(peer), _p(bounce), _p(out), local.nbytes,
                                      nthreads, warm, reps)


# ---- numpy views of torch tensors' storage bits (helpers for tests) -----------------------

def torch_bits(t):
    """Raw storage of a CPU torch tensor as numpy (uint16 for half types, float32 otherwise)."""
    import torch
    t = t.detach().contiguous().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def torch_dtype_code(dt):
    import torch
    return {torch.float32: DT_F32, torch.float16: DT_F16, torch.bfloat16: DT_BF16}[dt]


def sum_torch(a, b):
    """Oracle sum of two torch tensors (any device); returns a CPU tensor of the same dtype."""
    import torch
    code = torch_dtype_code(a.dtype)
    o = sum_bits(code, torch_bits(a).reshape(-1), torch_bits(b).reshape(-1))
    if code == DT_F32:
        return torch.from_numpy(o).reshape(a.shape)
    return torch.from_numpy(o.view(np.int16)).view(a.dtype).reshape(a.shape)
