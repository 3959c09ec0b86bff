"""Seeded synthetic tensors for the all-reduce data path.

The reference's tests draw inputs from torch's CUDA generator at run time
(step4/test_exact.py:15-17, step4/test_stress.py:17-19), which is not
reproducible without that GPU.  This module is a counter-based generator:
element i of stream (seed, lane) is a pure integer hash of (seed, lane, i), so
any host produces the same values, any slice can be produced alone, and both
"ranks" can regenerate each other's input, which is the trick those tests rely on.

All integer work is done on 64-bit words holding 32-bit values, products of two
32-bit values never wrap, so the same code runs on numpy arrays and (through
`torch_hash_uniform`) on int64 torch tensors on the GPU.
"""
import numpy as np

_M32 = np.uint64(0xFFFFFFFF)


def _mix32(x):
    """Bijective avalanche mix of 32-bit values held in uint64 words."""
    x = x ^ (x >> np.uint64(16))
    x = (x * np.uint64(0x7FEB352D)) & _M32
    x = x ^ (x >> np.uint64(15))
    x = (x * np.uint64(0x846CA68B)) & _M32
    x = x ^ (x >> np.uint64(16))
    return x


def _key(seed, lane):
    k = np.array([(int(seed) * 0x9E3779B1 + int(lane) * 0x85EBCA77 + 0x165667B1) & 0xFFFFFFFF], dtype=np.uint64)
    return _mix32(_mix32(k) ^ np.uint64((int(seed) >> 32) & 0xFFFFFFFF))[0]


def bits32(seed, n, lane=0, start=0):
    """n 32-bit words of stream (seed, lane) starting at counter `start`, as uint64."""
    i = np.arange(start, start + n, dtype=np.uint64)
    lo = i & _M32
    hi = i >> np.uint64(32)
    k = _key(seed, lane)
    return _mix32(((_mix32(lo ^ k) + hi) & _M32) ^ (k >> np.uint64(7)))


def uniform01(seed, n, lane=0, start=0):
    """float64 in [0,1) with 24 random bits (exactly representable in fp32)."""
    return (bits32(seed, n, lane, start) >> np.uint64(8)).astype(np.float64) * (1.0 / 16777216.0)


def uniform(seed, n, lo=-4.0, hi=4.0, start=0):
    """fp32 U[lo,hi): lo + (hi-lo)*u computed in fp64 then rounded once to fp32."""
    return (lo + (hi - lo) * uniform01(seed, n, 0, start)).astype(np.float32)


def normal(seed, n, std=1.0, start=0):
    """fp32 N(0,std^2) by Box-Muller on two independent lanes."""
    u1 = uniform01(seed, n, 1, start)
    u2 = uniform01(seed, n, 2, start)
    r = np.sqrt(-2.0 * np.log1p(-u1))            # 1-u1 in (0,1]
    z = r * np.cos(2.0 * np.pi * u2)
    return (z * std).astype(np.float32)


def prefill_activations(seed, n, std=0.02, outlier_frac=0.001, outlier_mag=8.0, start=0):
    """fp32 N(0,std^2) with a fraction of elements replaced by +-outlier_mag
    (the 16 MB prefill workload: narrow activations with rare large channels)."""
    x = normal(seed, n, std, start)
    sel = bits32(seed, n, 3, start)
    thresh = np.uint64(int(outlier_frac * 4294967296.0))
    mask = sel < thresh
    sign = np.where((bits32(seed, n, 4, start) & np.uint64(1)) == 0, 1.0, -1.0).astype(np.float32)
    x[mask] = (sign * np.float32(outlier_mag))[mask]
    return x


def arrival_script(seed, ncalls, nrails, depth, rails_per_call=None):
    """Seeded random arrival order for a pipelined, multi-rail sequence of calls.

    Returns a list of rail ids; each rail consumes its own occurrences in FIFO
    order (a rail's queue is a FIFO, step4/libtbvcoll.cpp:249,273).  The order is
    a random linear extension of the protocol's partial order: call c's fragment
    on rail r may arrive only after call c-1's fragment on rail r, and only after
    every fragment of call c-depth has arrived (call c is packed on the caller's
    stream after call c-depth's sum).
    """
    if rails_per_call is None:
        rails_per_call = [nrails] * ncalls
    rnd = bits32(seed, ncalls * nrails * 2 + 8, 5)
    nxt = [0] * nrails                      # per rail: index into its own call list
    per_rail_calls = [[c for c in range(ncalls) if r < rails_per_call[c]] for r in range(nrails)]
    arrived = [0] * ncalls                  # fragments arrived per call
    out, k, done_prefix = [], 0, 0
    total = sum(rails_per_call)
    while len(out) < total:
        ready = []
        for r in range(nrails):
            if nxt[r] < len(per_rail_calls[r]):
                c = per_rail_calls[r][nxt[r]]
                if c < done_prefix + depth:
                    ready.append(r)
        if not ready:
            raise RuntimeError("arrival_script: no fragment is ready (depth too small?)")
        r = ready[int(rnd[k]) % len(ready)]
        k += 1
        c = per_rail_calls[r][nxt[r]]
        arrived[c] += 1
        while done_prefix < ncalls and arrived[done_prefix] == rails_per_call[done_prefix]:
            done_prefix += 1
        nxt[r] += 1
        out.append(r)
    return out


def torch_hash_uniform(seed, n, lo=-4.0, hi=4.0, device="cuda"):
    """Same values as `uniform(seed, n, lo, hi)`, generated on `device` with int64
    torch ops (for the stress mix, where host generation of 16 MB tensors per
    call would dominate the run)."""
    import torch
    M = 0xFFFFFFFF

    def mix(x):
        x = x ^ (x >> 16)
        x = (x * 0x7FEB352D) & M
        x = x ^ (x >> 15)
        x = (x * 0x846CA68B) & M
        x = x ^ (x >> 16)
        return x

    k = int(_key(seed, 0))
    i = torch.arange(n, dtype=torch.int64, device=device)
    lo32 = i & M
    hi32 = i >> 32
    h = mix(((mix(lo32 ^ k) + hi32) & M) ^ (k >> 7))
    u = (h >> 8).to(torch.float64) * (1.0 / 16777216.0)
    return (lo + (hi - lo) * u).to(torch.float32)
