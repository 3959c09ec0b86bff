#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/.  Run from the repo root:

    python tests/golden/make_golden.py

The reference holds no stored vectors for this path (its tests regenerate inputs
from torch's CUDA generator at run time, step4/test_exact.py:15-17), so these
fixtures are produced here, WITHOUT the oracle:
  * inputs come from the package's counter-based generator;
  * expected sums come from torch's CPU add in the storage dtype (the same
    check the reference makes, step4/test_exact.py:31), and for the 16-bit types
    are cross-checked in this script against an exact rational brute force
    (tests/exact_round.py); the script refuses to write on any disagreement;
  * ring traces come from the small event simulation in this file, written
    from the protocol description (slot = seq % NSLOT, per-rail FIFO queues,
    last-arriving rail releases), not from the oracle's model.
"""
import os
import sys
from collections import deque

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from libtbvcoll_amd import synth          # noqa: E402
from exact_round import Format            # noqa: E402

TD = {"bf16": torch.bfloat16, "f16": torch.float16}


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def from_bits(b, name):
    return torch.from_numpy(b.view(np.int16).copy()).view(TD[name])


def check_exact(name, a, b, o):
    fmt = Format(name)
    for x, y, z in zip(a.tolist(), b.tolist(), o.tolist()):
        want = fmt.add(x, y)
        if want is None:
            assert fmt.is_nan(z), (name, hex(x), hex(y), hex(z))
        else:
            assert want == z, (name, hex(x), hex(y), hex(z), hex(want))


def config1():
    """Two bf16 vectors of 4096 elements, N(0,1), seeds 0 and 1."""
    a = torch.from_numpy(synth.normal(0, 4096)).to(torch.bfloat16)
    b = torch.from_numpy(synth.normal(1, 4096)).to(torch.bfloat16)
    o = a + b
    ab, bb, ob = bits(a), bits(b), bits(o)
    check_exact("bf16", ab, bb, ob)
    o32 = (a.float() + b.float()).to(torch.bfloat16)
    assert torch.equal(o, o32)
    np.savez(os.path.join(HERE, "c1_bf16_4096.npz"), a=ab, b=bb, out=ob)


SPECIAL = {
    # zeros, smallest/largest subnormals, smallest normal, ones, ties, max finite, inf
    "bf16": [0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x807F, 0x0080, 0x8080, 0x0081, 0x3F80, 0xBF80, 0x3F81,
             0x3B80, 0x3C00, 0x4000, 0x4049, 0x4300, 0x4301, 0x7F7F, 0xFF7F, 0x7F00, 0x7EFF, 0x7F80, 0xFF80,
             0x3380, 0x3400, 0xB400, 0x3F00, 0x3E80, 0x0100, 0x8100, 0x00FF],
    "f16": [0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x83FF, 0x0400, 0x8400, 0x0401, 0x3C00, 0xBC00, 0x3C01,
            0x1400, 0x1000, 0x4000, 0x4248, 0x5BFF, 0x5C00, 0x7BFF, 0xFBFF, 0x7800, 0x77FF, 0x7C00, 0xFC00,
            0x1001, 0x0C00, 0x8C00, 0x3800, 0x3400, 0x0800, 0x8800, 0x07FF],
}


def edge_cases(name):
    """Curated specials crossed with each other, plus seeded random bit patterns
    (finite ones only for the random part).  NaN results are left out: their
    payload is not pinned."""
    fmt = Format(name)
    sp = SPECIAL[name]
    a = [x for x in sp for _ in sp]
    b = [y for _ in sp for y in sp]
    r = synth.bits32(99 if name == "bf16" else 98, 2048, 6)
    ra = (r & np.uint64(0xFFFF)).astype(np.uint16)
    rb = ((r >> np.uint64(16)) & np.uint64(0xFFFF)).astype(np.uint16)
    keep = np.array([not (fmt.is_nan(int(x)) or fmt.is_nan(int(y)) or fmt.is_inf(int(x)) or fmt.is_inf(int(y)))
                     for x, y in zip(ra, rb)])
    a = np.array(a + ra[keep][:1000].tolist(), dtype=np.uint16)
    b = np.array(b + rb[keep][:1000].tolist(), dtype=np.uint16)
    o = bits(from_bits(a, name) + from_bits(b, name))
    nan = np.array([fmt.add(int(x), int(y)) is None for x, y in zip(a, b)])
    a, b, o = a[~nan], b[~nan], o[~nan]
    check_exact(name, a, b, o)
    np.savez(os.path.join(HERE, f"edge_{name}.npz"), a=a, b=b, out=o)


def edge_f32():
    sp = np.array([0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x007FFFFF, 0x00800000, 0x3F800000, 0xBF800000,
                   0x3F800001, 0x33800000, 0x34000000, 0x4B800000, 0x4B800001, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F000000,
                   0x7F800000, 0xFF800000, 0x00400000, 0x80400000], dtype=np.uint32)
    a = np.repeat(sp, len(sp)); b = np.tile(sp, len(sp))
    r = synth.bits32(97, 4096, 6).astype(np.uint32)
    ra, rb = r[:2048], r[2048:]
    fin = ((ra & 0x7F800000) != 0x7F800000) & ((rb & 0x7F800000) != 0x7F800000)
    a = np.concatenate([a, ra[fin][:1000]]); b = np.concatenate([b, rb[fin][:1000]])
    # expected via exact arithmetic: float64 holds any fp32+fp32 sum exactly unless exponents differ by > 29,
    # where the sum rounds to the larger operand in both precisions; one rounding float64 -> float32 (RNE).
    with np.errstate(over="ignore", invalid="ignore"):
        o64 = a.view(np.float32).astype(np.float64) + b.view(np.float32).astype(np.float64)
        o = o64.astype(np.float32)
        t = (torch.from_numpy(a.view(np.float32).copy()) + torch.from_numpy(b.view(np.float32).copy())).numpy()
    nan = np.isnan(o)
    assert np.array_equal(o.view(np.uint32)[~nan], t.view(np.uint32)[~nan])
    np.savez(os.path.join(HERE, "edge_f32.npz"), a=a[~nan], b=b[~nan], out=o.view(np.uint32)[~nan])


def simulate_ring(call_nbytes, script, nslot, nrails, rail1max, depth):
    """Event simulation of the slot ring; returns (slots, rails, released-per-arrival)."""
    queues = [deque() for _ in range(nrails)]
    count = {}
    slots, rails, released = [], [], []
    seq, nxt, done = 0, 0, 0
    finished = set()
    k = 0
    while True:
        while nxt < len(call_nbytes) and seq - done < depth:
            seq += 1
            r = 1 if call_nbytes[nxt] <= rail1max else nrails
            slots.append(seq % nslot); rails.append(r)
            for q in queues[:r]:
                assert len(q) < nslot
                q.append((seq, seq % nslot, r))
            nxt += 1
        if k >= len(script):
            break
        s, slot, r = queues[script[k]].popleft()
        count[s] = count.get(s, 0) + 1
        if count[s] == r:
            released.append(s)
            finished.add(s)
            while done + 1 in finished:
                done += 1
        else:
            released.append(0)
        k += 1
    return slots, rails, released


def ring_traces():
    out = {}
    big, small = 4 << 20, 8192
    cases = {
        "ns2_r1": (2, 1, [small] * 7, 1),
        "ns4_r2_mixed": (4, 2, [big, small, big, big, small, small, big, big, big], 1),
        "ns4_r2_pipe3": (4, 2, [big] * 16, 3),
        "ns2_r2_pipe2": (2, 2, [big, big, small, big, big, small, big], 2),
    }
    for name, (nslot, nrails, calls, depth) in cases.items():
        rpc = [1 if c <= 98304 else nrails for c in calls]
        script = synth.arrival_script(7, len(calls), nrails, depth, rpc)
        slots, rails, released = simulate_ring(calls, script, nslot, nrails, 98304, depth)
        out[name + "_cfg"] = np.array([nslot, nrails, depth], dtype=np.int64)
        out[name + "_calls"] = np.array(calls, dtype=np.int64)
        out[name + "_script"] = np.array(script, dtype=np.int64)
        out[name + "_slots"] = np.array(slots, dtype=np.int64)
        out[name + "_rails"] = np.array(rails, dtype=np.int64)
        out[name + "_released"] = np.array(released, dtype=np.int64)
    np.savez(os.path.join(HERE, "ring_traces.npz"), **out)


if __name__ == "__main__":
    config1()
    edge_cases("bf16")
    edge_cases("f16")
    edge_f32()
    ring_traces()
    print("golden vectors written to", HERE)
