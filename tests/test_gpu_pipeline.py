"""GPU tests of the protocol around the kernels: multi-rail chunked pipeline with a
seeded arrival order, the async stress mix, the watchdog, and every mode switch."""
import ctypes
import os
import threading
import time

import numpy as np
import pytest
import torch

from gpu_util import DT, bits_np, dev, first_diff, say, session
from libtbvcoll_amd import synth

pytestmark = pytest.mark.gpu


def oracle_sum(orc, a, b):
    return orc.sum_torch(a.cpu(), b.cpu())


# ---------------------------------------------------------------- multi-rail chunked pipeline (64 MiB fp16)

@pytest.mark.parametrize("railsum", [0, 1])
def test_multirail_pipeline_seeded_arrival_order(orc, railsum):
    """fp16 [8192x4096] = 64 MiB as 16 chunks of CAP = 4 MiB, 2 rails x NSLOT = 4; every
    (chunk, rail) fragment arrives by side-stream copy + flag bump in a seeded random
    order; the result must equal the single-shot sum bit for bit."""
    nslot, cap, nchunks = 4, 4 << 20, 16
    numel = nchunks * cap // 2
    with session(rails=2, cap=cap, TBV_NSLOT=nslot, TBV_RAILSUM=railsum, TBV_WDOG=20) as tbv:
        a = dev(synth.normal(41, numel), torch.float16)
        p = dev(synth.normal(42, numel), torch.float16)
        out = torch.empty_like(a)
        script = synth.arrival_script(5, nchunks, 2, nslot - 1)
        k, released, slots, rails = orc.ring_model([cap] * nchunks, script, nslot, 2, 98304, nslot - 1)
        assert k == 2 * nchunks and sorted(x for x in released if x) == list(range(1, nchunks + 1))
        tbv.arrival_script(script)
        per = cap // 2
        for c in range(nchunks):
            tbv.stage_peer(p[c * per:(c + 1) * per])
        say("pipeline railsum", railsum, "script", script)
        assert tbv.all_reduce_chunked(a, out)
        torch.cuda.synchronize()
        assert not tbv.err()
        # observed arrivals follow the script: k-th arrival came from rail script[k], in per-rail FIFO order
        log = tbv.arrival_log()
        assert [r for _, r in log] == script
        for rail in (0, 1):
            assert [s for s, r in log if r == rail] == list(range(1, nchunks + 1))
        assert torch.equal(out, a + p)                               # single-shot sum, torch's kernel
        assert first_diff(out, oracle_sum(orc, a, p)) is None        # and the CPU oracle, all 32 Mi elements
        tbv.arrival_script([])


def test_chunked_ragged_tail_and_mixed_rails(orc):
    """A payload that is not a multiple of the cap, with a last chunk small enough to use one rail."""
    cap = 256 << 10
    with session(rails=2, cap=cap, TBV_NSLOT=3) as tbv:
        for name in ("bf16", "f32"):
            dt = DT[name]
            esz = 2 if name != "f32" else 4
            numel = (5 * cap + 6000) // esz
            a = dev(synth.uniform(51, numel), dt); p = dev(synth.uniform(52, numel), dt)
            out = torch.empty_like(a)
            per = cap // esz
            for c in range(6):
                tbv.stage_peer(p[c * per:min((c + 1) * per, numel)])
            assert tbv.all_reduce_chunked(a, out)
            torch.cuda.synchronize()
            assert first_diff(out, oracle_sum(orc, a, p)) is None
        assert not tbv.err()


# ---------------------------------------------------------------- async stress mix

def test_async_stress_mix(orc):
    """5,000 consecutive all-reduces, sizes uniform over {8 KB, 64 KB, 1 MB, 16 MB}, dtypes cycling
    bf16/fp16/fp32, values U[-4,4] seeded per call, progress threads and the 10 s watchdog live, no
    synchronisation between calls inside a window; every output is checked bit for bit against torch's
    add on the regenerated inputs (as step4/test_stress.py:33-35) and every 50th against the CPU oracle."""
    sizes = [8 << 10, 64 << 10, 1 << 20, 16 << 20]
    dts = [torch.bfloat16, torch.float16, torch.float32]
    ncalls, window = 5000, 100
    pick = synth.bits32(2024, ncalls, 7)
    with session(rails=2, cap=16 << 20, TBV_NSLOT=4, TBV_WDOG=10) as tbv:
        bad, checked_oracle = [], 0
        for w0 in range(0, ncalls, window):
            keep = []
            for it in range(w0, min(w0 + window, ncalls)):
                nb = sizes[int(pick[it]) % 4]; dt = dts[it % 3]
                numel = nb // (4 if dt == torch.float32 else 2)
                x = synth.torch_hash_uniform(2 * it, numel).to(dt)
                p = synth.torch_hash_uniform(2 * it + 1, numel).to(dt)
                out = torch.empty_like(x)
                tbv.stage_peer(p)
                assert tbv.all_reduce(x, out)
                keep.append((it, x, p, out))
            torch.cuda.synchronize()
            for it, x, p, out in keep:
                if not torch.equal(out, x + p):
                    bad.append(it)
                if it % 50 == 0:
                    assert first_diff(out, oracle_sum(orc, x, p)) is None, it
                    checked_oracle += 1
            if w0 % 1000 == 0:
                say("stress mix", w0, "bad", len(bad))
        assert not bad, (len(bad), bad[:5])
        assert checked_oracle == ncalls // 50 and not tbv.err()
        pre, xfer, post, enq, n = tbv.stats4()
        assert n == ncalls and xfer > 0 and enq > 0                  # rail 0 saw every call
        tbv.rails(); tbv.hist()


# ---------------------------------------------------------------- watchdog (condition forced from the host)

def test_watchdog_releases_gpu_and_error_is_sticky(orc):
    """The peer never signals call 3: within TBV_WDOG seconds the progress thread must log, set the
    error flag, still raise the GPU's flag (the stream drains), and every later call must fail."""
    with session(rails=2, cap=1 << 20, TBV_WDOG=1) as tbv:
        a = dev(synth.normal(1, 1 << 18), torch.bfloat16); p = dev(synth.normal(2, 1 << 18), torch.bfloat16)
        out = torch.empty_like(a)
        for _ in range(2):
            tbv.stage_peer(p); assert tbv.all_reduce(a, out)
        torch.cuda.synchronize()
        assert torch.equal(out, a + p) and not tbv.err()
        tbv.withhold(3, 1)                                           # rail 1 of call 3 is never signalled
        tbv.stage_peer(p)
        t0 = time.time()
        assert tbv.all_reduce(a, out)                                # enqueue itself succeeds
        torch.cuda.synchronize()                                     # returns: the flag was raised despite the error
        dt = time.time() - t0
        assert 0.8 < dt < 4.0, dt
        assert tbv.err()
        with pytest.raises(RuntimeError):
            tbv.all_reduce(a, out)                                   # rc -1: unrecoverable (step4/libtbvcoll.cpp:419)
        tbv.withhold(0, 0)


def test_watchdog_on_missing_pack_completion(orc):
    """The pack kernel of call 2 never raises its completion word (forced from the host): the progress
    threads give up after TBV_WDOG, set the error flag and still release the GPU."""
    with session(rails=2, cap=1 << 20, TBV_WDOG=1, TBV_FUSEWAIT=0) as tbv:
        a = dev(synth.normal(1, 1 << 18), torch.bfloat16); p = dev(synth.normal(2, 1 << 18), torch.bfloat16)
        out = torch.empty_like(a)
        tbv.stage_peer(p); assert tbv.all_reduce(a, out)
        torch.cuda.synchronize()
        assert torch.equal(out, a + p)
        tbv.withhold(2, -1)
        tbv.stage_peer(p)
        t0 = time.time()
        assert tbv.all_reduce(a, out)
        torch.cuda.synchronize()
        assert 0.8 < time.time() - t0 < 4.0
        assert tbv.err()
        with pytest.raises(RuntimeError):
            tbv.all_reduce(a, out)
        tbv.withhold(0, 0)


# ---------------------------------------------------------------- every mode gives the same bits

MODES = {
    "kwait": {"TBV_KWAIT": 1},
    "event": {"TBV_GPUSIG": 0},
    "sync": {"TBV_ASYNC": 0},
    "tag": {"TBV_TAG": 1},
    "cached_bounce": {"TBV_UNCACHED": 0},
    "recv_cached": {"TBV_UNCACHED": 1},
    "railsum": {"TBV_RAILSUM": 1},
    "fusewait": {"TBV_FUSEWAIT": 1 << 30},
    "stream_gate_only": {"TBV_FUSEWAIT": 0, "TBV_DEFERSIG": 0, "TBV_ONEKERNEL": 0},
    "no_defer": {"TBV_DEFERSIG": 0},
    "two_kernels": {"TBV_ONEKERNEL": 0},
    "fusewait_96k": {"TBV_FUSEWAIT": 98304},
    "fusewait_no_defer": {"TBV_FUSEWAIT": 1 << 30, "TBV_DEFERSIG": 0},
    "block512": {"TBV_BLOCK": 512, "TBV_UNROLL": 2, "TBV_GRIDCAP": 256},
    "host_wire": {"TBV_WIRE": "host"},
    "host_wire_tag": {"TBV_WIRE": "host", "TBV_TAG": 1},
    "host_wire_chunk": {"TBV_WIRE": "host", "TBV_CHUNK": 40000},
    "stream_wire": {"TBV_WIRE": "stream"},
    "chunk": {"TBV_CHUNK": 65536},
    "nslot2": {"TBV_NSLOT": 2},
    "nslot32": {"TBV_NSLOT": 32},
    "unroll4": {"TBV_UNROLL": 4, "TBV_GRIDCAP": 200},
    "pin": {"TBV_CPU": 0},
    "streaming": {"TBV_STREAMING": 1},
    "streaming_unroll2": {"TBV_STREAMING": 1, "TBV_UNROLL": 2},
    "merge_off": {"TBV_MERGE": 0},
    "staged_two_launches": {"TBV_STAGEDMERGE": 0},
    "fusewait_small": {"TBV_FUSEWAIT": 8192},
}


@pytest.mark.parametrize("mode", sorted(MODES))
def test_modes_bit_exact(orc, mode):
    with session(rails=2, cap=4 << 20, **MODES[mode]) as tbv:
        k = 0
        for name in ("bf16", "f16", "f32"):
            dt = DT[name]
            for nb in (8192, 57344, 229376, 4 << 20):
                numel = nb // (4 if name == "f32" else 2)
                outs = []
                for rep in range(6):                                  # back to back: slots get reused
                    k += 1
                    a = dev(synth.normal(1000 + k, numel), dt); p = dev(synth.normal(5000 + k, numel), dt)
                    out = torch.empty_like(a)
                    tbv.stage_peer(p)
                    assert tbv.all_reduce(a, out)
                    outs.append((a, p, out))
                torch.cuda.synchronize()
                for a, p, out in outs:
                    assert torch.equal(out, a + p), (mode, name, nb)
                assert first_diff(outs[-1][2], oracle_sum(orc, outs[-1][0], outs[-1][1])) is None
        # mirror mode too (reads the send bounce back through the side stream)
        a = dev(synth.normal(77, 300000), torch.float16)
        out = torch.empty_like(a)
        assert tbv.all_reduce(a, out)
        torch.cuda.synchronize()
        assert torch.equal(out, a + a)
        assert not tbv.err()
        if mode == "kwait":
            torch.cuda.synchronize()
            last = tbv.seq()
            assert tbv.footprints() == [last, last, last, last, 0]      # wait in, wait out, pack, sum done; no timeout
        if mode == "tag":
            checks, bad_plain, bad_sys = tbv.tag_counts()
            assert checks == k + 1 and bad_plain == 0 and bad_sys == 0


def test_resident_peer_fused_and_unfused(orc):
    """Early peer: payload already in the receive slots, flag up on entry; optional pack+sum fusion."""
    n = 16 << 20
    a = dev(synth.prefill_activations(100, n // 2), torch.bfloat16)
    b = dev(synth.prefill_activations(101, n // 2), torch.bfloat16)
    want = oracle_sum(orc, a, b)
    for fuse, merge, streaming in ((0, 1, 0), (1, 1, 0), (0, 0, 0), (0, 1, 1), (1, 1, 1), (0, 0, 1)):
        with session(rails=2, cap=n, TBV_FUSE=fuse, TBV_MERGE=merge, TBV_STREAMING=streaming) as tbv:
            tbv.peer_resident(b)
            out = torch.empty_like(a)
            for _ in range(9):
                assert tbv.all_reduce(a, out)
            torch.cuda.synchronize()
            assert first_diff(out, want) is None
            # the send bounce holds the local tensor in both variants
            slot = tbv.seq() % 4
            import ctypes
            hip = ctypes.CDLL("libamdhip64.so.7")
            hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
            img = torch.empty_like(a)
            assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(slot), n, 3) == 0
            assert torch.equal(img.view(torch.int16), a.view(torch.int16))
            # a smaller call under the same resident payload, then a staged one overriding it
            small = a[:4096].clone(); o2 = torch.empty_like(small)
            assert tbv.all_reduce(small, o2)
            p3 = dev(synth.normal(9, 4096), torch.bfloat16)
            tbv.stage_peer(p3); o3 = torch.empty_like(small)
            assert tbv.all_reduce(small, o3)
            torch.cuda.synchronize()
            assert torch.equal(o2, small + b[:4096]) and torch.equal(o3, small + p3)
            tbv.peer_resident(None)
            assert not tbv.err()


@pytest.mark.parametrize("streaming,segment", [(0, 0), (1, 0), (0, 1 << 20)])
def test_resident_peer_merged_launch_ragged(orc, streaming, segment):
    """Early peer above the one-kernel size: pack blocks and sum blocks share one launch.  Ragged byte counts,
    three dtypes, in place and out of place, slots reused; the bounce image is read back too.  With `segment` the
    payloads are several segments long, so each call is a row of merged launches of which only the last raises the
    completion word (what payloads beyond 256 MiB get by default)."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so.7")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    cap = 6 << 20
    extra = {"TBV_MERGEMAX": segment} if segment else {}
    with session(rails=2, cap=cap, TBV_NSLOT=3, TBV_STREAMING=streaming, TBV_UNROLL=(2 if streaming else 0), **extra) as tbv:
        for name in ("bf16", "f16", "f32"):
            dt = DT[name]
            esz = 4 if name == "f32" else 2
            peer = dev(synth.uniform(70, cap // esz), dt)
            tbv.peer_resident(peer)
            for k, numel in enumerate(((1 << 20) // esz + 1, (3 << 20) // esz + 7, cap // esz, (2 << 20) // esz + 3, (5 << 20) // esz - 1)):
                a = dev(synth.uniform(71 + k, numel), dt)
                want = oracle_sum(orc, a, peer[:numel])
                out = torch.empty_like(a)
                say("merged", name, numel, "streaming", streaming, "segment", segment)
                assert tbv.all_reduce(a, out)
                torch.cuda.synchronize()
                assert first_diff(out, want) is None, (name, numel)
                img = torch.empty_like(a)
                assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), numel * esz, 3) == 0
                assert np.array_equal(bits_np(img), bits_np(a))
                c = a.clone()
                assert tbv.all_reduce(c)                               # in place
                torch.cuda.synchronize()
                assert first_diff(c, want) is None, (name, numel, "in place")
                # in place the peer must still be sent the ORIGINAL tensor: no sum block may overwrite a vector
                # before it has been packed
                assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), numel * esz, 3) == 0
                assert np.array_equal(bits_np(img), bits_np(a)), (name, numel, "bounce image of the in-place call")
                # an output that overlaps the local tensor without being it takes two launches: the image is intact
                # whatever the (undefined) output holds
                if numel > 4096:
                    base = torch.cat([a, a[:64]])
                    src, dst = base[:numel], base[64:64 + numel]
                    assert tbv.all_reduce(src, dst)
                    torch.cuda.synchronize()
                    assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), numel * esz, 3) == 0
                    assert np.array_equal(bits_np(img), bits_np(a)), (name, numel, "bounce image of the overlapping call")
            tbv.peer_resident(None)
        assert not tbv.err()


@pytest.mark.parametrize("streaming", [0, 1])
def test_resident_peer_stripped_kernels(orc, streaming):
    """The stripped kernels of the early-peer step at sizes of whole tiles and with a ragged last tile (whole vectors
    short of a tile, a few odd bytes): out of place (merged launch) and in place (the reference's outp == NULL: the
    fused body, one lane loads a vector once, stores it to the bounce and stores the sum over it).  Every call's
    output equals the oracle's sum AND its bounce image equals the ORIGINAL tensor; then bursts of back-to-back
    in-place calls on distinct tensors, checked after each burst."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so.7")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    cap = 16 << 20
    with session(rails=2, cap=cap, TBV_NSLOT=4, TBV_STREAMING=streaming) as tbv:
        for name, sizes in (("bf16", (2 << 20, 6 << 20, 8 << 20, 16 << 20, (8 << 20) + 48, (11 << 20) + 2, (16 << 20) - 6)),
                            ("f16", (16 << 20, (9 << 20) + 8194)), ("f32", (4 << 20, 16 << 20, (10 << 20) + 4))):
            dt = DT[name]
            esz = 4 if name == "f32" else 2
            peer = dev(synth.uniform(170, cap // esz), dt)
            tbv.peer_resident(peer)
            for k, nbytes in enumerate(sizes):
                numel = nbytes // esz
                a = dev(synth.uniform(171 + k, numel), dt)
                want = oracle_sum(orc, a, peer[:numel])
                img = torch.empty_like(a)
                out = torch.empty_like(a)
                say("out of place", name, nbytes, "streaming", streaming)
                assert tbv.all_reduce(a, out)
                torch.cuda.synchronize()
                assert first_diff(out, want) is None, (name, nbytes, "out of place")
                assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 4), nbytes, 3) == 0
                assert np.array_equal(bits_np(img), bits_np(a)), (name, nbytes, "bounce image, out of place")
                for it in range(4):
                    c = a.clone()
                    say("in place", name, nbytes, "streaming", streaming, it)
                    assert tbv.all_reduce(c)
                    torch.cuda.synchronize()
                    assert first_diff(c, want) is None, (name, nbytes, it)
                    assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 4), nbytes, 3) == 0
                    assert np.array_equal(bits_np(img), bits_np(a)), (name, nbytes, it, "bounce image")
            tbv.peer_resident(None)
        # back to back, no synchronisation inside a burst
        peer = dev(synth.uniform(180, cap // 2), torch.bfloat16)
        tbv.peer_resident(peer)
        srcs = [dev(synth.uniform(181 + i, cap // 2), torch.bfloat16) for i in range(6)]
        wants = [x + peer for x in srcs]
        work = [x.clone() for x in srcs]
        say("in place, whole tiles, bursts", streaming)
        for rnd in range(12):
            for w in work:
                assert tbv.all_reduce(w)
            torch.cuda.synchronize()
            for x, w, want in zip(srcs, work, wants):
                assert torch.equal(w.view(torch.int16), want.view(torch.int16)), rnd
                w.copy_(x)
        tbv.peer_resident(None)
        assert not tbv.err()


# (the two block sizes: waiting blocks are capped in waves, so wider blocks must not take the wave slots that the
# deposit kernel, whose completion raises the flag, needs)
@pytest.mark.parametrize("env", [{}, {"TBV_GATEDGRID": 1024, "TBV_GATEDUNROLL": 2}, {"TBV_STREAMING": 1}, {"TBV_STAGEDMERGE": 0},
                                 {"TBV_BLOCK": 512}, {"TBV_BLOCK": 1024}])
def test_staged_call_in_one_launch(orc, env):
    """The peer's payload is not there when the call is made and the call is above the one-kernel size: pack blocks
    and gated sum blocks share one launch.  Ragged sizes, three dtypes, out of place and in place (the sum blocks
    then also wait for the last pack block), slots reused back to back; the bounce image must be the original
    tensor every time, and a 16 MiB call in place must equal the out-of-place result."""
    hip = ctypes.CDLL("libamdhip64.so.7")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    cap = 16 << 20
    with session(rails=2, cap=cap, TBV_NSLOT=3, **env) as tbv:
        for name in ("bf16", "f16", "f32"):
            dt = DT[name]
            esz = 4 if name == "f32" else 2
            # (from 8 MiB the staged launch has a stripped form whose last tile may be ragged: whole vectors short of a
            # tile, a few odd bytes, and both)
            sizes = [(1 << 20) // esz + 8, (3 << 20) // esz + 7, (2 << 20) // esz + 3, (5 << 20) // esz - 1,
                     (9 << 20) // esz + 24, (12 << 20) // esz + 1, (8 << 20) // esz + 4099] + ([cap // esz] if name == "bf16" else [])
            for k, numel in enumerate(sizes):
                a = dev(synth.uniform(171 + k, numel), dt); p = dev(synth.uniform(271 + k, numel), dt)
                want = oracle_sum(orc, a, p)
                out = torch.empty_like(a)
                say("staged one launch", name, numel, env)
                tbv.stage_peer(p)
                assert tbv.all_reduce(a, out)
                torch.cuda.synchronize()
                assert first_diff(out, want) is None, (name, numel)
                img = torch.empty_like(a)
                assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), numel * esz, 3) == 0
                assert np.array_equal(bits_np(img), bits_np(a))
                c = a.clone()
                tbv.stage_peer(p)
                assert tbv.all_reduce(c)                               # in place
                torch.cuda.synchronize()
                assert first_diff(c, want) is None, (name, numel, "in place")
                assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), numel * esz, 3) == 0
                assert np.array_equal(bits_np(img), bits_np(a)), (name, numel, "bounce image of the in-place call")
            # back to back without synchronising: slots and relay words are reused while earlier calls still run
            numel = (2 << 20) // esz + 16
            keep = []
            for k in range(8):
                a = dev(synth.uniform(400 + k, numel), dt); p = dev(synth.uniform(500 + k, numel), dt)
                out = a.clone() if k % 2 else torch.empty_like(a)
                tbv.stage_peer(p)
                assert tbv.all_reduce(out if k % 2 else a, None if k % 2 else out)
                keep.append((a, p, out))
            torch.cuda.synchronize()
            for a, p, out in keep:
                assert torch.equal(out, a + p), name
        assert not tbv.err()


def test_early_peer_then_staged_then_early_again(orc):
    """Early-peer mode mixed with staged calls: a staged call deposits its own payload into its receive slot, so
    the next early-peer call that lands on that slot must get the resident payload put back (through the wire)
    instead of summing the stale staged bytes; a full-size call restores the slot for good."""
    nslot, n = 4, 1 << 20
    with session(rails=2, cap=n, TBV_NSLOT=nslot) as tbv:
        b = dev(synth.uniform(11, n // 2), torch.bfloat16)
        tbv.peer_resident(b)
        outs = []
        for k in range(3 * nslot + 2):                       # slots get reused several times
            numel = (n // 2) if k % 5 == 4 else (4096 + 512 * k)
            a = dev(synth.uniform(100 + k, numel), torch.bfloat16)
            out = torch.empty_like(a)
            if k % 3 == 1:                                    # every third call brings its own payload
                p = dev(synth.uniform(500 + k, numel), torch.bfloat16)
                tbv.stage_peer(p)
            else:
                p = b[:numel]
            assert tbv.all_reduce(a, out)
            outs.append((k, a, p, out))
        torch.cuda.synchronize()
        for k, a, p, out in outs:
            assert first_diff(out, oracle_sum(orc, a, p)) is None, k
        assert not tbv.err()
        tbv.peer_resident(None)


def test_early_peer_cannot_release_a_call_still_waiting_for_rail_1(orc):
    """A two-rail staged call whose rail-1 fragment the host holds back, followed by one-rail early-peer calls.
    The call that wraps onto the held call's slot would raise that slot's flag on entry and so pass the held
    call's gate while half of its receive slot is still empty; it must not be issued before the held call has
    been released.  A second thread lifts the hold after 60 ms: the wrapping call has to have waited for it.
    Every kernel exits normally; the held transfer is bounded by the watchdog."""
    import threading
    nslot, big, small = 4, 1 << 20, 8192
    with session(rails=2, cap=big, TBV_NSLOT=nslot, TBV_WDOG=5) as tbv:
        b = dev(synth.uniform(21, big // 2), torch.bfloat16)
        tbv.peer_resident(b)
        a0 = dev(synth.uniform(22, big // 2), torch.bfloat16); p0 = dev(synth.uniform(23, big // 2), torch.bfloat16)
        o0 = torch.zeros_like(a0)
        smalls = [dev(synth.uniform(30 + k, small // 2), torch.bfloat16) for k in range(2 * nslot)]
        outs = [torch.empty_like(x) for x in smalls]
        # the model: with the slot guard the host cannot issue call 1+NSLOT before rail 1 of call 1 has arrived
        calls = [big] + [small] * nslot
        assert orc.ring_model2(calls, [0] * (nslot + 1) + [1], nslot, 2, 98304, 0, slot_guard=1)[0] == -1
        assert orc.ring_model2(calls, [0] * (nslot + 1) + [1], nslot, 2, 98304, 0, slot_guard=0)[4] == 1
        torch.cuda.synchronize()
        tbv.hold_rail(1, True)
        tbv.stage_peer(p0)
        assert tbv.all_reduce(a0, o0)                          # seq 1: staged, two rails, rail 1 held
        for k in range(nslot - 1):
            assert tbv.all_reduce(smalls[k], outs[k])          # seq 2..NSLOT: early peer, one rail, other slots
        lifter = threading.Timer(0.06, lambda: tbv.hold_rail(1, False))
        # while this thread waits inside the library, a call from another thread is refused (one caller at a time)
        # instead of sharing the sequence counter and the ring with it
        intruder_rc = []
        fn = tbv.raw_fn()
        spare = torch.zeros(64, device="cuda")
        stream_handle = torch.cuda.current_stream().cuda_stream
        intruder = threading.Timer(0.02, lambda: intruder_rc.append(
            fn(ctypes.c_void_p(spare.data_ptr()), None, 256, 0, ctypes.c_void_p(stream_handle))))
        t0 = time.time()
        lifter.start(); intruder.start()
        assert tbv.all_reduce(smalls[nslot - 1], outs[nslot - 1])   # seq 1+NSLOT wraps onto slot 1: waits for call 1's release
        waited = time.time() - t0
        intruder.join()
        assert intruder_rc == [-1], intruder_rc
        for k in range(nslot, len(smalls)):
            assert tbv.all_reduce(smalls[k], outs[k])
        lifter.join()
        torch.cuda.synchronize()
        assert not tbv.err()
        assert waited > 0.04, waited
        assert first_diff(o0, oracle_sum(orc, a0, p0)) is None
        for x, o in zip(smalls, outs):
            assert torch.equal(o, x + b[:small // 2])
        tbv.peer_resident(None)


def test_full_size_properties(orc):
    """Size-independent properties at the 16 MiB bench shape: commutativity (swap local and peer),
    x + 0 = x, x + (-x) = +0, and in-place equals out-of-place."""
    n = 16 << 20
    a = dev(synth.prefill_activations(100, n // 2), torch.bfloat16)
    b = dev(synth.prefill_activations(101, n // 2), torch.bfloat16)
    with session(rails=2, cap=n) as tbv:
        o1 = torch.empty_like(a); o2 = torch.empty_like(a); o3 = torch.empty_like(a); o4 = torch.empty_like(a)
        tbv.stage_peer(b); assert tbv.all_reduce(a, o1)
        tbv.stage_peer(a); assert tbv.all_reduce(b, o2)
        z = torch.zeros_like(a)
        tbv.stage_peer(z); assert tbv.all_reduce(a, o3)
        neg = -a
        tbv.stage_peer(neg); assert tbv.all_reduce(a, o4)
        c = a.clone()
        tbv.stage_peer(b); assert tbv.all_reduce(c)
        torch.cuda.synchronize()
        assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))
        assert torch.equal(o3, a)
        assert int(o4.view(torch.int16).count_nonzero()) == 0         # +0 everywhere, never -0
        assert torch.equal(c.view(torch.int16), o1.view(torch.int16))
        assert first_diff(o1, oracle_sum(orc, a, b)) is None
        assert not tbv.err()


def test_many_caller_streams_share_hardware_queues(orc):
    """The runtime multiplexes streams onto a few hardware queues.  With more live streams than queues a
    caller's gated stream and a rail's side stream can land on one queue, where a side-stream copy would
    sit behind the gate it is meant to release.  The engine probes every new caller stream and moves such
    streams to the host wire; every call must complete (no watchdog) and be exact."""
    streams = [torch.cuda.Stream() for _ in range(10)]
    with session(rails=2, cap=1 << 20, TBV_WDOG=5) as tbv:
        k = 0
        for rep in range(2):
            for st in streams:
                for nb in (8192, 1 << 20):
                    k += 1
                    a = dev(synth.normal(300 + k, nb // 2), torch.bfloat16); p = dev(synth.normal(900 + k, nb // 2), torch.bfloat16)
                    out = torch.empty_like(a)
                    torch.cuda.synchronize()
                    with torch.cuda.stream(st):
                        tbv.stage_peer(p)
                        assert tbv.all_reduce(a, out)
                    st.synchronize()
                    assert not tbv.err(), (rep, k)
                    assert torch.equal(out, a + p)
        # pinned host memory as the peer's payload
        hp = torch.from_numpy(synth.normal(5, 4096)).to(torch.bfloat16).pin_memory()
        a = dev(synth.normal(6, 4096), torch.bfloat16); out = torch.empty_like(a)
        tbv.stage_peer(hp)
        assert tbv.all_reduce(a, out)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), oracle_sum(orc, a, hp))


@pytest.mark.parametrize("seed,env", [(1, {}), (2, {"TBV_RAILSUM": 1}), (3, {"TBV_FUSEWAIT": 0, "TBV_DEFERSIG": 0, "TBV_ONEKERNEL": 0}),
                                      (4, {"TBV_WIRE": "host"}), (5, {"TBV_FUSEWAIT": 262144, "TBV_NSLOT": 2})])
def test_seeded_mix_of_everything(orc, seed, env):
    """1500 calls drawn from a seeded stream: sizes from 2 bytes to the cap including odd element counts,
    three dtypes, in place or not, aligned or offset pointers, peer staged / mirrored, two caller streams
    used alternately (synchronised when switching, as a caller must), occasional chunked calls over the
    cap.  Every result is compared with torch's add of the same operands; every 25th with the oracle."""
    cap = 1 << 20
    r = synth.bits32(7000 + seed, 1500 * 8, 7).reshape(1500, 8)
    dts = [torch.bfloat16, torch.float16, torch.float32]
    streams = [torch.cuda.current_stream(), torch.cuda.Stream()]
    with session(rails=2, cap=cap, **env) as tbv:
        cur = 0
        pend = []
        for it in range(1500):
            q = [int(v) for v in r[it]]
            dt = dts[q[0] % 3]
            esz = 4 if dt == torch.float32 else 2
            kind = q[1] % 10
            if kind < 3:
                numel = 1 + q[2] % 300
            elif kind < 8:
                numel = 1 + q[2] % (cap // esz)
            elif kind == 8:
                numel = cap // esz
            else:
                numel = cap // esz + 1 + q[2] % (3 * cap // esz)      # over the cap: chunked entry point
            off = (q[3] % 4) if q[3] % 5 == 0 else 0
            inplace = q[4] % 4 == 0
            mirror = q[5] % 7 == 0
            if q[6] % 40 == 0:                                         # switch streams the way a caller must
                torch.cuda.synchronize()
                cur ^= 1
            chunked = numel * esz > cap
            with torch.cuda.stream(streams[cur]):
                base = synth.torch_hash_uniform(10 * it + seed, numel + 4).to(dt)
                a = base[off:off + numel]
                p = None if mirror else synth.torch_hash_uniform(10 * it + 5 + seed, numel).to(dt)
                want = a + (a if mirror else p)
                keep_a = a.clone() if it % 25 == 0 else None       # operands for the oracle (a is overwritten in place)
                out = a if inplace else torch.empty(numel + 4, dtype=dt, device="cuda")[off:off + numel]
                if p is not None:
                    if chunked:
                        per = cap // esz
                        for c0 in range(0, numel, per):
                            tbv.stage_peer(p[c0:min(c0 + per, numel)])
                    else:
                        tbv.stage_peer(p)
                if chunked:
                    assert tbv.all_reduce_chunked(a, None if inplace else out)
                else:
                    assert tbv.all_reduce(a, None if inplace else out)
                pend.append((it, out, want, base, p, keep_a))
            if len(pend) >= 64 or it == 1499:
                torch.cuda.synchronize()
                for k, o, w, _, pp, ka in pend:
                    assert torch.equal(o, w), (seed, k, o.numel(), o.dtype)
                    if ka is not None:
                        assert first_diff(o, oracle_sum(orc, ka, ka if pp is None else pp)) is None
                pend = []
        assert not tbv.err()


def test_gates_inside_kernels_while_another_stream_keeps_the_gpu_busy(orc):
    """The kernels that wait for their flag inside (the one-kernel decode call, the pack + gated sum launch of a staged
    large call) hold their wave slots while they wait, and what raises the flag (the emulated peer's deposit kernel on a
    side stream) needs slots too.  Here a second stream keeps every CU busy with large elementwise kernels while 2000
    decode calls and 200 staged 1-4 MiB calls run: every result exact, no watchdog, no in-kernel wait that ran into
    its bound (footprint 4 stays 0; TBV_KWAIT=2 keeps the footprints without the diagnostic wait kernel)."""
    with session(rails=2, cap=4 << 20, TBV_NSLOT=4, TBV_WDOG=5, TBV_KWAIT=2) as tbv:
        bg = torch.cuda.Stream()
        big = torch.ones(64 << 20, dtype=torch.float32, device="cuda")        # 256 MiB: each pass keeps all CUs busy for ~100 us
        main = torch.cuda.current_stream()

        def load_gpu(n):
            with torch.cuda.stream(bg):
                for _ in range(n):
                    big.mul_(1.0000001)

        load_gpu(50)
        t0 = time.time()
        pend, bad = [], 0
        for it in range(2200):
            staged_big = it % 11 == 10
            nb = [1 << 20, 2 << 20, (3 << 20) + 4096, 4 << 20][(it // 11) % 4] + 16 if staged_big else 8192
            if staged_big and nb > (4 << 20):
                nb = 4 << 20
            dt = (torch.bfloat16, torch.float16, torch.float32)[it % 3]
            numel = nb // (4 if dt == torch.float32 else 2)
            a = synth.torch_hash_uniform(2 * it + 7, numel).to(dt)
            p = synth.torch_hash_uniform(2 * it + 8, numel).to(dt)
            inplace = it % 5 == 0
            out = a.clone() if inplace else torch.empty_like(a)
            tbv.stage_peer(p)
            assert tbv.all_reduce(out if inplace else a, None if inplace else out), it
            pend.append((it, a, p, out))
            if it % 8 == 0:
                load_gpu(4)                                                  # keep the other stream's queue full
            if len(pend) >= 64:
                main.synchronize()
                if tbv.err():
                    break                                                    # stop at the first failure
                bad += sum(0 if torch.equal(o, x + y) else 1 for _, x, y, o in pend)
                pend = []
        main.synchronize()
        bad += sum(0 if torch.equal(o, x + y) else 1 for _, x, y, o in pend)
        say("contention: 2200 calls in", round(time.time() - t0, 2), "s; bad", bad, "footprints", tbv.footprints())
        torch.cuda.synchronize()
        assert not tbv.err(), "a watchdog tripped"
        assert bad == 0
        assert tbv.footprints()[4] == 0                                      # no in-kernel wait ran into its bound
        want = oracle_sum(orc, pend[-1][1], pend[-1][2]) if pend else None
        assert want is None or first_diff(pend[-1][3], want) is None


def test_grids_beyond_the_small_counter_groups(orc):
    """Grids of more than 4064 blocks count their completion in groups of 64 instead of 32 (the tuning knobs allow up
    to 8128 blocks): pack, merged launch and sum at that size, staged and early peer, completion words included."""
    n = 32 << 20
    with session(rails=2, cap=n, TBV_UNROLL=1, TBV_GRIDCAP=8128, TBV_NSLOT=2) as tbv:
        a = dev(synth.uniform(61, n // 2, -4.0, 4.0), torch.bfloat16)
        b = dev(synth.uniform(62, n // 2, -4.0, 4.0), torch.bfloat16)
        want = a + b
        for k in range(3):
            out = torch.empty_like(a)
            say("8128-block grids, staged", k)
            tbv.stage_peer(b)
            assert tbv.all_reduce(a, out)
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), want.view(torch.int16))
        tbv.peer_resident(b)
        for k in range(3):
            out = torch.empty_like(a)
            say("8128-block grids, early peer", k)
            assert tbv.all_reduce(a, out)
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), want.view(torch.int16))
        tbv.peer_resident(None)
        sl = slice(0, 1 << 20)
        assert first_diff(out[sl], orc.sum_torch(a[sl].cpu(), b[sl].cpu())) is None
        assert not tbv.err()
