#!/usr/bin/env python3
"""Benchmark of the all-reduce data path on one MI355X.

A step is one tbv_ar_allreduce call through the C ABI on the 16 MiB bf16 prefill
workload with the peer's payload already in the receive slots: the local tensor is
copied into the uncached send bounce (completion word raised), and local + received
is written to the output.  Algorithmic bytes per step are 5N (pack 2N + sum 3N).

The headline (`value`, `roofline`) is the HBM-bound form of that step: 16 ring slots
and 12 rotating local/output tensors, 896 MiB touched in turn, so every operand comes
from HBM and not from the 256 MB Infinity Cache.  Prints ONE JSON line that also carries

  region           what the timed region costs beside its steps (start and stop latency of a drained
                   stream), from a second region of twice the steps
  long_run         the same leg over 2000 steps when --steps is small
  cold_two_launches, cold_fused_4N   the same cold step as pack kernel + sum kernel, and
                   as one kernel that reads the local tensor once (4N)
  cold_staged      the same cold step when the peer's payload is NOT there yet: deposited per call
                   through the emulated wire (one launch: pack blocks + gated sum blocks), and
                   cold_gated_flag_up, that launch with its flag already up
  resident         the step with everything it touches resident in the Infinity Cache
                   (4 slots, one local/output tensor): a cache figure, labelled so
  achievable       what plain read / write / copy kernels reach on this GPU (1 GiB
                   buffers, and 16 MiB cache-cold), and the launch-to-launch floor
  decode_latency   p50/p99 of (flag raised -> sum complete) for the 8 KB decode
                   workload, 10,000 back-to-back calls: library default (one kernel per
                   call) and, as decode_latency_stream_gate, the reference's sequence
                   pack kernel, hipStreamWaitValue64, sum kernel
  host_cost_per_call   time inside tbv_ar_allreduce and of its last launch, idle and busy stream
  pipeline_64MiB_fp16  64 MiB fp16 as 16 chunks of 4 MiB over 2 rails x 4 slots
  cold_int8_codec      the cold step with the int8 payload codec on
  sum_rmsnorm_fusion   the sum fused with the following RMSNorm against the two kernels apart
  cpu_baseline     the CPU oracle's restatement of the same step on the host cores.
"""
import argparse
import ctypes
import gc
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12                      # MI355X HBM3E, bytes/s
N_PREFILL = 16 << 20                   # 2048 x 4096 bf16
N_DECODE = 8192                        # 1 x 4096 bf16
COLD_NSLOT, COLD_NBUF = 16, 12         # 2 x 16 x 16 MiB of rings + 2 x 12 x 16 MiB of tensors = 896 MiB
TRAFFIC_FILE = os.path.join("profiles", "prefill16MiB_cold_pmc_fetch_write.txt")
TRACE_FILE = os.path.join("profiles", "prefill16MiB_cold_kernel_trace.txt")
TUNING_KEYS = ("TBV_NSLOT", "TBV_FUSE", "TBV_MERGE", "TBV_MERGEMAX", "TBV_STREAMING", "TBV_FUSEWAIT", "TBV_DEFERSIG", "TBV_ONEKERNEL", "TBV_CODEC", "TBV_CODEC_MIN",
               "TBV_STAGEDMERGE", "TBV_FORCEGATE", "TBV_GATEDGRID", "TBV_GATEDUNROLL", "TBV_ROWGRID", "TBV_CODECGRID")


def pct(xs, q):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, int(q * len(xs)))]


def traffic_from_profile(kernel):
    """HBM-side bytes per launch of `kernel` as the committed counter summary states them
    (a line `TRAFFIC kernel=<name> bytes_per_launch=<n>`); None when the file has no such line."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            for ln in f:
                m = re.match(r"\s*TRAFFIC kernel=(\S+) bytes_per_launch=(\d+)", ln)
                if m and m.group(1) == kernel:
                    return int(m.group(2))
    except OSError:
        pass
    return None


def avg_from_profile(kernel):
    """Average duration (us) of `kernel` as the committed rocprofv3 kernel-trace summary states it
    (a line `KERNEL_AVG kernel=<name> avg_ns=<n> ...`); None when the file has no such line."""
    try:
        with open(os.path.join(ROOT, TRACE_FILE)) as f:
            for ln in f:
                m = re.match(r"\s*KERNEL_AVG kernel=(\S+) avg_ns=([0-9.]+)", ln)
                if m and m.group(1) == kernel:
                    return float(m.group(2)) / 1e3
    except OSError:
        pass
    return None


def own_warmup(warmup, nslot, nbuf):
    """Untimed steps before the clock: at least two full periods of the (tensor, slot) rotation."""
    import math
    return max(warmup, 2 * math.lcm(nslot, nbuf), 48)


def run_prefill(tbv, torch, synth, st, steps, warmup, nslot, nbuf, env=(), long_steps=0, check="exact", staged=False, fit_region=False,
                inplace=False):
    """`steps` timed calls after `warmup` untimed ones (never fewer than two turns of every rotating tensor and
    ring slot, so no buffer is touched for the first time inside the clock), then an optional long run, then a
    pass of the same steps with the dispatch timestamps of every kernel launch.  With `staged` the peer's payload
    is handed to the emulated wire before every call instead of sitting in the receive slots beforehand.  With
    `inplace` every call overwrites its local tensor (the reference's outp == NULL); the rotating tensors then
    accumulate, and exactness is checked on a last round of calls from fresh copies."""
    n = N_PREFILL
    for k in TUNING_KEYS:
        os.environ.pop(k, None)
    os.environ["TBV_NSLOT"] = str(nslot)
    for k, v in env:
        os.environ[k] = str(v)
    tbv.shutdown()
    tbv.init(0, "rail0,rail1", "", cap_bytes=n)
    a = torch.from_numpy(synth.prefill_activations(100, n // 2)).to(torch.bfloat16).cuda()
    b = torch.from_numpy(synth.prefill_activations(101, n // 2)).to(torch.bfloat16).cuda()
    locs = [a] + [a.clone() for _ in range(nbuf - 1)]
    outs = [torch.empty_like(a) for _ in range(nbuf)]
    fn = tbv.raw_fn()
    ps = ctypes.c_void_p(st.cuda_stream)
    ptrs = [(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(o.data_ptr())) for x, o in zip(locs, outs)]
    if inplace:
        locs[0] = a.clone()            # `a` itself stays intact for the check
        ptrs = [(ctypes.c_void_p(x.data_ptr()), None) for x in locs]
    if not staged:
        tbv.peer_resident(b)           # the peer's payload sits in every receive slot before the clock starts
    stage, pb = tbv.lib().tbv_emu_stage_peer, ctypes.c_void_p(b.data_ptr())
    counter = [0]

    def step():
        pa, po = ptrs[counter[0] % nbuf]
        counter[0] += 1
        if staged and stage(pb, n) != 0:
            raise RuntimeError("tbv_emu_stage_peer failed")
        rc = fn(pa, po, n, 2, ps)
        if rc != 0:
            raise RuntimeError(f"tbv_ar_allreduce rc={rc}")

    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev_us = [None]

    def timed(k, events=False):
        """Host clock around exactly k steps between two device-wide synchronisations.  With `events`, two events on the
        caller's stream bracket the launches after the first (the first one's start-up, the host's launch latency on a
        drained stream, is not a launch duration): device time / (k - 1) is the average launch.  (The two event records
        cost the region about 10 us of their own, so the host-clocked figure comes from a region without them.)"""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step()
        if events and k > 1:
            ev[0].record(st)
        for _ in range(k - 1):
            step()
        if events and k > 1:
            ev[1].record(st)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ev_us[0] = ev[0].elapsed_time(ev[1]) * 1e3 / (k - 1) if events and k > 1 else None
        return dt

    for _ in range(own_warmup(warmup, nslot, nbuf)):
        step()
    torch.cuda.synchronize()
    # the last of the warm-up has the shape of the timed region (drained stream, a short burst, drained again): the
    # first such region after a long queue of launches runs 10-15 % slower than the ones that follow it
    # (nothing stands between it and the timed region: a pause of even 20 us before a region costs its first launch
    # 4-9 us, the progress threads having gone to sleep and the GPU idle)
    tbv.stats4()                       # drop what the warm-up (and the first call's stream probe) accumulated
    gc.collect()
    gc.disable()                       # no collector pause inside a region of a few hundred microseconds
    for _ in range(2):
        timed(min(steps, 48))
    wall = timed(steps)
    if not fit_region:
        # a comparison leg (not the headline, whose K steps are timed exactly once): best of three regions, so that a
        # slow spell of the host (these legs need a call every 12-14 us from it) does not pass for GPU time
        wall = min(wall, timed(steps), timed(steps))
    # the same region again with the two events in it; a region of few steps is repeated and the median taken, since one
    # host hiccup inside a 20-step region moves its average by several percent
    ev_runs = []
    for _ in range(5 if steps <= 500 else 1):
        timed(steps, events=True)
        if ev_us[0]:
            ev_runs.append(ev_us[0])
    ev_timed_us = sorted(ev_runs)[len(ev_runs) // 2] if ev_runs else None
    tbv.stats4()
    # what the region costs beside its steps: a second region of twice the steps gives slope and intercept
    region = None
    if fit_region and steps <= 500:
        w2 = min(timed(2 * steps) for _ in range(3))
        w1 = min([wall] + [timed(steps) for _ in range(2)])
        e2 = min(timed(2 * steps, events=True) for _ in range(3))
        e1 = min(timed(steps, events=True) for _ in range(3))
        region = {"steps_1x_us": round(w1 * 1e6, 2), "steps_2x_us": round(w2 * 1e6, 2), "per_step_us": round((w2 - w1) / steps * 1e6, 3),
                  "fixed_us": round((2 * w1 - w2) * 1e6, 2), "fixed_us_with_two_event_records": round((2 * e1 - e2) * 1e6, 2),
                  "what": "best of three host-clocked regions of K and of 2K steps: per_step = (T(2K) - T(K)) / K is the steady step, fixed = "
                          "2 T(K) - T(2K) is what one region pays for starting on a drained stream and for seeing the end of the last kernel"}
    long_wall = timed(long_steps, events=True) if long_steps else None
    ev_long_us = ev_us[0] if long_steps else None
    # host cost of one call (time inside tbv_ar_allreduce), from a burst short enough never to wait for room in the ring;
    # three calls first, so that the burst does not pay for waking progress threads that went to sleep during the long run's drain
    torch.cuda.synchronize()
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    tbv.stats4()
    burst = min(nslot - 1, 12)
    marks = [time.perf_counter()]
    for _ in range(burst):
        step()
        marks.append(time.perf_counter())
    enq_py = sorted(marks[i + 1] - marks[i] for i in range(burst))[burst // 2] * 1e6     # the median: the first call may have to wake the threads
    torch.cuda.synchronize()           # the averages are per completed transfer: let all of them complete
    # The library's own figure is an average per completed transfer (as the reference's, step4/libtbvcoll.cpp:518-529), and a call
    # whose peer payload is already in place has no transfer to complete: there the caller's clock around the ctypes call stands in.
    enq = tbv.stats4()[3] if staged else enq_py
    want = a + b
    if inplace:
        # repeated sums of small numbers stay finite; for the check every tensor starts again from `a`
        torch.cuda.synchronize()
        for x in locs:
            x.copy_(a)
        for _ in range(nbuf):
            step()
        torch.cuda.synchronize()
        outs = locs
    if check == "codec":
        # with the int8 codec every element is within half a quantisation step of each operand's group of 128
        # (step = (max - min) / 255), plus the rounding of the result to bf16
        def step_of(t):
            g = t.float().reshape(-1, 128)
            return ((g.amax(1) - g.amin(1)) / 255.0).repeat_interleave(128)
        steps2 = step_of(a) + step_of(b)
        bound = steps2 * 0.5005 + ((a.float() + b.float()).abs() + steps2) * 2.0 ** -8 + 1e-12
        ok = all(bool(((o.float() - (a.float() + b.float())).abs() <= bound).all()) for o in outs)
    else:
        ok = all(bool(torch.equal(o, want)) for o in outs)    # the timed path computed the sum, bit for bit
    tbv.stats4()

    ksteps = max(min(steps, 1000), 240)
    tbv.kernel_timing(True)
    for _ in range(ksteps):
        step()
    n_pack, pack_us, pack_min = tbv.kernel_times(0)
    n_sum, sum_us, sum_min = tbv.kernel_times(1)
    tbv.kernel_timing(False)
    torch.cuda.synchronize()
    err = tbv.err()
    tbv.shutdown()
    gc.enable()
    for k, _ in env:
        os.environ.pop(k, None)
    return {"wall": wall, "steps": steps, "long_wall": long_wall, "long_steps": long_steps, "ok": ok and not err, "enq_us": enq,
            "ev_us": ev_timed_us, "ev_runs": ev_runs, "ev_long_us": ev_long_us, "region": region,
            "pack_us": pack_us, "pack_min_us": pack_min, "n_pack": n_pack, "sum_us": sum_us, "sum_min_us": sum_min, "n_sum": n_sum}


def kernel_roofline(nbytes, us, min_us, launches, ceiling_gbps=None):
    if not us or us <= 0:
        return None
    gbps = nbytes / (us * 1e-6) / 1e9
    r = {"algorithmic_bytes": nbytes, "avg_launch_us": round(us, 3), "min_launch_us": round(min_us, 3), "launches": launches,
         "achieved": round(gbps, 1), "unit": "GB/s", "frac": round(gbps * 1e9 / HBM_PEAK, 4)}
    if ceiling_gbps:
        r["frac_of_measured_copy_ceiling"] = round(gbps / ceiling_gbps, 4)
    return r


def run_achievable(tbv):
    """Plain streaming kernels shipped in the library: the denominators this GPU really offers."""
    gib = 1 << 30
    out = {"what": "in-tree read / write / copy kernels (16-byte vectors, 256-lane blocks), dispatch timestamps; 1 GiB buffers, "
                   "and 16 MiB launches walking a 1 GiB pool (cache-cold)"}
    for name, kind, nbytes, pool, reps, mult in (("read_1GiB", 0, gib, gib, 10, 1), ("write_1GiB", 1, gib, gib, 10, 1),
                                                 ("copy_1GiB", 2, gib, gib, 10, 2), ("copy_plain_1GiB", 3, gib, gib, 10, 2),
                                                 ("copy_16MiB_cold", 2, N_PREFILL, gib, 120, 2), ("read_16MiB_cold", 0, N_PREFILL, gib, 120, 1)):
        mean, mn = tbv.hbm_probe(kind, nbytes, pool, reps)
        out[name] = {"GBps": round(mult * nbytes / (mean * 1e-6) / 1e9, 1), "avg_us": round(mean, 2), "min_us": round(mn, 2),
                     "frac_of_peak": round(mult * nbytes / (mean * 1e-6) / HBM_PEAK, 4)}
    out["empty_kernel_launch_to_launch_us"] = round(tbv.launch_floor(2000), 2)
    fl = tbv.step_floor(N_PREFILL, 480)
    out["step_floor_16MiB_cold"] = {"us": round(fl, 2), "GBps_4N": round(4 * N_PREFILL / (fl * 1e-6) / 1e9, 1),
                                    "what": "a kernel that only moves the step's four streams (reads local and received, writes the uncached bounce and "
                                            "the bf16 sum; no counting, no completion word, no gate) on the same cache-cold rotation: no form of the "
                                            "step can be shorter than this"}
    return out


def run_decode(tbv, torch, synth, st, iters, fusewait):
    n = N_DECODE
    for k in TUNING_KEYS:
        os.environ.pop(k, None)
    os.environ["TBV_NSLOT"] = "4"
    os.environ["TBV_FUSEWAIT"] = str(n) if fusewait else "0"
    os.environ["TBV_DEFERSIG"] = "1" if fusewait else "0"
    os.environ["TBV_ONEKERNEL"] = "1" if fusewait else "0"
    tbv.shutdown()
    tbv.init(0, "rail0", "", cap_bytes=n)
    npeer = 64
    locs = [torch.from_numpy(synth.normal(2 * i, n // 2)).to(torch.bfloat16).cuda() for i in range(npeer)]
    peers = [torch.from_numpy(synth.normal(2 * i + 1, n // 2)).to(torch.bfloat16).cuda() for i in range(npeer)]
    outs = [torch.empty_like(locs[0]) for _ in range(npeer)]
    tbv.latency_probe(True)
    with torch.cuda.stream(st):
        for it in range(200):
            tbv.stage_peer(peers[it % npeer]); tbv.all_reduce(locs[it % npeer], outs[it % npeer])
        torch.cuda.synchronize()
        tbv.latencies()
        tbv.stats4()
        t0 = time.perf_counter()
        for it in range(iters):
            k = it % npeer
            tbv.stage_peer(peers[k])
            if not tbv.all_reduce(locs[k], outs[k]):
                raise RuntimeError("decode call not handled")
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    _, _, post, enq, _ = tbv.stats4()
    lat = tbv.latencies()
    ok = all(bool(torch.equal(outs[k], locs[k] + peers[k])) for k in range(npeer)) and not tbv.err()
    tbv.latency_probe(False)
    tbv.shutdown()
    for k in TUNING_KEYS:
        os.environ.pop(k, None)
    return {"p50_us": round(pct(lat, 0.50), 2), "p99_us": round(pct(lat, 0.99), 2), "min_us": round(min(lat), 2),
            "samples": len(lat), "us_per_call_wall": round(wall / iters * 1e6, 2), "bit_exact": ok,
            "host_enqueue_us": round(enq, 2), "host_post_us": round(post, 2),
            "gate": "one kernel per call: pack, completion word, flag poll, sum (library default up to 1 MiB)" if fusewait
            else "pack kernel, hipStreamWaitValue64, sum kernel (TBV_FUSEWAIT=0 TBV_DEFERSIG=0 TBV_ONEKERNEL=0)",
            "measured": "host clock: just before the progress thread raises the flag -> host sees the sum's done word; "
                        "host_enqueue_us is the time inside tbv_ar_allreduce per call in this back-to-back loop (it includes waiting for "
                        "ring room behind the emulated wire), host_post_us its last launch; the *_idle_us pair is the same call on a drained stream"}


def run_host_cost(tbv, torch, synth, st, calls=2000):
    """Time inside tbv_ar_allreduce per call (enqueue) and of its last launch (post), from the library's own
    statistics, when the caller is never held up by back-pressure: the stream is drained between calls (idle
    stream) or the calls are issued back to back with the peer's payload already in place (busy stream, the
    GPU work of these sizes is shorter than the host's)."""
    import ctypes
    out = {"what": "tbv_ar_stats' enqueue / post per call in us; idle = stream drained between calls, peer staged per call; "
                   "busy = back to back, peer's payload resident, the caller never waits for ring room"}
    for nb, name in ((N_DECODE, "8KB"), (4 << 20, "4MiB"), (N_PREFILL, "16MiB")):
        for k in TUNING_KEYS:
            os.environ.pop(k, None)
        os.environ["TBV_NSLOT"] = "4"
        tbv.shutdown()
        tbv.init(0, "rail0", "", cap_bytes=nb)
        a = torch.from_numpy(synth.normal(3, nb // 2)).to(torch.bfloat16).cuda()
        b = torch.from_numpy(synth.normal(4, nb // 2)).to(torch.bfloat16).cuda()
        o = torch.empty_like(a)
        fn = tbv.raw_fn()
        pa, po, ps = ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(o.data_ptr()), ctypes.c_void_p(st.cuda_stream)
        res = {}
        with torch.cuda.stream(st):
            for _ in range(100):
                tbv.stage_peer(b); fn(pa, po, nb, 2, ps); torch.cuda.synchronize()
            tbv.stats4()
            for _ in range(calls):
                tbv.stage_peer(b); fn(pa, po, nb, 2, ps); torch.cuda.synchronize()
            _, _, post, enq, _ = tbv.stats4()
            res["idle"] = {"enqueue_us": round(enq, 2), "post_us": round(post, 2)}
            if nb > (4 << 20):         # GPU-bound beyond this size: back-to-back calls wait for ring room
                res["bit_exact"] = bool(torch.equal(o, a + b)) and not tbv.err()
                out[name] = res
                continue
            tbv.peer_resident(b)
            for _ in range(200):
                fn(pa, po, nb, 2, ps)
            torch.cuda.synchronize(); tbv.stats4()
            t0 = time.perf_counter()
            for _ in range(10 * calls):
                fn(pa, po, nb, 2, ps)
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            _, _, post, enq, _ = tbv.stats4()
            res["busy"] = {"enqueue_us": round(enq, 2), "post_us": round(post, 2), "caller_loop_us_per_call": round((t1 - t0) / (10 * calls) * 1e6, 2)}
            res["bit_exact"] = bool(torch.equal(o, a + b)) and not tbv.err()
            tbv.peer_resident(None)
        out[name] = res
    tbv.shutdown()
    os.environ.pop("TBV_NSLOT", None)
    return out


def run_pipeline(tbv, torch, synth, st, reps=20):
    """64 MiB fp16 as 16 chunks of CAP = 4 MiB over 2 rails x 4 slots, each (chunk, rail) fragment deposited by a
    side-stream copy and signalled by a 64-bit flag; three packs ahead, so sums overlap arrivals."""
    cap, nchunks = 4 << 20, 16
    numel = nchunks * cap // 2
    for k in TUNING_KEYS:
        os.environ.pop(k, None)
    os.environ["TBV_NSLOT"] = "4"
    tbv.shutdown()
    tbv.init(0, "rail0,rail1", "", cap_bytes=cap)
    a = torch.from_numpy(synth.normal(41, numel)).to(torch.float16).cuda()
    p = torch.from_numpy(synth.normal(42, numel)).to(torch.float16).cuda()
    out = torch.empty_like(a)
    per = cap // 2
    times = []
    with torch.cuda.stream(st):
        for r in range(reps + 3):
            for c in range(nchunks):
                tbv.stage_peer(p[c * per:(c + 1) * per])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            tbv.all_reduce_chunked(a, out)
            st.synchronize()           # the caller's stream is complete: the result is there for whatever the caller queues next
            t1 = time.perf_counter()
            torch.cuda.synchronize()   # (a device-wide wait also visits the rails' side streams: 50 us more, none of it the path's)
            if r >= 3:
                times.append(t1 - t0)
    ok = bool(torch.equal(out, a + p)) and not tbv.err()
    tbv.shutdown()
    os.environ.pop("TBV_NSLOT", None)
    med = pct(times, 0.5)
    return {"us": round(med * 1e6, 1), "min_us": round(min(times) * 1e6, 1), "GBps_5N": round(5 * numel * 2 / med / 1e9, 1),
            "bit_exact": ok, "reps": reps,
            "what": "tbv_ar_allreduce_chunked, 16 x 4 MiB fp16, 2 rails x NSLOT 4, every fragment through the emulated wire; "
                    "host clock from the call to the completion of the caller's stream, median"}


def run_rmsnorm_fusion(tbv, torch, synth, st):
    """Sum fused with the following RMSNorm (one row kernel: read local and received, write the sum and the
    normalised row, 4N) against the sum kernel followed by a norm-only launch (3N + 2N), on the prefill shape
    (cache-cold, 24 rotating buffer sets) and on decode shapes; both orders bit-identical."""
    lib = tbv.load()
    hidden = 4096
    out = {"what": "tbv_emu_run_sum_norm mode 1 (fused, 4N) vs tbv_emu_run_sum + mode 0 (sum 3N, then norm 2N); bf16, hidden 4096; "
                   "GPU events around 240 launches over 24 rotating buffer sets (4 for the decode shapes), best of three runs; us per step"}
    w = torch.from_numpy(1.0 + 0.25 * synth.normal(5, hidden)).to(torch.bfloat16).cuda()
    ps = st.cuda_stream
    for rows in (1, 128, 2048):
        nset = 24 if rows == 2048 else 4
        n = rows * hidden * 2
        A = [torch.from_numpy(synth.normal(10 + i, rows * hidden)).to(torch.bfloat16).cuda() for i in range(2)]
        sets = [(A[0].clone(), A[1].clone(), torch.empty_like(A[0]), torch.empty_like(A[0])) for _ in range(nset)]

        cold = 4 if rows == 2048 else 0     # the prefill shape rotates over 1.5 GiB of buffers: cache-cold hints, as the engine's streaming profile

        def fused(i):
            a, b, o, nm = sets[i % nset]
            lib.tbv_emu_run_sum_norm(1 + cold, o.data_ptr(), a.data_ptr(), b.data_ptr(), nm.data_ptr(), w.data_ptr(), 1e-6, rows, hidden, 2, ps)

        def separate(i):
            a, b, o, nm = sets[i % nset]
            lib.tbv_emu_run_sum(o.data_ptr(), a.data_ptr(), b.data_ptr(), n, 2, ps)
            lib.tbv_emu_run_sum_norm(0 + cold, None, o.data_ptr(), None, nm.data_ptr(), w.data_ptr(), 1e-6, rows, hidden, 2, ps)

        res = {}
        with torch.cuda.stream(st):
            for name, fn in (("fused", fused), ("separate", separate)):
                for i in range(2 * nset):
                    fn(i)
                runs = []
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    torch.cuda.synchronize()
                    e0.record()
                    for i in range(240):
                        fn(i)
                    e1.record()
                    torch.cuda.synchronize()
                    runs.append(e0.elapsed_time(e1) * 1e3 / 240)
                res[name] = min(runs)
                res[name + "_runs"] = [round(x, 2) for x in runs]
            fused(0); torch.cuda.synchronize(); f_out, f_nm = sets[0][2].clone(), sets[0][3].clone()
            separate(0); torch.cuda.synchronize()
            same = bool(torch.equal(f_out, sets[0][2])) and bool(torch.equal(f_nm.view(torch.int16), sets[0][3].view(torch.int16)))
        out[f"rows_{rows}"] = {"fused_us": round(res["fused"], 2), "separate_us": round(res["separate"], 2),
                               "saved_us": round(res["separate"] - res["fused"], 2), "bit_identical": same, "fused_runs_us": res["fused_runs"],
                               "fused_GBps_4N": round(4 * n / res["fused"] / 1e3, 1), "fused_frac_of_peak": round(4 * n / (res["fused"] * 1e-6) / HBM_PEAK, 4)}
    return out


def run_codec_accuracy(tbv, torch, synth, st):
    """The codec's own accuracy metric: relative L2 error and SNR of the coded all-reduce (through the library, 2 MiB
    bf16 calls with TBV_CODEC=1) against the exact sum of the two operands, whole-tensor and on the non-outlier elements,
    on the prefill distribution with and without its 0.1 % outliers, on N(0,1) and on U[-4,4]."""
    from libtbvcoll_amd import codec_metric
    numel = 1 << 20
    for k in TUNING_KEYS:
        os.environ.pop(k, None)
    os.environ["TBV_NSLOT"] = "4"
    os.environ["TBV_CODEC"] = "1"
    tbv.shutdown()
    tbv.init(0, "rail0,rail1", "", cap_bytes=2 * numel)
    out = {"what": "relative L2 error (and SNR) of out = decode(own image) + decode(peer image) against float64(a) + float64(b); "
                   "`typical` = over the elements that are not outliers (|x| < cut in both operands); stretched groups = groups of 128 of "
                   "either operand that hold an outlier; rel_l2_uncoded = the same figure for the plain bf16 all-reduce; 2^20 bf16 elements",
           "group": 128, "code_bits": 8}
    with torch.cuda.stream(st):
        for name, gen, cut in codec_metric.distributions(synth):
            a = torch.from_numpy(gen(100, numel)).to(torch.bfloat16).cuda()
            b = torch.from_numpy(gen(101, numel)).to(torch.bfloat16).cuda()
            o = torch.empty_like(a)
            tbv.stage_peer(b)
            if not tbv.all_reduce(a, o):
                raise RuntimeError("coded call not handled")
            torch.cuda.synchronize()
            m = codec_metric.accuracy(o.float().cpu().numpy(), a.float().cpu().numpy(), b.float().cpu().numpy(), cut, (a + b).float().cpu().numpy())
            m["outlier_cut"] = cut
            out[name] = m
    ok = not tbv.err()
    tbv.shutdown()
    for k in ("TBV_NSLOT", "TBV_CODEC"):
        os.environ.pop(k, None)
    out["no_transfer_error"] = ok
    out["reading"] = ("without outliers the coded sum is within 0.4-0.6 % of the exact one (44-48 dB; plain bf16: 0.18 %); one element in a "
                      "thousand at +-8 stretches a fifth of the groups and the error on the other elements is about 16 % (16 dB), while "
                      "the whole-tensor figure still reads 1.3 % because the outliers carry the norm")
    return out


def run_cpu_baseline(torch, synth):
    """The oracle's restatement of the same step (memcpy pack + fp32-upcast sum, RNE) on the host cores."""
    from oracle import oracle
    n = N_PREFILL
    a = oracle.torch_bits(torch.from_numpy(synth.prefill_activations(100, n // 2)).to(torch.bfloat16)).copy()
    b = oracle.torch_bits(torch.from_numpy(synth.prefill_activations(101, n // 2)).to(torch.bfloat16)).copy()
    cores = max(1, min(16, os.cpu_count() or 1))
    t1 = oracle.time_reduce_copy(oracle.DT_BF16, a, b, 1, 2, 200)
    tn = oracle.time_reduce_copy(oracle.DT_BF16, a, b, cores, 5, 2000)
    nd = N_DECODE
    da = oracle.torch_bits(torch.from_numpy(synth.normal(0, nd // 2)).to(torch.bfloat16)).copy()
    db = oracle.torch_bits(torch.from_numpy(synth.normal(1, nd // 2)).to(torch.bfloat16)).copy()
    td = oracle.time_reduce_copy(oracle.DT_BF16, da, db, 1, 100, 2000)
    return {"value": round(5 * n / tn / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port", "host_cpu_count": os.cpu_count(),
            "host_cpus_usable": len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else None,
            "single_thread_GBps": round(5 * n / t1 / 1e9, 2), "decode_8KB_single_thread_us": round(td * 1e6, 2),
            "sample": f"16 MiB bf16 prefill step (pack 2N + sum 3N), median of 2000 steps on {cores} threads "
                      f"(static contiguous partition) and of 200 steps on 1 thread, about 10 s of CPU work; 8 KB decode step: median of 2000 on 1 thread"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--decode-iters", type=int, default=10000)
    ap.add_argument("--legs", default="cold,two,fused,staged,resident,achievable,decode,host,pipeline,codec,rmsnorm,cpu",
                    help="comma list of the extra legs to run beside the headline (cold) leg")
    ap.add_argument("--headline-env", default="", help="TBV_X=v,... applied to the headline leg (for profiling one variant)")
    ap.add_argument("--rotate", default=f"{COLD_NSLOT},{COLD_NBUF}",
                    help="ring slots, rotating local/output tensors of the headline leg (4,1 = the cache-resident shape; for experiments)")
    ap.add_argument("--calibrate-copy", type=int, default=0,
                    help="also run this many plain 16 MiB device copies (known 16 MiB read + 16 MiB written), "
                         "so a counter run of this command holds a kernel of known traffic to scale by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    legs = set(x for x in args.legs.split(",") if x)

    import torch
    from libtbvcoll_amd import synth, tbvcoll as tbv
    if not os.path.exists(os.path.join(ROOT, "libtbvcoll_amd", "libtbvcoll.so")):       # load what is built; build only if nothing is
        import __graft_entry__
        __graft_entry__.build()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the data path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)

    # one caller stream for every part: each extra live stream makes it likelier that the runtime puts the
    # caller's stream and a rail's side stream on the same hardware queue (the engine would then fall back
    # to its slower host wire, which only matters for the emulated peer, not for the timed kernels)
    st = torch.cuda.Stream()
    n = N_PREFILL
    henv = tuple(tuple(kv.split("=", 1)) for kv in args.headline_env.split(",") if kv)
    fused_headline = dict(henv).get("TBV_FUSE") == "1"
    two_headline = dict(henv).get("TBV_MERGE") == "0" and not fused_headline
    long_steps = 2000 if args.steps < 1000 else 0
    h_nslot, h_nbuf = (int(x) for x in args.rotate.split(","))
    cold = run_prefill(tbv, torch, synth, st, args.steps, args.warmup, h_nslot, h_nbuf, env=henv, long_steps=long_steps, fit_region=True)
    if args.calibrate_copy:
        src = torch.empty(N_PREFILL, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(args.calibrate_copy):
            dst.copy_(src)
        torch.cuda.synchronize()

    ach = None
    if "achievable" in legs:
        try:
            ach = run_achievable(tbv)
        except Exception as e:                  # noqa: BLE001 - the headline does not depend on it
            print(f"bench.py: achievable leg failed: {type(e).__name__}: {e}", file=sys.stderr)
    ceiling = ach["copy_1GiB"]["GBps"] if ach else None
    alg_step = (4 if fused_headline else 5) * n
    ms = cold["wall"] / args.steps * 1e3
    dom_kernel = "sum" if two_headline else ("pack+sum fused" if fused_headline else "pack+sum merged launch")
    dom_bytes = 3 * n if two_headline else alg_step
    # One launch per step (merged, fused): the launch's average duration is measured live inside the timed region, by two
    # events on the caller's stream around the launches that follow the first one (device time / (steps - 1)).  The
    # dispatch timestamps of every single launch (a further pass, what rocprofv3's kernel trace averages too) are
    # reported beside it: a dispatch is stamped as started when its packet is taken up, while its predecessor still
    # drains, so their mean reads 0.1-0.5 us longer than the step.
    traffic_kernel = "k_step_sum" if two_headline else ("k_step_pack_sum" if fused_headline else "k_merged")
    traffic = traffic_from_profile(traffic_kernel)
    if two_headline:
        roof = kernel_roofline(dom_bytes, cold["sum_us"], cold["sum_min_us"], cold["n_sum"], ceiling) or {}
        timing = "dispatch timestamps of every sum launch in a further pass of the same steps"
    else:
        roof = kernel_roofline(dom_bytes, cold["ev_us"] or cold["sum_us"], cold["sum_min_us"], max(args.steps - 1, 1), ceiling) or {}
        roof["avg_launch_us_regions"] = [round(x, 3) for x in cold["ev_runs"]]
        roof["per_dispatch_timestamps"] = {"avg_us": round(cold["sum_us"], 3), "min_us": round(cold["sum_min_us"], 3), "launches": cold["n_sum"],
                                           "frac": round(dom_bytes / (cold["sum_us"] * 1e-6) / HBM_PEAK, 4) if cold["sum_us"] else None}
        timing = ("avg_launch_us: the timed region run again right after the host-clocked one, with two events on the caller's stream "
                  "around the launches after the first, device time / (steps - 1); median of the regions listed in avg_launch_us_regions "
                  "(the event records cost a region about 10 us, so they stay out of the host-clocked one); per_dispatch_timestamps: start and end stamps of every launch in a further pass "
                  "(what a kernel trace averages)")
    roof["denominator"] = ("4N: the local tensor is read once" if fused_headline else "3N (sum kernel alone)" if two_headline else
                           "5N = pack 2N + sum 3N algorithmic bytes; the sum blocks' read of the local tensor is issued but served by the L2, see frac_fabric")
    if traffic and roof.get("avg_launch_us"):
        roof["frac_fabric"] = round(traffic / (roof["avg_launch_us"] * 1e-6) / HBM_PEAK, 4)
        roof["fabric_GBps"] = round(traffic / (roof["avg_launch_us"] * 1e-6) / 1e9, 1)
        roof["fabric_denominator"] = "bytes that crossed the fabric per launch by FETCH_SIZE + WRITE_SIZE (4.0 N for the merged launch)"
        if ceiling:
            roof["frac_fabric_of_measured_copy_ceiling"] = round(traffic / (roof["avg_launch_us"] * 1e-6) / 1e9 / ceiling, 4)
    pavg = avg_from_profile(traffic_kernel)
    if pavg and roof.get("avg_launch_us"):
        roof["profile_avg_launch_us"] = round(pavg, 3)
        roof["profile_frac"] = round(dom_bytes / (pavg * 1e-6) / HBM_PEAK, 4)
        roof["profile_source"] = TRACE_FILE
    line = {
        "metric": "reduce-copy GB/s at 16MB bf16", "value": round(alg_step / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "prefill all-reduce step, bf16 [2048x4096] = 16 MiB local + peer payload pre-staged in the receive "
                               "slots; values N(0,0.02^2) with 0.1% outliers at +-8; cache-cold: 16 ring slots and 12 rotating "
                               "local/output tensors (896 MiB touched in turn, beyond the 256 MB Infinity Cache)",
                   "step": "one kernel reading the local tensor once (4N)" if fused_headline else
                           ("pack kernel 2N + sum kernel 3N = 5N" if two_headline else
                            "pack 2N + sum 3N = 5N in one launch (pack blocks and sum blocks side by side)"),
                   "frac_of_peak": round(alg_step / (ms * 1e-3) / HBM_PEAK, 4),
                   "frac_of_peak_is": "value / 8 TB/s by the host clock over the timed region: it carries the region's fixed cost "
                                      "(region.fixed_us / steps per step) on top of the launch average in roofline.avg_launch_us",
                   "frac_of_measured_copy_ceiling": round(alg_step / (ms * 1e-3) / 1e9 / ceiling, 4) if ceiling else None,
                   "nslot": h_nslot, "rotating_tensors": h_nbuf, "rails": 2, "accumulate": "f32, round to nearest even", "bit_exact_vs_torch_add": cold["ok"],
                   "untimed_warmup_steps": own_warmup(args.warmup, h_nslot, h_nbuf) + 2 * min(args.steps, 48),
                   "host_enqueue_us_per_call": round(cold["enq_us"], 2),
                   "host_enqueue_is": "median host time of a call in a burst of 12 on a drained stream, by the caller's clock around the ctypes call "
                                      "(staged legs: the library's own average of the time inside tbv_ar_allreduce)",
                   "headline_env": dict(henv)},
        "roofline": dict({"bound": "hbm", "kernel": dom_kernel, "peak": HBM_PEAK / 1e9}, **roof,
                         traffic=traffic, traffic_source=(TRAFFIC_FILE if traffic else None),
                         timing=timing),
    }
    if cold["region"]:
        line["region"] = cold["region"]
        line["region"]["steady_value_GBps"] = round(alg_step / (cold["region"]["per_step_us"] * 1e-6) / 1e9, 1)
        line["region"]["steady_frac_of_peak"] = round(alg_step / (cold["region"]["per_step_us"] * 1e-6) / HBM_PEAK, 4)
    if two_headline:
        line["kernels"] = {"pack": kernel_roofline(2 * n, cold["pack_us"], cold["pack_min_us"], cold["n_pack"], ceiling)}
    if cold["long_wall"]:
        lms = cold["long_wall"] / cold["long_steps"] * 1e3
        line["long_run"] = {"steps": cold["long_steps"], "ms_per_step": round(lms, 5), "value": round(alg_step / (lms * 1e-3) / 1e9, 1),
                            "unit": "GB/s", "frac_of_peak": round(alg_step / (lms * 1e-3) / HBM_PEAK, 4),
                            "avg_launch_us": round(cold["ev_long_us"], 3) if cold["ev_long_us"] else None,
                            "what": "the same leg over 2000 steps in one region (host clock; and the in-region event average)"}
    if ach:
        line["achievable"] = ach
    sub_steps = min(max(args.steps, 500), 2000)
    line["comparison_legs"] = (f"the legs below that repeat the 16 MiB step in another form run {sub_steps} steps per region; their "
                               "ms_per_step is the host clock over the best of three such regions (the headline's value is "
                               "one region of exactly --steps steps)")

    def leg(name, fn):
        """One extra leg; a failure is recorded in the line instead of costing the headline its output."""
        try:
            fn()
        except Exception as e:              # noqa: BLE001 - whatever it was, say so and go on
            line.setdefault("leg_errors", {})[name] = f"{type(e).__name__}: {e}"
            try:
                tbv.shutdown()
            except Exception:               # noqa: BLE001
                pass

    def leg_two():
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, env=(("TBV_MERGE", 0),))
        rms = r["wall"] / sub_steps * 1e3
        line["cold_two_launches"] = {"what": "the same cache-cold step as a pack kernel then a sum kernel (TBV_MERGE=0), 5N", "steps": sub_steps,
                                     "ms_per_step": round(rms, 5), "value": round(5 * n / (rms * 1e-3) / 1e9, 1), "unit": "GB/s",
                                     "frac_of_peak": round(5 * n / (rms * 1e-3) / HBM_PEAK, 4), "bit_exact": r["ok"],
                                     "pack": kernel_roofline(2 * n, r["pack_us"], r["pack_min_us"], r["n_pack"], ceiling),
                                     "sum": kernel_roofline(3 * n, r["sum_us"], r["sum_min_us"], r["n_sum"], ceiling)}

    if "two" in legs and not two_headline:
        leg("two", leg_two)

    def leg_fused():
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, env=(("TBV_FUSE", 1),))
        rms = r["wall"] / sub_steps * 1e3
        line["cold_fused_4N"] = {"what": "the same cache-cold step as one kernel that reads the local tensor once (TBV_FUSE=1); "
                                         "its algorithmic bytes are 4N", "steps": sub_steps,
                                 "ms_per_step": round(rms, 5), "value": round(4 * n / (rms * 1e-3) / 1e9, 1), "unit": "GB/s",
                                 "frac_of_peak": round(4 * n / (rms * 1e-3) / HBM_PEAK, 4), "bit_exact": r["ok"],
                                 "kernel": kernel_roofline(4 * n, r["sum_us"], r["sum_min_us"], r["n_sum"], ceiling)}

    if "fused" in legs and not fused_headline:
        leg("fused", leg_fused)

    def leg_inplace():
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, inplace=True)
        rms = r["wall"] / sub_steps * 1e3
        line["cold_in_place"] = {"what": "the same cache-cold step in place (the reference's outp == NULL: the output is the local tensor). "
                                         "Library default: the fused body (one lane loads a vector once and does both stores), 4N", "steps": sub_steps,
                                 "ms_per_step": round(rms, 5), "value": round(4 * n / (rms * 1e-3) / 1e9, 1), "unit": "GB/s",
                                 "frac_of_peak": round(4 * n / (rms * 1e-3) / HBM_PEAK, 4), "bit_exact": r["ok"],
                                 "kernel": kernel_roofline(4 * n, r["sum_us"], r["sum_min_us"], r["n_sum"], ceiling)}

    if "fused" in legs:
        leg("inplace", leg_inplace)

    def leg_staged():
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, staged=True)
        rms = r["wall"] / sub_steps * 1e3
        line["cold_staged"] = {"what": "the same cache-cold step when the peer's payload is NOT in the receive slot at the call: it is handed to the emulated "
                                       "wire per call (deposit kernel on a side stream + 64-bit flag after this call's pack completion word); one launch "
                                       "per call: pack blocks, then sum blocks that poll the flag inside the kernel.  Calls on one stream run one after "
                                       "the other, so every step pays the whole emulated chain (pack's word seen by the host, deposit launched and run, "
                                       "arrival seen, flag raised and seen by the waiting kernel) beside its own 5N",
                               "steps": sub_steps, "ms_per_step": round(rms, 5), "value": round(5 * n / (rms * 1e-3) / 1e9, 1), "unit": "GB/s",
                               "bit_exact": r["ok"], "host_enqueue_us_per_call": round(r["enq_us"], 2),
                               "kernel": kernel_roofline(5 * n, r["sum_us"], r["sum_min_us"], r["n_sum"]),
                               "kernel_note": "the launch's duration includes the time its sum blocks wait for the flag"}
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, env=(("TBV_FORCEGATE", 1),))
        rms = r["wall"] / sub_steps * 1e3
        line["cold_gated_flag_up"] = {"what": "the staged call's launch (pack blocks + gated sum blocks) with its flag already up when the kernel starts "
                                              "(TBV_FORCEGATE=1 on the early-peer workload): what the gate's bounded grid costs against the headline's "
                                              "ungated merged launch",
                                      "steps": sub_steps, "ms_per_step": round(rms, 5), "value": round(5 * n / (rms * 1e-3) / 1e9, 1), "unit": "GB/s",
                                      "frac_of_peak": round(5 * n / (rms * 1e-3) / HBM_PEAK, 4), "bit_exact": r["ok"],
                                      "host_enqueue_us_per_call": round(r["enq_us"], 2),
                                      "kernel": kernel_roofline(5 * n, r["ev_us"] or r["sum_us"], r["sum_min_us"], sub_steps - 1, ceiling)}
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, env=(("TBV_STAGEDMERGE", 0),), staged=True)
        rms = r["wall"] / sub_steps * 1e3
        line["cold_staged_three_launches"] = {"what": "cold_staged in the reference's launch sequence: pack kernel, hipStreamWaitValue64, sum kernel (TBV_STAGEDMERGE=0)",
                                              "steps": sub_steps, "ms_per_step": round(rms, 5), "bit_exact": r["ok"],
                                              "host_enqueue_us_per_call": round(r["enq_us"], 2),
                                              "pack": kernel_roofline(2 * n, r["pack_us"], r["pack_min_us"], r["n_pack"]),
                                              "sum": kernel_roofline(3 * n, r["sum_us"], r["sum_min_us"], r["n_sum"])}

    if "staged" in legs:
        leg("staged", leg_staged)

    def leg_resident():
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, 4, 1)
        rms = r["wall"] / sub_steps * 1e3
        line["resident"] = {"bound": "infinity-cache",
                            "what": "the same step with 4 ring slots and one local/output tensor: everything it touches (160 MiB) stays "
                                    "in the 256 MB Infinity Cache, so this is a cache figure, not an HBM one",
                            "steps": sub_steps, "ms_per_step": round(rms, 5), "value": round(5 * n / (rms * 1e-3) / 1e9, 1), "unit": "GB/s",
                            "bit_exact": r["ok"], "kernel": kernel_roofline(5 * n, r["sum_us"], r["sum_min_us"], r["n_sum"])}

    if "resident" in legs:
        leg("resident", leg_resident)

    def leg_decode():
        line["decode_latency"] = run_decode(tbv, torch, synth, st, args.decode_iters, fusewait=True)
        line["decode_latency_stream_gate"] = run_decode(tbv, torch, synth, st, args.decode_iters, fusewait=False)

    if "decode" in legs:
        leg("decode", leg_decode)

    def leg_host():
        line["host_cost_per_call"] = run_host_cost(tbv, torch, synth, st)
        if "decode_latency" in line:      # the decode loop above runs back to back: its enqueue time includes waits for ring room
            idle = line["host_cost_per_call"]["8KB"]["idle"]
            line["decode_latency"]["host_enqueue_idle_us"] = idle["enqueue_us"]
            line["decode_latency"]["host_post_idle_us"] = idle["post_us"]

    if "host" in legs:
        leg("host", leg_host)

    def leg_pipeline():
        line["pipeline_64MiB_fp16"] = run_pipeline(tbv, torch, synth, st)

    if "pipeline" in legs:
        leg("pipeline", leg_pipeline)

    def leg_codec():
        img = 2176 * ((n // 2 + 2047) // 2048)
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, env=(("TBV_CODEC", 1),), check="codec")
        rms = r["wall"] / sub_steps * 1e3
        line["cold_int8_codec"] = {"what": "the same cache-cold step with the int8 payload codec (TBV_CODEC=1; group 128, asymmetric; off by default). "
                                           "The peer's image is in place, so the step is ONE kernel: read the local tensor, write its image, read "
                                           "the peer's image, write the sum of the two decodes (N + 0.53 N + 0.53 N + N = 3.06 N)",
                                   "steps": sub_steps, "ms_per_step": round(rms, 5), "wire_bytes": img, "wire_fraction_of_payload": round(img / n, 4),
                                   "result_within_half_step_of_each_operand": r["ok"],
                                   "kernel": kernel_roofline(2 * n + 2 * img, r["sum_us"], r["sum_min_us"], r["n_sum"], ceiling)}
        r = run_prefill(tbv, torch, synth, st, sub_steps, args.warmup, COLD_NSLOT, COLD_NBUF, env=(("TBV_CODEC", 1), ("TBV_MERGE", 0)), check="codec")
        line["cold_int8_codec"]["two_launches"] = {
            "what": "the quantise kernel (N + 0.53 N) followed by the dequantising sum, which reads this rank's own image back (2 x 0.53 N + N): "
                    "what a call whose peer image is not there yet takes (TBV_MERGE=0 here)",
            "ms_per_step": round(r["wall"] / sub_steps * 1e3, 5), "result_within_half_step_of_each_operand": r["ok"],
            "pack": kernel_roofline(n + img, r["pack_us"], r["pack_min_us"], r["n_pack"], ceiling),
            "sum": kernel_roofline(n + 2 * img, r["sum_us"], r["sum_min_us"], r["n_sum"], ceiling)}

    def leg_codec_accuracy():
        line["cold_int8_codec"]["accuracy"] = run_codec_accuracy(tbv, torch, synth, st)

    if "codec" in legs:
        leg("codec", leg_codec)
        if "cold_int8_codec" in line:
            leg("codec_accuracy", leg_codec_accuracy)

    def leg_rmsnorm():
        line["sum_rmsnorm_fusion"] = run_rmsnorm_fusion(tbv, torch, synth, st)

    if "rmsnorm" in legs:
        leg("rmsnorm", leg_rmsnorm)

    def leg_cpu():
        line["cpu_baseline"] = run_cpu_baseline(torch, synth)

    if "cpu" in legs:
        leg("cpu", leg_cpu)
    print(json.dumps(line), flush=True)
    if not cold["ok"]:
        sys.exit(1)


if __name__ == "__main__":
    main()
