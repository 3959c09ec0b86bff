#!/usr/bin/env python3
"""Benchmark of the all-reduce data path on one MI355X.

A step is one tbv_ar_allreduce call through the C ABI on the 16 MiB bf16 prefill
workload with the peer's payload already resident in the receive slots: pack copy
into the uncached send bounce (with completion word), the 64-bit flag wait, the
sum kernel into the output.  Algorithmic bytes per step are 5N (pack 2N + sum 3N).

Prints ONE JSON line.  Besides the throughput it carries
  roofline      the sum kernel (the dominant one) against the 8 TB/s HBM peak,
                timed with HIP events recorded on the caller's stream around every
                launch of a second pass of the same steps;
  cpu_baseline  the CPU oracle's restatement of the same step on the host cores;
  cache_cold    the same step with buffers rotated beyond the Infinity Cache;
  decode_latency  p50/p99 of (flag raised -> sum complete) for the 8 KB decode
                workload, 10,000 back-to-back calls: library default (flag polled
                inside the sum kernel) and, as decode_latency_stream_gate, gated by
                hipStreamWaitValue64 as the reference does.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12                      # MI355X HBM3E, bytes/s
# Bytes the sum kernel moves between L2 and memory per 16 MiB launch, from rocprofv3 counter runs of this
# command (profiles/prefill16MiB_pmc_fetch_write.txt): FETCH_SIZE 16407.5 KiB x 1.9972 (what the counter
# reads for a plain 16 MiB copy, 8203.5 KiB for 16384 KiB) + WRITE_SIZE 16384.0 KiB x 1.0.
SUM_TRAFFIC_BYTES = int((16407.5 * (16384.0 / 8203.5) + 16384.0) * 1024)
N_PREFILL = 16 << 20                   # 2048 x 4096 bf16
N_DECODE = 8192                        # 1 x 4096 bf16


def pct(xs, q):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, int(q * len(xs)))]


def run_prefill(tbv, torch, synth, st, steps, warmup, fuse, nslot=4, nbuf=1):
    """nslot=4, nbuf=1 is the workload as specified (everything a step touches, 160 MiB, fits the 256 MB
    Infinity Cache).  nslot=16 with nbuf=12 rotating local/out tensors touches 896 MiB in turn, so every
    step's operands come from HBM: the cache-cold figure."""
    n = N_PREFILL
    os.environ["TBV_NSLOT"] = str(nslot)
    os.environ["TBV_FUSE"] = "1" if fuse else "0"
    tbv.shutdown()
    tbv.init(0, "rail0,rail1", "", cap_bytes=n)
    a = torch.from_numpy(synth.prefill_activations(100, n // 2)).to(torch.bfloat16).cuda()
    b = torch.from_numpy(synth.prefill_activations(101, n // 2)).to(torch.bfloat16).cuda()
    out = torch.empty_like(a)
    locs = [a] + [a.clone() for _ in range(nbuf - 1)]
    outs = [out] + [torch.empty_like(a) for _ in range(nbuf - 1)]
    fn = tbv.raw_fn()
    ps = ctypes.c_void_p(st.cuda_stream)
    ptrs = [(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(o.data_ptr())) for x, o in zip(locs, outs)]
    tbv.peer_resident(b)               # the peer's payload sits in every receive slot before the clock starts
    counter = [0]

    def step():
        pa, po = ptrs[counter[0] % nbuf]
        counter[0] += 1
        rc = fn(pa, po, n, 2, ps)
        if rc != 0:
            raise RuntimeError(f"tbv_ar_allreduce rc={rc}")

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    want = a + b
    ok = all(bool(torch.equal(o, want)) for o in outs)    # the timed path computed the sum, bit for bit
    enq = tbv.stats4()[3]

    # second pass of the same steps with an event pair around every kernel launch
    ksteps = min(steps, 1000)
    tbv.kernel_timing(True)
    for _ in range(ksteps):
        step()
    n_pack, pack_us, pack_min = tbv.kernel_times(0)
    n_sum, sum_us, sum_min = tbv.kernel_times(1)
    tbv.kernel_timing(False)
    torch.cuda.synchronize()
    err = tbv.err()
    tbv.shutdown()
    return {"wall": wall, "ok": ok and not err, "enq_us": enq, "pack_us": pack_us, "pack_min_us": pack_min, "n_pack": n_pack,
            "sum_us": sum_us, "sum_min_us": sum_min, "n_sum": n_sum}


def run_decode(tbv, torch, synth, st, iters, fusewait):
    n = N_DECODE
    os.environ["TBV_NSLOT"] = "4"
    os.environ["TBV_FUSE"] = "0"
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
        t0 = time.perf_counter()
        for it in range(iters):
            k = it % npeer
            tbv.stage_peer(peers[k])
            if not tbv.all_reduce(locs[k], outs[k]):
                raise RuntimeError("decode call not handled")
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    lat = tbv.latencies()
    ok = all(bool(torch.equal(outs[k], locs[k] + peers[k])) for k in range(npeer)) and not tbv.err()
    tbv.latency_probe(False)
    tbv.shutdown()
    os.environ.pop("TBV_FUSEWAIT", None)
    os.environ.pop("TBV_DEFERSIG", None)
    os.environ.pop("TBV_ONEKERNEL", None)
    return {"p50_us": round(pct(lat, 0.50), 2), "p99_us": round(pct(lat, 0.99), 2), "min_us": round(min(lat), 2),
            "samples": len(lat), "us_per_call_wall": round(wall / iters * 1e6, 2), "bit_exact": ok,
            "gate": "one kernel per call: pack, completion word, flag poll, sum (library default up to 1 MiB)" if fusewait
            else "pack kernel, hipStreamWaitValue64, sum kernel (TBV_FUSEWAIT=0 TBV_DEFERSIG=0 TBV_ONEKERNEL=0)",
            "measured": "host clock: just before the progress thread raises the flag -> host sees the sum's done word"}


def run_cpu_baseline(torch, synth):
    """The oracle's restatement of the same step (memcpy pack + fp32-upcast sum, RNE) on the host cores."""
    from oracle import oracle
    n = N_PREFILL
    a = oracle.torch_bits(torch.from_numpy(synth.prefill_activations(100, n // 2)).to(torch.bfloat16)).copy()
    b = oracle.torch_bits(torch.from_numpy(synth.prefill_activations(101, n // 2)).to(torch.bfloat16)).copy()
    cores = max(1, min(16, os.cpu_count() or 1))
    t1 = oracle.time_reduce_copy(oracle.DT_BF16, a, b, 1, 2, 40)
    tn = oracle.time_reduce_copy(oracle.DT_BF16, a, b, cores, 5, 300)
    nd = N_DECODE
    da = oracle.torch_bits(torch.from_numpy(synth.normal(0, nd // 2)).to(torch.bfloat16)).copy()
    db = oracle.torch_bits(torch.from_numpy(synth.normal(1, nd // 2)).to(torch.bfloat16)).copy()
    td = oracle.time_reduce_copy(oracle.DT_BF16, da, db, 1, 100, 2000)
    return {"value": round(5 * n / tn / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "single_thread_GBps": round(5 * n / t1 / 1e9, 2), "decode_8KB_single_thread_us": round(td * 1e6, 2),
            "sample": f"16 MiB bf16 prefill step (pack 2N + sum 3N), median of 300 steps on {cores} threads "
                      f"(static contiguous partition) and of 40 steps on 1 thread; 8 KB decode step: median of 2000 on 1 thread"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--decode-iters", type=int, default=10000)
    ap.add_argument("--fuse", type=int, default=0, help="1: pack+sum in one kernel when the peer is resident (4N)")
    ap.add_argument("--calibrate-copy", type=int, default=0,
                    help="also run this many plain 16 MiB device copies (known 16 MiB read + 16 MiB written), "
                         "so a counter run of this command holds a kernel of known traffic to scale by")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-decode", action="store_true")
    ap.add_argument("--skip-cold", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1", file=sys.stderr)
        sys.exit(2)

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
    pre = run_prefill(tbv, torch, synth, st, args.steps, args.warmup, bool(args.fuse))
    if args.calibrate_copy:
        src = torch.empty(N_PREFILL, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(args.calibrate_copy):
            dst.copy_(src)
        torch.cuda.synchronize()
    n = N_PREFILL
    alg_step = (4 if args.fuse else 5) * n
    ms = pre["wall"] / args.steps * 1e3
    dom_bytes = (4 if args.fuse else 3) * n
    achieved = dom_bytes / (pre["sum_us"] * 1e-6) / 1e9 if pre["sum_us"] > 0 else 0.0
    line = {
        "metric": "reduce-copy GB/s at 16MB bf16", "value": round(alg_step / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "prefill all-reduce step, bf16 [2048x4096] = 16 MiB local + peer payload resident in the "
                               "receive slots; values N(0,0.02^2) with 0.1% outliers at +-8",
                   "step": "pack+sum fused (4N)" if args.fuse else "pack 2N + flag wait + sum 3N = 5N",
                   "nslot": 4, "rails": 2, "accumulate": "f32, round to nearest even", "bit_exact_vs_torch_add": pre["ok"],
                   "residency": "everything a step touches (local 16 + bounce ring 64 + receive ring 64 + out 16 MiB) fits the "
                                "256 MB Infinity Cache; cache_cold in this line is the same step with the buffers rotated beyond it",
                   "host_enqueue_us_per_call": round(pre["enq_us"], 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 4), "traffic": None if args.fuse else SUM_TRAFFIC_BYTES,
                     "kernel": "pack+sum" if args.fuse else "sum", "algorithmic_bytes": dom_bytes,
                     "avg_launch_us": round(pre["sum_us"], 3), "min_launch_us": round(pre["sum_min_us"], 3),
                     "launches": pre["n_sum"]},
        "kernels": {"pack": {"algorithmic_bytes": 2 * n, "avg_launch_us": round(pre["pack_us"], 3),
                             "min_launch_us": round(pre["pack_min_us"], 3), "launches": pre["n_pack"],
                             "GBps": round(2 * n / (pre["pack_us"] * 1e-6) / 1e9, 1) if pre["pack_us"] > 0 else None}},
    }
    if not args.skip_cold:
        cold = run_prefill(tbv, torch, synth, st, min(args.steps, 1000), min(args.warmup, 100), bool(args.fuse), nslot=16, nbuf=12)
        cms = cold["wall"] / min(args.steps, 1000) * 1e3
        line["cache_cold"] = {"what": "same step with NSLOT=16 and 12 rotating local/out tensors (896 MiB touched in turn, "
                                      "beyond the 256 MB Infinity Cache)",
                              "value": round(alg_step / (cms * 1e-3) / 1e9, 1), "unit": "GB/s", "ms_per_step": round(cms, 5),
                              "sum_avg_us": round(cold["sum_us"], 3), "pack_avg_us": round(cold["pack_us"], 3),
                              "sum_frac_of_peak": round(dom_bytes / (cold["sum_us"] * 1e-6) / HBM_PEAK, 4) if cold["sum_us"] else None,
                              "bit_exact": cold["ok"]}
    if not args.skip_decode:
        line["decode_latency"] = run_decode(tbv, torch, synth, st, args.decode_iters, fusewait=True)
        line["decode_latency_stream_gate"] = run_decode(tbv, torch, synth, st, args.decode_iters, fusewait=False)
    if not args.skip_cpu:
        line["cpu_baseline"] = run_cpu_baseline(torch, synth)
    print(json.dumps(line), flush=True)
    if not pre["ok"]:
        sys.exit(1)


if __name__ == "__main__":
    main()
