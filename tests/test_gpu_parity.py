"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle.

The first two tests are this build's counterparts of the reference's own drivers
(step4/test_exact.py, step4/test_stress.py): same structure, same equality checks,
with the second rank replaced by the emulated peer.  Integer and floating point
results must match the oracle bit for bit (the sum is a correctly rounded
operation: there is no tolerance).
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from gpu_util import DT, bits_np, dev, first_diff, same_bits, say, session
from libtbvcoll_amd import synth

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def oracle_sum(orc, a, b):
    return orc.sum_torch(a.cpu(), b.cpu())


# ---------------------------------------------------------------- counterpart of step4/test_exact.py

@pytest.mark.parametrize("mode", ["async", "sync"])
def test_exact(orc, mode):
    env = {"TBV_ASYNC": 0} if mode == "sync" else {}
    with session(rails=2, cap=4 << 20, **env) as tbv:
        assert tbv.is_async() == (mode == "async")
        for name in ("f32", "bf16", "f16"):
            dt = DT[name]
            for nb in (57344, 229376, 1048576):
                say("exact", mode, name, nb)
                numel = nb // torch.tensor([], dtype=dt).element_size()
                f0 = synth.uniform(1234, numel, -5.0, 5.0)
                f1 = synth.uniform(1235, numel, -5.0, 5.0)
                mine, peer = dev(f0, dt), dev(f1, dt)
                out = torch.empty_like(mine)
                tbv.stage_peer(peer)
                assert tbv.all_reduce(mine.clone(), out), f"{name} {nb} not handled"
                torch.cuda.synchronize()
                ref_dt = mine + peer                                    # same arithmetic, torch's kernel
                ref_32 = (mine.float() + peer.float()).to(dt)           # single rounding from fp32
                assert torch.equal(out, ref_dt) and torch.equal(out, ref_32)
                assert first_diff(out, oracle_sum(orc, mine, peer)) is None
        assert not tbv.err()


# ---------------------------------------------------------------- counterpart of step4/test_stress.py

@pytest.mark.parametrize("name,nb,rails,iters", [("bf16", 57344, 2, 2000), ("f16", 229376, 2, 2000), ("f32", 8192, 1, 2000),
                                                 ("bf16", 8192, 1, 10000)])     # last: the decode config, NSLOT=4, CAP=8 KB
def test_stress_back_to_back(orc, name, nb, rails, iters):
    dt = DT[name]
    numel = nb // torch.tensor([], dtype=dt).element_size()
    with session(rails=rails, cap=nb, TBV_NSLOT=4) as tbv:
        say("stress", name, nb, "iters", iters)

        def gen(it, r):
            return synth.torch_hash_uniform(it * 2 + r, numel, -5.0, 5.0).to(dt)

        outs, ins, peers = [], [], []
        for it in range(iters):
            x, p = gen(it, 0), gen(it, 1)
            out = torch.empty_like(x)
            tbv.stage_peer(p)
            assert tbv.all_reduce(x, out)
            outs.append(out); ins.append(x); peers.append(p)      # keep inputs alive: no allocator reuse
        torch.cuda.synchronize()
        bad = [it for it in range(iters) if not torch.equal(outs[it], gen(it, 0) + gen(it, 1))]
        assert not bad, f"{len(bad)}/{iters} mismatching calls, first {bad[0]}"
        for it in range(0, iters, 97):                             # and a sample against the CPU oracle
            assert first_diff(outs[it], oracle_sum(orc, ins[it], peers[it])) is None
        # the device-side generator gives what the host generator gives
        assert np.array_equal(synth.torch_hash_uniform(7, 1000, -5.0, 5.0).cpu().numpy(), synth.uniform(7, 1000, -5.0, 5.0))
        assert not tbv.err()


# ---------------------------------------------------------------- golden vectors through the GPU

def test_config1_golden_on_gpu(orc):
    g = np.load(os.path.join(G, "c1_bf16_4096.npz"))
    a = torch.from_numpy(g["a"].view(np.int16)).view(torch.bfloat16).cuda()
    b = torch.from_numpy(g["b"].view(np.int16)).view(torch.bfloat16).cuda()
    with session(rails=1, cap=8192) as tbv:
        out = torch.empty_like(a)
        tbv.stage_peer(b)
        assert tbv.all_reduce(a, out)
        torch.cuda.synchronize()
        assert np.array_equal(bits_np(out), g["out"])


@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
def test_edge_golden_on_gpu(orc, name):
    """Zeros, subnormals, ties, overflow to Inf: the committed edge cases."""
    g = np.load(os.path.join(G, f"edge_{name}.npz"))
    if name == "f32":
        a = torch.from_numpy(g["a"].view(np.float32).copy()).cuda(); b = torch.from_numpy(g["b"].view(np.float32).copy()).cuda()
    else:
        a = torch.from_numpy(g["a"].view(np.int16)).view(DT[name]).cuda()
        b = torch.from_numpy(g["b"].view(np.int16)).view(DT[name]).cuda()
    with session(rails=1, cap=1 << 20) as tbv:
        out = torch.empty_like(a)
        tbv.stage_peer(b)
        assert tbv.all_reduce(a, out)
        torch.cuda.synchronize()
        got, want = bits_np(out), g["out"]
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, [(hex(int(bits_np(a)[i])), hex(int(bits_np(b)[i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:5]]


# ---------------------------------------------------------------- shapes the reference's callers can produce

@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
def test_ragged_sizes_inplace_and_offsets(orc, name):
    dt = DT[name]
    esz = torch.tensor([], dtype=dt).element_size()
    with session(rails=2, cap=1 << 20, TBV_RAIL1MAX=4096) as tbv:
        for numel in (1, 2, 3, 7, 8, 9, 63, 64, 65, 511, 4097, 8191, 30001, (1 << 20) // esz):
            for off in (0, 1, 3):                       # element offsets: caller pointers that are not 16-byte aligned
                say("ragged", name, numel, "off", off)
                base_a = dev(synth.normal(numel * 3 + off, numel + 8), dt)
                base_o = torch.zeros(numel + 8, dtype=dt, device="cuda")
                if numel + off > base_a.numel() or (numel + off) * esz > tbv.cap():
                    continue
                a = base_a[off:off + numel]
                o = base_o[off:off + numel]
                p = dev(synth.normal(numel * 5 + 1, numel), dt)
                want = oracle_sum(orc, a, p)
                tbv.stage_peer(p)
                assert tbv.all_reduce(a, o)
                torch.cuda.synchronize()
                assert first_diff(o, want) is None, (numel, off)
                assert float(base_o[:off].abs().sum()) == 0 and float(base_o[off + numel:].abs().sum()) == 0   # no overrun
                tbv.stage_peer(p)                       # in place (out=None)
                a2 = a.clone() if off == 0 else base_a.clone()[off:off + numel]
                assert tbv.all_reduce(a2)
                torch.cuda.synchronize()
                assert first_diff(a2, want) is None, ("inplace", numel, off)
        assert not tbv.err()


def test_guards_and_return_codes(orc):
    with session(rails=2, cap=5000) as tbv:
        assert tbv.cap() == 8192                                     # rounded up to 4096
        t = torch.zeros(8192 // 2 + 1, dtype=torch.bfloat16, device="cuda")
        assert tbv.all_reduce(t) is False                            # over the cap: caller falls back
        assert tbv.all_reduce(torch.zeros(0, dtype=torch.float32, device="cuda")) is True
        assert tbv.all_reduce(torch.zeros(4, dtype=torch.float64, device="cuda")) is False
        assert tbv.all_reduce(torch.zeros(4, dtype=torch.float32)) is False          # not on the GPU
        assert tbv.all_reduce(torch.zeros(8, 8, device="cuda")[:, ::2]) is False     # not contiguous
        x = torch.ones(16, device="cuda")
        assert tbv.all_reduce(x, torch.empty(15, device="cuda")) is False
        assert tbv.all_reduce(x, torch.empty(16, device="cuda", dtype=torch.float16)) is False
        fn = tbv.raw_fn()
        st = torch.cuda.current_stream().cuda_stream
        assert fn(ctypes.c_void_p(t.data_ptr()), None, 8194, 2, ctypes.c_void_p(st)) == -2
        assert fn(ctypes.c_void_p(x.data_ptr()), None, 64, 7, ctypes.c_void_p(st)) == -1   # unknown dtype
        assert tbv.seq() == 0                                        # nothing above consumed a sequence number
        # init is idempotent: a second call changes nothing
        assert tbv.lib().tbv_ar_init(1, b"a,b,c", b"", 1, 1 << 20) == 0 and tbv.lib().tbv_ar_cap() == 8192
        # an empty call through the raw C function (the Python wrapper answers those itself): it takes a sequence
        # number like any other call, touches nothing and leaves no error behind, in every launch form
        keep = x.clone()
        for k in range(1, 7):
            assert fn(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(x.data_ptr()), 0, k % 3, ctypes.c_void_p(st)) == 0
            assert tbv.seq() == k
        torch.cuda.synchronize()
        assert torch.equal(x, keep) and not tbv.err()
    for env in ({"TBV_ONEKERNEL": 0}, {"TBV_FUSEWAIT": 0, "TBV_DEFERSIG": 0, "TBV_ONEKERNEL": 0}, {"TBV_ASYNC": 0}):
        with session(rails=2, cap=8192, **env) as tbv:
            fn = tbv.raw_fn()
            x = torch.ones(16, device="cuda"); keep = x.clone()
            for k in range(1, 6):
                say("empty call", env, k)
                assert fn(ctypes.c_void_p(x.data_ptr()), None, 0, 0, ctypes.c_void_p(st)) == 0
            tbv.stage_peer(keep)
            assert tbv.all_reduce(x)                                   # and the ring goes on working after them
            torch.cuda.synchronize()
            assert torch.equal(x, keep + keep) and not tbv.err() and tbv.seq() == 6


def test_mirror_mode_and_send_slot_image(orc):
    """With no peer payload staged the peer echoes this rank's send slot: out = in + in,
    which exercises pack -> completion word -> side-stream read of the bounce slot."""
    with session(rails=2, cap=1 << 20, TBV_RAIL1MAX=16384) as tbv:
        for name in ("bf16", "f16", "f32"):
            dt = DT[name]
            for numel in (5, 4096, 100003):
                say("mirror", name, numel)
                a = dev(synth.uniform(numel, numel, -3.0, 3.0), dt)
                out = torch.empty_like(a)
                assert tbv.all_reduce(a, out)
                torch.cuda.synchronize()
                assert first_diff(out, oracle_sum(orc, a, a)) is None
                slot = tbv.seq() % tbv.lib().tbv_emu_nslot()
                nb = a.numel() * a.element_size()
                img = torch.empty(nb, dtype=torch.uint8, device="cuda")
                hip = ctypes.CDLL("libamdhip64.so.7")                # the runtime torch already loaded
                hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
                assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(slot), nb, 3) == 0
                want = orc.pack(a.cpu().contiguous().view(torch.uint8).numpy())
                assert np.array_equal(img.cpu().numpy(), want)


# ---------------------------------------------------------------- counterpart of step4/test_tbvcoll.py

def test_latency_and_phase_breakdown(orc, capfd):
    """In place on constant rank+1 tensors (1.0 here, 2.0 from the peer -> 3.0), 30 warm-up calls,
    then timed calls per size; the phase averages and the stderr dumps behave as the reference's:
    per-call averages, reset on read, histogram by log2 size, per-rail lines."""
    import re
    import time
    sizes = [4096, 57344, 229376, 1048576]
    iters = 300
    with session(rails=2, cap=max(sizes)) as tbv:
        for dt in (torch.float32, torch.bfloat16):
            for nb in sizes:
                numel = nb // torch.tensor([], dtype=dt).element_size()
                peer = torch.full((numel,), 2.0, dtype=dt, device="cuda")
                tbv.stage_peer_repeat(peer)
                t = torch.full((numel,), 1.0, dtype=dt, device="cuda")
                for _ in range(30):
                    assert tbv.all_reduce(t)
                    t.fill_(1.0)
                torch.cuda.synchronize()
                tbv.stats4()
                t0 = time.perf_counter()
                for _ in range(iters):
                    tbv.all_reduce(t)
                    t.fill_(1.0)
                torch.cuda.synchronize()
                tot = (time.perf_counter() - t0) / iters
                pre, xfer, post, enq, n = tbv.stats4()
                assert n == iters and pre == 0.0 and 0 < xfer < 5e4 and 0 < post < enq < 1e4
                assert tbv.stats4() == (0.0, 0.0, 0.0, 0.0, 0)          # reading resets
                c = torch.full((numel,), 1.0, dtype=dt, device="cuda")
                assert tbv.all_reduce(c)
                torch.cuda.synchronize()
                assert torch.equal(c, torch.full_like(c, 3.0))           # exactly 3, not just close to it
                say("phases", dt, nb, f"total {tot * 1e6:.1f} us enq {enq:.1f} xfer {xfer:.1f} post {post:.1f} "
                    f"algbw {nb * 8 / tot / 1e9:.2f} Gb/s")
        capfd.readouterr()
        tbv.rails()
        tbv.hist()
        err = capfd.readouterr().err
        calls_per_size = 2 * (30 + iters + 1)
        # sizes 4096 and 57344 travel on one rail, the larger two on both
        assert re.search(r"rail0: post +[\d.]+ +arrival +[\d.]+ +\(%d calls\)" % (4 * calls_per_size), err), err
        assert re.search(r"rail1: post +[\d.]+ +arrival +[\d.]+ +\(%d calls\)" % (2 * calls_per_size), err), err
        for nb, rails in ((4096, 1.0), (57344, 1.0), (229376, 2.0), (1048576, 2.0)):
            bucket = 1 << (nb.bit_length() - 1)
            m = re.search(r" +%d B~ : +(\d+) calls  mean +[\d.]+ us  mean rails ([\d.]+)" % bucket, err)
            assert m and int(m.group(1)) == calls_per_size and float(m.group(2)) == rails, (nb, err)
        tbv.hist()
        assert " B~ :" not in capfd.readouterr().err                      # the dump reset the histogram
        tbv.stage_peer_repeat(None)


@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
def test_nan_and_inf_propagation(orc, name):
    """NaN in -> NaN out, Inf - Inf -> NaN, Inf + finite -> Inf: the positions must agree with the oracle and all
    non-NaN results must match it bit for bit.  Which NaN comes out (payload, sign) is not pinned."""
    dt = DT[name]
    n = 4096
    a = synth.normal(3, n); b = synth.normal(4, n)
    a[::7] = np.inf; b[::11] = -np.inf; a[5::13] = np.nan; b[9::17] = np.nan; a[::77] = -np.inf
    ta, tb = dev(a, dt), dev(b, dt)
    with session(rails=1, cap=1 << 20) as tbv:
        out = torch.empty_like(ta)
        tbv.stage_peer(tb)
        assert tbv.all_reduce(ta, out)
        torch.cuda.synchronize()
        want = oracle_sum(orc, ta, tb)
        nan = torch.isnan(want)
        assert int(nan.sum()) > 400 and torch.equal(torch.isnan(out.cpu()), nan)
        if name == "f32":
            g, w = out.cpu().numpy().view(np.uint32), want.numpy().view(np.uint32)
        else:
            g, w = bits_np(out), bits_np(want)
        keep = ~nan.numpy()
        assert np.array_equal(g[keep], w[keep])
        assert int(torch.isinf(out).sum()) > 500


def test_one_gibibyte_calls(orc):
    """The largest sizes: 1 GiB calls (two rails of 512 MiB each, 64 Mi vectors per kernel) in two dtypes, in place and
    out of place, and 1.5 GiB as two pipelined chunks.  Checked in full against the GPU's own add (bit-identical for
    these types) and on both ends of the tensor against the CPU restatement."""
    n = 1 << 30
    with session(rails=2, cap=n, TBV_NSLOT=2) as tbv:
        assert tbv.cap() == n
        for name in ("bf16", "f32"):
            dt = DT[name]
            numel = n // torch.empty(0, dtype=dt).element_size()
            g = torch.Generator(device="cuda"); g.manual_seed(77)
            a = (torch.rand(numel, device="cuda", generator=g) * 8 - 4).to(dt)
            b = (torch.rand(numel, device="cuda", generator=g) * 8 - 4).to(dt)
            want = a + b
            out = torch.empty_like(a)
            say("1 GiB", name, "out of place")
            tbv.stage_peer(b); assert tbv.all_reduce(a, out)
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int32), want.view(torch.int32)), name
            k = 1 << 20
            for sl in (slice(0, k), slice(numel - k, numel)):
                assert first_diff(out[sl], oracle_sum(orc, a[sl], b[sl])) is None, name
            say("1 GiB", name, "in place")
            x = a.clone()
            tbv.stage_peer(b); assert tbv.all_reduce(x)
            torch.cuda.synchronize()
            assert torch.equal(x.view(torch.int32), want.view(torch.int32)), name
            if name == "bf16":
                # the peer's payload already in place: four merged launches of 256 MiB each (in place: the fused body)
                say("1 GiB", name, "early peer")
                tbv.peer_resident(b)
                out.zero_()
                assert tbv.all_reduce(a, out)
                x = a.clone()
                assert tbv.all_reduce(x)
                torch.cuda.synchronize()
                assert torch.equal(out.view(torch.int32), want.view(torch.int32)), "early peer"
                assert torch.equal(x.view(torch.int32), want.view(torch.int32)), "early peer, in place"
                tbv.peer_resident(None)
            del x, out, want
        # 1.5 GiB over the 1 GiB cap: two chunks through the pipeline entry point
        numel = 3 * (n // 4)
        a = (torch.rand(numel, device="cuda") * 8 - 4).to(torch.bfloat16)
        b = (torch.rand(numel, device="cuda") * 8 - 4).to(torch.bfloat16)
        out = torch.empty_like(a)
        per = n // 2
        say("1.5 GiB chunked")
        tbv.stage_peer(b[:per]); tbv.stage_peer(b[per:])
        assert tbv.all_reduce(a, out) is False                   # over the cap: the plain call declines
        assert tbv.all_reduce_chunked(a, out)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), (a + b).view(torch.int16))
        assert not tbv.err()
