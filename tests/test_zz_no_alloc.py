"""The entry point that allocates nothing, tbv_step_noalloc, against the existing kernel entry points
(tbv_emu_run_pack for the bounce image, tbv_emu_run_sum for the output): bit-exact, on two calls in a
row, the second with a smaller input.  Named to be collected last."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import DT, bits_np, dev, say, session
from libtbvcoll_amd import synth

pytestmark = pytest.mark.gpu


def _hip():
    hip = ctypes.CDLL("libamdhip64.so.7")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    return hip


@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
def test_no_alloc_step_matches_existing_entry_points(orc, name):
    hip = _hip()
    dt = DT[name]
    esz = 4 if name == "f32" else 2
    cap = 8 << 20
    with session(rails=1, cap=cap, TBV_NSLOT=4) as tbv:
        lib = tbv.lib()
        st = torch.cuda.current_stream().cuda_stream
        words = torch.zeros(16, dtype=torch.int64).pin_memory()       # host-visible completion words
        pack_word = words.data_ptr()
        done_word = words.data_ptr() + 64
        seq = 0
        # two calls in a row on the same GPU (they share the built-in counters), the second smaller;
        # then a small one that takes the two-launch path, and the cached-bounce variant
        for numel, uncached in (((6 << 20) // esz + 4, 1), ((1 << 20) // esz + 12, 1), (2048 // esz, 1), ((3 << 20) // esz, 0)):
            nbytes = numel * esz
            a = dev(synth.normal(900 + numel % 97, numel), dt)
            b = dev(synth.normal(901 + numel % 89, numel), dt)
            # the existing entry points: pack into send slot 1, sum into out_ref
            out_ref = torch.empty_like(a)
            assert lib.tbv_emu_run_pack(a.data_ptr(), nbytes, 1, st) == 0
            assert lib.tbv_emu_run_sum(out_ref.data_ptr(), a.data_ptr(), b.data_ptr(), nbytes, tbv_dt(name), st) == 0
            torch.cuda.synchronize()
            img_ref = torch.empty_like(a)
            assert hip.hipMemcpy(img_ref.data_ptr(), lib.tbv_emu_send_slot(1), nbytes, 3) == 0
            # the entry point that allocates nothing: bounce = send slot 2 (uncached) or a plain tensor (cached)
            out = torch.full_like(a, 7.0)
            cached_bounce = torch.zeros(numel + 8, dtype=dt, device="cuda")
            bounce = lib.tbv_emu_send_slot(2) if uncached else cached_bounce.data_ptr()
            seq += 1
            say("no-alloc step", name, numel, "uncached bounce" if uncached else "cached bounce", "seq", seq)
            rc = lib.tbv_step_noalloc(out.data_ptr(), a.data_ptr(), b.data_ptr(), bounce, uncached, nbytes, tbv_dt(name),
                                      pack_word, done_word, seq, st)
            assert rc == 0
            torch.cuda.synchronize()
            img = torch.empty_like(a)
            assert hip.hipMemcpy(img.data_ptr(), bounce, nbytes, 3) == 0
            assert np.array_equal(bits_np(out), bits_np(out_ref)), (name, numel)
            assert np.array_equal(bits_np(img), bits_np(img_ref)), (name, numel)
            assert np.array_equal(bits_np(img), bits_np(a))
            assert int(words[0]) == seq and int(words[8]) == seq          # both completion words were raised
            # in place, without completion words
            c = a.clone()
            assert lib.tbv_step_noalloc(c.data_ptr(), c.data_ptr(), b.data_ptr(), bounce, uncached, nbytes, tbv_dt(name),
                                        None, None, seq, st) == 0
            torch.cuda.synchronize()
            assert np.array_equal(bits_np(c), bits_np(out_ref))
            # in place the bounce must still receive the ORIGINAL tensor (no sum block may run ahead of the pack)
            assert hip.hipMemcpy(img.data_ptr(), bounce, nbytes, 3) == 0
            assert np.array_equal(bits_np(img), bits_np(a)), (name, numel, "bounce image of the in-place call")
            # and the CPU oracle agrees with both entry points
            assert np.array_equal(bits_np(out), bits_np(orc.sum_torch(a.cpu(), b.cpu()))), (name, numel, "oracle")
        # limits and argument checks: clear errors, nothing launched
        a = dev(synth.normal(1, 64), dt); o = torch.empty_like(a)
        big = (1 << 30) + 16
        assert lib.tbv_step_noalloc(o.data_ptr(), a.data_ptr(), a.data_ptr(), lib.tbv_emu_send_slot(0), 1, big, tbv_dt(name), None, None, 1, st) == -2
        assert lib.tbv_step_noalloc(o.data_ptr(), a.data_ptr() + 2, a.data_ptr(), lib.tbv_emu_send_slot(0), 1, 64, tbv_dt(name), None, None, 1, st) == -1
        assert lib.tbv_step_noalloc(o.data_ptr(), a.data_ptr(), a.data_ptr(), lib.tbv_emu_send_slot(0), 1, 64, 9, None, None, 1, st) == -1
        assert lib.tbv_step_noalloc(o.data_ptr(), a.data_ptr(), a.data_ptr(), lib.tbv_emu_send_slot(0), 1, 0, tbv_dt(name), None, None, 1, st) == 0
        assert not tbv.err()


def tbv_dt(name):
    return {"f32": 0, "f16": 1, "bf16": 2}[name]


def test_no_alloc_step_without_init():
    """The entry point needs no tbv_ar_init: every buffer is the caller's."""
    from libtbvcoll_amd import tbvcoll
    tbvcoll.shutdown()
    lib = tbvcoll.load()
    n = (2 << 20) + 64
    a = dev(synth.uniform(5, n // 2), torch.bfloat16); b = dev(synth.uniform(6, n // 2), torch.bfloat16)
    out = torch.empty_like(a); bounce = torch.empty_like(a)
    words = torch.zeros(16, dtype=torch.int64).pin_memory()
    st = torch.cuda.current_stream().cuda_stream
    for seq in (1, 2):
        assert lib.tbv_step_noalloc(out.data_ptr(), a.data_ptr(), b.data_ptr(), bounce.data_ptr(), 0, n, 2,
                                    words.data_ptr(), words.data_ptr() + 64, seq, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(out, a + b) and torch.equal(bounce.view(torch.int16), a.view(torch.int16))
        assert int(words[0]) == seq and int(words[8]) == seq


FIRST_CALL_UNDER_CAPTURE = r"""
import ctypes, sys
sys.path.insert(0, {root!r})
import torch
from libtbvcoll_amd import tbvcoll
lib = tbvcoll.load()                       # no tbv_ar_init, no earlier step: the counters' address is not bound yet
n = 1 << 20
a = torch.ones(n // 2, dtype=torch.bfloat16, device="cuda"); b = torch.full_like(a, 2.0)
out = torch.zeros_like(a); bounce = torch.zeros_like(a)
side = torch.cuda.Stream()
g = torch.cuda.CUDAGraph()
with torch.cuda.graph(g, stream=side):
    out.zero_()                            # something of the program's own, so the graph is not empty
    rc = lib.tbv_step_noalloc(out.data_ptr(), a.data_ptr(), b.data_ptr(), bounce.data_ptr(), 0, n, 2, None, None, 1,
                              torch.cuda.current_stream().cuda_stream)
print("CAPTURED_RC", rc, flush=True)
g.replay(); torch.cuda.synchronize()
print("AFTER_REPLAY", float(out.float().abs().max()), flush=True)
rc = lib.tbv_step_noalloc(out.data_ptr(), a.data_ptr(), b.data_ptr(), bounce.data_ptr(), 0, n, 2, None, None, 2,
                          torch.cuda.current_stream().cuda_stream)
torch.cuda.synchronize()
print("EAGER_RC", rc, bool(torch.equal(out, a + b)), flush=True)
"""


def test_first_no_alloc_step_inside_a_capture_is_refused():
    """The first call on a device looks up the address of the built-in counters, which is not allowed while a stream is
    being captured: such a call is refused with -1 (and launches nothing) instead of breaking the capture.  Needs a
    process in which neither tbv_ar_init nor an earlier step has run, hence the child process."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    say("first no-alloc step under capture, in a fresh process")
    p = subprocess.run([sys.executable, "-c", FIRST_CALL_UNDER_CAPTURE.format(root=root)], capture_output=True, text=True, timeout=240)
    assert "CAPTURED_RC -1" in p.stdout, (p.stdout, p.stderr[-2000:])
    assert "inside a stream capture" in p.stderr
    assert "AFTER_REPLAY 0.0" in p.stdout                        # the refused call recorded nothing into the graph
    assert "EAGER_RC 0 True" in p.stdout, (p.stdout, p.stderr[-2000:])


@pytest.mark.parametrize("uncached", [0, 1])
def test_no_alloc_step_in_a_graph(uncached):
    """Recorded into a HIP graph (the callers the entry point is for) and replayed four times with the program's own
    eager work and synchronisations in between; every replay checked against the eager result.  With an uncached
    bounce (a send slot of the initialised library) the step is the one-launch form, else pack kernel + sum kernel."""
    from libtbvcoll_amd import tbvcoll
    tbvcoll.shutdown()
    lib = tbvcoll.load()
    if uncached:
        tbvcoll.init(0, "rail0", "", cap_bytes=4 << 20)
    n = (2 << 20) + 64
    a = dev(synth.uniform(15, n // 2), torch.bfloat16); b = dev(synth.uniform(16, n // 2), torch.bfloat16)
    out = torch.empty_like(a); bounce = torch.empty_like(a)
    bptr = lib.tbv_emu_send_slot(1) if uncached else bounce.data_ptr()
    hip = _hip()
    words = torch.zeros(16, dtype=torch.int64).pin_memory()
    eager = torch.cuda.current_stream().cuda_stream
    # first call outside any capture: it looks up the counters' address on this device
    assert lib.tbv_step_noalloc(out.data_ptr(), a.data_ptr(), b.data_ptr(), bptr, uncached, n, 2,
                                words.data_ptr(), words.data_ptr() + 64, 1, eager) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, a + b)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    say("capture")
    with torch.cuda.graph(graph, stream=side):
        rc = lib.tbv_step_noalloc(out.data_ptr(), a.data_ptr(), b.data_ptr(), bptr, uncached, n, 2,
                                  words.data_ptr(), words.data_ptr() + 64, 7, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    for k in range(4):
        # the program's own eager work and a synchronisation between replays; new inputs each time
        a.copy_(dev(synth.uniform(20 + k, n // 2), torch.bfloat16)); b.mul_(0.5)
        out.zero_(); bounce.zero_(); words.zero_()
        if uncached:
            assert hip.hipMemcpy(bptr, bounce.data_ptr(), n, 3) == 0
        torch.cuda.synchronize()
        say("replay", k)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, a + b), k
        if uncached:
            assert hip.hipMemcpy(bounce.data_ptr(), bptr, n, 3) == 0
        assert torch.equal(bounce.view(torch.int16), a.view(torch.int16)), k
        assert int(words[0]) == 7 and int(words[8]) == 7, k
    tbvcoll.shutdown()
