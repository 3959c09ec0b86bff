"""The GroupCoordinator.all_reduce intercept (counterpart of step3b/vllm_tp_bench.py:77-140).

vLLM is not in this image, so the tests hand the intercept a stand-in `parallel_state`
module with the three things the patch touches: `GroupCoordinator` (with `world_size`,
`unique_name`, `all_reduce`), and `get_tp_group()`.  The CPU tests use a fake library
to pin routing, fallback accounting and error behaviour; the GPU test runs a toy
two-layer "decode loop" through the real library and through the fallback and compares
the output hashes, the reference's end-to-end gate."""
import types

import pytest
import torch

from libtbvcoll_amd import vllm_intercept


def make_ps(peer_of):
    """`peer_of(t)` plays the other rank in the original (RCCL) all-reduce."""
    class GroupCoordinator:
        def __init__(self, name, world_size):
            self.unique_name, self.world_size, self.orig_calls = name, world_size, 0

        def all_reduce(self, t):
            self.orig_calls += 1
            return t + peer_of(t)

    ps = types.SimpleNamespace(GroupCoordinator=GroupCoordinator)
    ps.tp = GroupCoordinator("tp:0", 2)
    ps.pp = GroupCoordinator("pp:0", 2)
    ps.single = GroupCoordinator("tp:0", 1)
    ps.get_tp_group = lambda: ps.tp
    return ps


class FakeLib:
    """Stands in for the binding: records calls, answers with a scripted return code."""
    def __init__(self, cap=1024, rc=0):
        self.cap_, self.rc, self.inits, self.calls = cap, rc, [], []

    def init(self, rank, devs, peer_ip, port=0, cap_bytes=0):
        self.inits.append((rank, devs, peer_ip, port, cap_bytes))

    def raw_fn(self):
        def fn(in_ptr, out_ptr, nb, dt, stream):
            self.calls.append((nb, dt))
            return self.rc
        return fn

    def cap(self):
        return self.cap_

    def stats5(self):
        return 0.0, 1.0, 2.0, 3.0, 0.0, len(self.calls)

    def is_async(self):
        return True


@pytest.fixture
def no_cuda_stream(monkeypatch):
    monkeypatch.setattr(torch.cuda, "current_stream", lambda: types.SimpleNamespace(cuda_stream=0))


def test_routing_fallback_and_accounting(no_cuda_stream):
    ps = make_ps(lambda t: torch.ones_like(t))
    lib = FakeLib(cap=1024)
    ic = vllm_intercept.install(ps, rank=1, devs="a,b", peer_ip="10.0.0.1", cap_bytes=1024, lib=lib)
    try:
        x = torch.zeros(8)
        assert ps.single.all_reduce(x) is x                                  # world size 1: untouched, no init
        assert lib.inits == []
        assert torch.equal(ps.pp.all_reduce(x), x + 1) and ps.pp.orig_calls == 1   # not the TP group: original
        assert lib.inits == []
        out = ps.tp.all_reduce(x)                                            # TP group: lazy init, then the library
        assert lib.inits == [(1, "a,b", "10.0.0.1", 18996, 1024)]
        assert lib.calls == [(32, 0)] and out.shape == x.shape and ps.tp.orig_calls == 0
        # over the cap, unsupported dtype, non-contiguous: fall back to the original and count it
        assert torch.equal(ps.tp.all_reduce(torch.zeros(1000)), torch.ones(1000))
        assert torch.equal(ps.tp.all_reduce(torch.zeros(4, dtype=torch.float64)), torch.ones(4, dtype=torch.float64))
        nc = torch.zeros(4, 4)[:, ::2]
        assert torch.equal(ps.tp.all_reduce(nc), nc + 1)
        assert ic.counters["n"] == 1 and ic.counters["fallback"] == 3 and ps.tp.orig_calls == 3
        lib.rc = -2                                                          # the library says "over my cap"
        assert torch.equal(ps.tp.all_reduce(x), x + 1)
        assert ic.counters["fallback"] == 4
        lib.rc = -1                                                          # any other code is an error
        with pytest.raises(RuntimeError):
            ps.tp.all_reduce(x)
        rep = ic.report()
        assert rep["mode"] == "ASYNC" and rep["n"] == 1 and rep["enq_us"] == 3.0
    finally:
        ic.uninstall()
    assert ps.GroupCoordinator.all_reduce is ic.orig


def test_fused_norm_routing_and_fallback(no_cuda_stream):
    """all_reduce_rmsnorm: the fused entry point for the TP group when the library takes the call, else the plain
    all-reduce (library or original) followed by the fp32 formula; both give (reduced, normed)."""
    ps = make_ps(lambda t: torch.ones_like(t))
    lib = FakeLib(cap=1 << 20)
    taken = []

    def fused(t, weight, eps, out=None):
        taken.append((tuple(t.shape), eps))
        if t.shape[-1] > 64:                      # plays "rows too long": the library declines
            return None
        out.copy_(t + 1)
        return torch.full_like(t, 5.0)

    lib.all_reduce_rmsnorm = fused
    ic = vllm_intercept.install(ps, rank=0, devs="a", cap_bytes=1 << 20, lib=lib)
    try:
        w = torch.full((8,), 2.0)
        x = torch.arange(16.0).reshape(2, 8)
        red, nrm = ic.all_reduce_rmsnorm(ps.tp, x, w, 1e-6)
        assert taken == [((2, 8), 1e-6)] and torch.equal(red, x + 1) and torch.equal(nrm, torch.full_like(x, 5.0))
        assert ic.counters["fused_norm"] == 1 and ic.counters["n"] == 1 and ps.tp.orig_calls == 0
        # declined by the library: plain all-reduce through the library's raw function, norm by the formula
        big = torch.ones(2, 128)
        red, nrm = ic.all_reduce_rmsnorm(ps.tp, big, torch.full((128,), 2.0), 0.0)
        assert len(taken) == 2 and lib.calls[-1] == (2 * 128 * 4, 0) and ic.counters["fused_norm"] == 1
        # another group: the original all-reduce, then the formula (x + 1 = 2 everywhere: rms 2, normed 1 * weight)
        red, nrm = ic.all_reduce_rmsnorm(ps.pp, torch.ones(2, 8), w, 0.0)
        assert ps.pp.orig_calls == 1 and torch.equal(red, torch.full((2, 8), 2.0)) and torch.allclose(nrm, torch.full((2, 8), 2.0))
        # world size 1: nothing to reduce, the norm is still computed
        red, nrm = ic.all_reduce_rmsnorm(ps.single, torch.full((1, 8), 3.0), w, 0.0)
        assert torch.equal(red, torch.full((1, 8), 3.0)) and torch.allclose(nrm, torch.full((1, 8), 2.0))
        # a weight of another dtype or length is not handed to the library
        n_before = len(taken)
        ic.all_reduce_rmsnorm(ps.tp, x, torch.full((8,), 2.0, dtype=torch.float64), 1e-6)
        assert len(taken) == n_before
    finally:
        ic.uninstall()


def test_rank0_passes_no_peer_address_and_eager_init(no_cuda_stream):
    ps = make_ps(lambda t: t)
    lib = FakeLib()
    ic = vllm_intercept.install(ps, rank=0, devs="a", peer_ip="10.0.0.2", eager=True, lib=lib)
    assert lib.inits == [(0, "a", "", 18996, 8 << 20)]                       # only rank 1 connects to a peer
    ic.uninstall()


def test_no_tp_group_means_no_interception(no_cuda_stream):
    ps = make_ps(lambda t: torch.ones_like(t))
    def boom():
        raise AssertionError("tensor parallel group is not initialised")
    ps.get_tp_group = boom
    lib = FakeLib()
    ic = vllm_intercept.install(ps, rank=0, devs="a", lib=lib)
    assert torch.equal(ps.tp.all_reduce(torch.zeros(4)), torch.ones(4)) and lib.inits == []
    ic.uninstall()


def test_output_hash_is_the_references_formula():
    import hashlib
    outs = [[1, 2, 3], (4, 5)]
    want = hashlib.sha256(b"[1, 2, 3][4, 5]").hexdigest()[:16]
    assert vllm_intercept.output_hash(outs) == want


@pytest.mark.gpu
def test_toy_decode_loop_hash_matches_fallback():
    """Greedy 'decode' of a toy two-layer model whose every layer ends in a TP all-reduce: the token ids
    produced through the library must hash to what the original all-reduce produces."""
    from gpu_util import session
    from libtbvcoll_amd import synth, tbvcoll
    hidden, vocab, steps, batch = 4096, 512, 24, 8
    w = [torch.from_numpy(synth.normal(10 + i, hidden * hidden, 0.02)).reshape(hidden, hidden).to(torch.bfloat16).cuda() for i in range(2)]
    head = torch.from_numpy(synth.normal(20, hidden * vocab, 0.02)).reshape(hidden, vocab).to(torch.bfloat16).cuda()
    emb = torch.from_numpy(synth.normal(21, vocab * hidden)).reshape(vocab, hidden).to(torch.bfloat16).cuda()

    def run(ps, stage):
        ids = torch.arange(batch, device="cuda") % vocab
        produced = [[] for _ in range(batch)]
        for _ in range(steps):
            h = emb[ids]
            for layer in range(2):
                part = (h @ w[layer]).contiguous()                 # this rank's partial sum
                peer = (part * 0.5 + 0.25).to(torch.bfloat16)      # what the other rank would contribute
                stage(peer)
                h = torch.tanh(ps.tp.all_reduce(part))
            ids = (h @ head).float().argmax(dim=-1)
            for b in range(batch):
                produced[b].append(int(ids[b]))
        return vllm_intercept.output_hash(produced), produced

    current = {}
    ps_ref = make_ps(lambda t: current["peer"])
    want, ids_ref = run(ps_ref, lambda p: current.__setitem__("peer", p))
    with session(rails=2, cap=1 << 20):
        tbvcoll.shutdown()                                          # the intercept initialises the library itself
        ps = make_ps(lambda t: (_ for _ in ()).throw(AssertionError("fallback must not be used")))
        ic = vllm_intercept.install(ps, rank=0, devs="rail0,rail1", cap_bytes=1 << 20, eager=True)
        try:
            got, ids = run(ps, tbvcoll.stage_peer)
        finally:
            ic.uninstall()
        assert ic.counters["n"] == steps * 2 and ic.counters["fallback"] == 0
        assert got == want, (ids[0][:8], ids_ref[0][:8])
        assert not tbvcoll.err()



@pytest.mark.gpu
def test_fused_norm_through_the_real_library():
    """all_reduce_rmsnorm of the intercept on the GPU: the reduced tensor and the normalised one equal the CPU
    restatement bit for bit when the library takes the call; rows it does not take come back from the fallback
    formula within 2 ulp of that restatement."""
    import numpy as np
    from gpu_util import bits_np, session
    from libtbvcoll_amd import synth, tbvcoll
    from oracle import oracle
    hidden, rows = 4096, 16
    a = torch.from_numpy(synth.normal(31, rows * hidden)).to(torch.bfloat16).reshape(rows, hidden)
    b = torch.from_numpy(synth.normal(32, rows * hidden)).to(torch.bfloat16).reshape(rows, hidden)
    w = torch.from_numpy(1.0 + 0.25 * synth.normal(33, hidden)).to(torch.bfloat16)
    want_out, want_normed = oracle.sum_rmsnorm(oracle.DT_BF16, bits_np(a), bits_np(b), bits_np(w), hidden, 1e-6)
    with session(rails=2, cap=1 << 20):
        tbvcoll.shutdown()
        peer = {}
        ps = make_ps(lambda t: peer["t"])
        ic = vllm_intercept.install(ps, rank=0, devs="rail0,rail1", cap_bytes=1 << 20, eager=True)
        try:
            A, B, W = a.cuda(), b.cuda(), w.cuda()
            tbvcoll.stage_peer(B)
            red, nrm = ic.all_reduce_rmsnorm(ps.tp, A, W, 1e-6)
            torch.cuda.synchronize()
            assert np.array_equal(bits_np(red).reshape(-1), want_out) and np.array_equal(bits_np(nrm).reshape(-1), want_normed)
            assert ic.counters["fused_norm"] == 1 and ps.tp.orig_calls == 0
            # a strided view is taken neither by the fused entry point nor by the plain one: original all-reduce + formula
            peer["t"] = B[:, ::2]
            red2, nrm2 = ic.all_reduce_rmsnorm(ps.tp, A[:, ::2], W[::2].contiguous(), 1e-6)
            torch.cuda.synchronize()
            x = (A[:, ::2] + B[:, ::2]).float()
            ref = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16) * W[::2]
            assert ps.tp.orig_calls == 1 and ic.counters["fallback"] == 1
            assert torch.equal(red2, A[:, ::2] + B[:, ::2]) and torch.equal(nrm2, ref)
        finally:
            ic.uninstall()
        assert not tbvcoll.err()
