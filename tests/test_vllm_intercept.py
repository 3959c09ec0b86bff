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

