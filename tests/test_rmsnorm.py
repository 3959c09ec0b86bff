"""All-reduce fused with the following RMSNorm: the CPU restatement pinned against torch's fp32 formula and
closed-form rows, and (-m gpu) the HIP row kernel and the fused entry point against the restatement.

Tolerances.  The reduced tensor `out` is bit-exact (it is the sum kernel's result).  The normalised tensor is
bit-exact between the GPU and the CPU restatement, because both take the fp32 sum of squares in the same stated
order and use correctly rounded division and square root.  Against torch's formula, whose summation order
differs, it is held to 2 units in the last place of the storage type on every element, with at least 99.5 %
of the elements identical."""
import numpy as np
import pytest
import torch

from libtbvcoll_amd import synth
from oracle import oracle

DTS = {"f32": (torch.float32, 0), "f16": (torch.float16, 1), "bf16": (torch.bfloat16, 2)}


def bits(t):
    return oracle.torch_bits(t).reshape(-1)


def from_bits(arr, dt):
    if dt == torch.float32:
        return torch.from_numpy(arr.copy())
    return torch.from_numpy(arr.view(np.int16).copy()).view(dt)


def torch_rmsnorm(x, w, eps):
    """The formula of the reference's caller (vLLM / HF RMSNorm): fp32 statistics, cast, then the weight in T."""
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    return (xf * torch.rsqrt(var + eps)).to(x.dtype) * w


def ulp_distance(a, b, dt):
    """Distance in units in the last place between two tensors of the same storage type (finite values)."""
    if dt == torch.float32:
        ia = a.view(torch.int32).to(torch.int64); ib = b.view(torch.int32).to(torch.int64)
        sign = 1 << 31
    else:
        ia = a.view(torch.int16).to(torch.int64) & 0xffff; ib = b.view(torch.int16).to(torch.int64) & 0xffff
        sign = 1 << 15
    ma = torch.where(ia & sign != 0, -(ia & (sign - 1)), ia); mb = torch.where(ib & sign != 0, -(ib & (sign - 1)), ib)
    return (ma - mb).abs()


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("hidden", [64, 4096, 5120, 16384])
def test_oracle_rmsnorm_against_torch_formula(name, hidden):
    dt, code = DTS[name]
    rows = 24
    x = torch.from_numpy(synth.normal(7 + hidden, rows * hidden)).to(dt).reshape(rows, hidden)
    w = torch.from_numpy(1.0 + 0.25 * synth.normal(8 + hidden, hidden)).to(dt)
    got = from_bits(oracle.rmsnorm_rows(code, bits(x), bits(w), hidden, 1e-6), dt).reshape(rows, hidden)
    want = torch_rmsnorm(x, w, 1e-6)
    d = ulp_distance(got, want, dt)
    assert int(d.max()) <= (8 if name == "f32" else 2), int(d.max())
    assert float((d == 0).float().mean()) >= (0.5 if name == "f32" else 0.995)


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
def test_oracle_rmsnorm_closed_forms(name):
    dt, code = DTS[name]
    hidden = 4096
    w = torch.from_numpy(synth.uniform(3, hidden)).to(dt)
    rows = []
    # one non-zero element v: mean of squares v^2/H, so x*s = v / (|v|/64) = +-64 there and 0 elsewhere
    r = torch.zeros(hidden); r[1234] = -3.0; rows.append(r)
    # every element the same power of two c: mean of squares c^2, x*s = 1 exactly
    rows.append(torch.full((hidden,), 0.5))
    # all zero with eps > 0: 0 * 1/sqrt(eps) = 0, no NaN
    rows.append(torch.zeros(hidden))
    # eps far above the mean of squares: s = 1/sqrt(eps) to within rounding; with eps = 4 that is x / 2
    rows.append(torch.full((hidden,), 2.0 ** -20))
    x = torch.stack(rows).to(dt)
    got0 = from_bits(oracle.rmsnorm_rows(code, bits(x[:2]), bits(w), hidden, 0.0), dt).reshape(2, hidden)
    assert torch.equal(got0[0][1234], (torch.tensor(-64.0).to(dt) * w[1234]))
    assert int(got0[0].count_nonzero()) == 1
    assert torch.equal(got0[1], torch.ones(hidden).to(dt) * w)                     # the weight lands on its own column
    z = from_bits(oracle.rmsnorm_rows(code, bits(x[2:3]), bits(w), hidden, 1e-6), dt)
    assert int(z.count_nonzero()) == 0 and not bool(torch.isnan(z).any())
    big = from_bits(oracle.rmsnorm_rows(code, bits(x[3:4]), bits(w), hidden, 4.0), dt)
    assert torch.equal(big, (x[3].float() * 0.5).to(dt) * w)


def test_oracle_sum_rmsnorm_is_sum_then_norm():
    dt, code = DTS["bf16"]
    hidden, rows = 1024, 9
    a = torch.from_numpy(synth.normal(1, rows * hidden)).to(dt); b = torch.from_numpy(synth.normal(2, rows * hidden)).to(dt)
    w = torch.from_numpy(synth.uniform(3, hidden)).to(dt)
    out, normed = oracle.sum_rmsnorm(code, bits(a), bits(b), bits(w), hidden, 1e-5)
    assert np.array_equal(out, oracle.sum_bits(code, bits(a), bits(b)))
    assert np.array_equal(normed, oracle.rmsnorm_rows(code, out, bits(w), hidden, 1e-5))
    assert np.array_equal(out, bits(a + b))                                        # torch's CPU add in the storage type


# ------------------------------------------------------------------ GPU

def _gpu_inputs(name, rows, hidden, seed):
    dt, code = DTS[name]
    a = torch.from_numpy(synth.normal(seed, rows * hidden)).to(dt).reshape(rows, hidden)
    b = torch.from_numpy(synth.normal(seed + 1, rows * hidden)).to(dt).reshape(rows, hidden)
    w = torch.from_numpy(1.0 + 0.25 * synth.normal(seed + 2, hidden)).to(dt)
    return dt, code, a, b, w


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("rows,hidden", [(1, 4096), (3, 64), (17, 5120), (128, 4096), (5, 16384), (2048, 4096), (5000, 512), (4097, 1024)])
def test_row_kernel_bit_exact_vs_oracle(name, rows, hidden):
    from gpu_util import say
    from libtbvcoll_amd import tbvcoll
    if name == "f32" and hidden * 4 > 65536:
        pytest.skip("row longer than 64 KiB")
    dt, code, a, b, w = _gpu_inputs(name, rows, hidden, 40 + rows)
    lib = tbvcoll.load()
    A, B, W = a.cuda(), b.cuda(), w.cuda()
    out = torch.empty_like(A); normed = torch.empty_like(A)
    st = torch.cuda.current_stream().cuda_stream
    say("row kernel", name, rows, hidden)
    assert lib.tbv_emu_run_sum_norm(1, out.data_ptr(), A.data_ptr(), B.data_ptr(), normed.data_ptr(), W.data_ptr(), 1e-6, rows, hidden, code, st) == 0
    torch.cuda.synchronize()
    want_out, want_normed = oracle.sum_rmsnorm(code, bits(a), bits(b), bits(w), hidden, 1e-6)
    assert np.array_equal(bits(out), want_out)
    assert np.array_equal(bits(normed), want_normed)
    # norm-only mode on the reduced tensor gives the same
    n2 = torch.empty_like(A)
    assert lib.tbv_emu_run_sum_norm(0, None, out.data_ptr(), None, n2.data_ptr(), W.data_ptr(), 1e-6, rows, hidden, code, st) == 0
    torch.cuda.synchronize()
    assert np.array_equal(bits(n2), want_normed)
    # the cache-cold variant of the looping form (mode + 4: non-temporal loads) computes the same bits
    o3 = torch.empty_like(A); n3 = torch.empty_like(A)
    assert lib.tbv_emu_run_sum_norm(1 + 4, o3.data_ptr(), A.data_ptr(), B.data_ptr(), n3.data_ptr(), W.data_ptr(), 1e-6, rows, hidden, code, st) == 0
    torch.cuda.synchronize()
    assert np.array_equal(bits(o3), want_out) and np.array_equal(bits(n3), want_normed)
    # and torch's own formula on the GPU agrees to 2 ulp
    d = ulp_distance(normed.cpu(), torch_rmsnorm(out, W, 1e-6).cpu(), dt)
    assert int(d.max()) <= (8 if name == "f32" else 2)


MODES = {"default": {}, "two_kernels": {"TBV_ONEKERNEL": 0}, "stream_gate": {"TBV_FUSEWAIT": 0, "TBV_DEFERSIG": 0, "TBV_ONEKERNEL": 0},
         "railsum": {"TBV_RAILSUM": 1}, "host_wire": {"TBV_WIRE": "host"}, "sync": {"TBV_ASYNC": 0}, "tag": {"TBV_TAG": 1}, "kwait": {"TBV_KWAIT": 1}}


@pytest.mark.gpu
@pytest.mark.parametrize("mode", sorted(MODES))
def test_allreduce_rmsnorm_entry_point(mode):
    """The fused entry point through the C ABI: decode shapes (1..128 rows) and a prefill shape, peer staged per call,
    early peer, in place and out of place; `out` and `normed` bit-exact against the CPU restatement."""
    from gpu_util import say, session
    hidden = 4096
    with session(rails=2, cap=16 << 20, **MODES[mode]) as tbv:
        k = 0
        for name in ("bf16", "f16", "f32"):
            for rows in (1, 2, 32, 128, 129, 2048 if name != "f32" else 1024):
                k += 1
                dt, code, a, b, w = _gpu_inputs(name, rows, hidden, 100 + 3 * k)
                want_out, want_normed = oracle.sum_rmsnorm(code, bits(a), bits(b), bits(w), hidden, 1e-5)
                A, B, W = a.cuda(), b.cuda(), w.cuda()
                for inplace in (False, True):
                    x = A.clone()
                    out = None if inplace else torch.empty_like(A)
                    tbv.stage_peer(B)
                    say("allreduce_rmsnorm", mode, name, rows, "in place" if inplace else "out of place")
                    normed = tbv.all_reduce_rmsnorm(x, W, 1e-5, out=out)
                    assert normed is not None
                    torch.cuda.synchronize()
                    assert np.array_equal(bits(x if inplace else out), want_out), (mode, name, rows)
                    assert np.array_equal(bits(normed), want_normed), (mode, name, rows)
        # the peer ran ahead: flag up on entry
        dt, code, a, b, w = _gpu_inputs("bf16", 64, hidden, 900)
        A, B, W = a.cuda(), b.cuda(), w.cuda()
        tbv.peer_resident(B)
        want_out, want_normed = oracle.sum_rmsnorm(code, bits(a), bits(b), bits(w), hidden, 1e-5)
        for _ in range(6):
            out = torch.empty_like(A)
            normed = tbv.all_reduce_rmsnorm(A, W, 1e-5, out=out)
            torch.cuda.synchronize()
            assert np.array_equal(bits(out), want_out) and np.array_equal(bits(normed), want_normed)
        tbv.peer_resident(None)
        # not taken (None: the caller falls back, nothing raised, nothing queued): over the cap, a row that is not a
        # multiple of 16 bytes, a row over 64 KiB, a view that is not 16-byte aligned
        seq0 = tbv.seq()
        assert tbv.all_reduce_rmsnorm(torch.zeros(4097, 4096, dtype=torch.bfloat16, device="cuda"), W, 1e-5) is None
        assert tbv.all_reduce_rmsnorm(torch.zeros(4, 100, dtype=torch.bfloat16, device="cuda"), torch.ones(100, dtype=torch.bfloat16, device="cuda"), 1e-5) is None
        assert tbv.all_reduce_rmsnorm(torch.zeros(2, 40000, dtype=torch.bfloat16, device="cuda"), torch.ones(40000, dtype=torch.bfloat16, device="cuda"), 1e-5) is None
        odd = torch.zeros(4 * 4096 + 4, dtype=torch.bfloat16, device="cuda")[4:].view(4, 4096)      # 8 bytes past a 16-byte boundary
        assert odd.data_ptr() % 16 == 8 and tbv.all_reduce_rmsnorm(odd, W, 1e-5) is None
        assert tbv.seq() == seq0 and not tbv.err()
        # many rows, gated inside the kernel (the row kernel's blocks loop over rows, so its grid can be capped)
        dt, code, a, b, w = _gpu_inputs("bf16", 3000, 1024, 950)
        A, B, W2 = a.cuda(), b.cuda(), w.cuda()
        want_out, want_normed = oracle.sum_rmsnorm(code, bits(a), bits(b), bits(w), 1024, 1e-5)
        out = torch.empty_like(A)
        tbv.stage_peer(B)
        normed = tbv.all_reduce_rmsnorm(A, W2, 1e-5, out=out)
        torch.cuda.synchronize()
        assert np.array_equal(bits(out), want_out) and np.array_equal(bits(normed), want_normed)
        assert not tbv.err()
