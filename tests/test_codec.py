"""int8 payload codec (group 128, asymmetric): the CPU restatement pinned by invariants, an independent float64
computation and hand-made groups; (-m gpu) the HIP kernels and the all-reduce with TBV_CODEC=1 against it, byte for
byte.  Accuracy statement: every decoded element is within scale/2 of the original, scale = (max - min)/255 of its
group of 128, so an all-reduce result is within (scale_own + scale_peer)/2 (+ one rounding to the storage type) of
the exact sum."""
import numpy as np
import pytest
import torch

from libtbvcoll_amd import synth
from oracle import oracle

DTS = {"f32": (torch.float32, 0), "f16": (torch.float16, 1), "bf16": (torch.bfloat16, 2)}


def bits(t):
    return oracle.torch_bits(t).reshape(-1)


def parse_image(img, n):
    """(scale[G], mn[G], codes[n]) from an image laid out as superblocks of 16 x (scale, mn) + 16 x 128 codes."""
    nsb = (n + 2047) // 2048
    sb = np.asarray(img, dtype=np.uint8).reshape(nsb, 2176)
    hdr = sb[:, :128].copy().view(np.float32).reshape(nsb, 16, 2)
    codes = sb[:, 128:].reshape(-1)[:n]
    G = (n + 127) // 128
    return hdr[:, :, 0].reshape(-1)[:G], hdr[:, :, 1].reshape(-1)[:G], codes


def test_library_and_restatement_agree_on_image_sizes():
    """The size of an image is host arithmetic in the library (no GPU needed): 2176 bytes per started superblock of
    2048 elements, the same as the CPU restatement says and as the format's closed form."""
    from libtbvcoll_amd import tbvcoll
    lib = tbvcoll.load()
    for code, esz in ((0, 4), (1, 2), (2, 2)):
        for n in (0, 1, 127, 128, 2047, 2048, 2049, 100000, 8 << 20):
            want = (n + 2047) // 2048 * 2176
            assert lib.tbv_emu_codec_image_bytes(n * esz, code) == want
            assert int(oracle.lib().orc_q8_image_bytes(n)) == want
    assert lib.tbv_emu_codec_image_bytes(4096, 5) == 0              # unknown dtype


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("n", [128, 2048, 2048 * 3 + 128 * 5 + 8, 100000])
def test_codec_invariants(name, n):
    dt, code = DTS[name]
    x = torch.from_numpy(synth.normal(3 + n, n) * 0.05).to(dt)
    x[::997] = 6.0                                                      # outliers stretch some groups
    img = oracle.q8_encode(code, bits(x))
    assert img.size == (n + 2047) // 2048 * 2176
    scale, mn, codes = parse_image(img, n)
    xf = x.float().numpy()
    dec = oracle.q8_decode(img, n)
    g = np.arange(n) // 128
    # the group header is the group's own minimum and (max - min) / 255, computed here with numpy reductions
    gmin = np.minimum.reduceat(xf, np.arange(0, n, 128)); gmax = np.maximum.reduceat(xf, np.arange(0, n, 128))
    assert np.array_equal(mn, gmin)
    assert np.array_equal(scale, np.where(gmax > gmin, (gmax - gmin) / np.float32(255.0), np.float32(1.0)).astype(np.float32))
    # round trip within half a step; slack for the fp32 roundings of the stated arithmetic: 255 * 3 * 2^-24 of a step
    # where a code sits on a rounding boundary, the same again for scale in the decode, and one rounding of the result
    big = np.maximum(np.abs(gmin), np.abs(gmax))[g].astype(np.float64)
    assert np.all(np.abs(dec.astype(np.float64) - xf) <= scale[g].astype(np.float64) * (0.5 + 1e-4) + big * 2.0 ** -23)
    assert np.all(codes[xf == gmin[g]] == 0)
    assert np.all(codes[(xf == gmax[g]) & (gmax[g] > gmin[g])] == 255)
    # codes are monotone in the value within a group
    for gi in range(0, (n + 127) // 128, 7):
        v = xf[gi * 128:(gi + 1) * 128]; c = codes[gi * 128:(gi + 1) * 128].astype(np.int32)
        o = np.argsort(v, kind="stable")
        assert np.all(np.diff(c[o]) >= 0)
    # an independent float64 computation of the codes agrees except at rounding boundaries, and then by one
    q64 = np.rint((xf.astype(np.float64) - gmin[g]) * np.where(gmax > gmin, 255.0 / (gmax.astype(np.float64) - gmin), 0.0)[g])
    d = np.abs(q64 - codes)
    assert d.max() <= 1 and (d == 0).mean() > 0.999


def test_codec_hand_made_groups():
    # 0, 1, ..., 127 scaled so that max - min = 255 * 0.5: codes are 2 * i (exact in fp32), decode gives the value back
    x = (np.arange(128, dtype=np.float32) * 1.0 - 3.0)
    x[127] = 124.5                                                     # min -3, max 124.5: range 127.5 = 255 * 0.5
    img = oracle.q8_encode(0, x)
    scale, mn, codes = parse_image(img, 128)
    assert scale[0] == np.float32(0.5) and mn[0] == np.float32(-3.0)
    assert np.array_equal(codes[:127], (2 * np.arange(127)).astype(np.uint8)) and codes[127] == 255
    assert np.array_equal(oracle.q8_decode(img, 128), x)
    # a constant group is exact; a group of -0.0 and +0.0 stores +0 as its minimum
    c = np.full(300, 1.2345, dtype=np.float32)
    assert np.array_equal(oracle.q8_decode(oracle.q8_encode(0, c), 300), c)
    z = np.zeros(128, dtype=np.float32); z[::2] = -0.0
    s, m, q = parse_image(oracle.q8_encode(0, z), 128)
    assert m.view(np.uint32)[0] == 0 and s[0] == 1.0 and not q.any()
    # half-way values round to even codes: values 0, 0.5, 1.5, 2.5, 255 with step 1 -> codes 0, 0, 2, 2, 255
    h = np.zeros(128, dtype=np.float32); h[1:5] = [0.5, 1.5, 2.5, 255.0]
    assert parse_image(oracle.q8_encode(0, h), 128)[2][:5].tolist() == [0, 0, 2, 2, 255]
    # absent elements of the last group and absent groups of the last superblock are zero bytes
    img = oracle.q8_encode(2, bits(torch.ones(130, dtype=torch.bfloat16)))
    sb = img.reshape(1, 2176)
    assert not sb[0, 16:128].any() and not sb[0, 128 + 130:].any()


@pytest.mark.parametrize("name", ["f16", "bf16", "f32"])
def test_codec_sum_is_decode_plus_decode(name):
    dt, code = DTS[name]
    n = 5000
    a = torch.from_numpy(synth.normal(1, n)).to(dt); b = torch.from_numpy(synth.normal(2, n)).to(dt)
    ia, ib = oracle.q8_encode(code, bits(a)), oracle.q8_encode(code, bits(b))
    got = oracle.q8_sum(code, ia, ib, n)
    want = (torch.from_numpy(oracle.q8_decode(ia, n)) + torch.from_numpy(oracle.q8_decode(ib, n))).to(dt)    # torch's fp32 add and cast
    assert np.array_equal(got, bits(want))
    assert np.array_equal(got, oracle.q8_sum(code, ib, ia, n))          # both ranks of a pair compute the same bits
    # accuracy against the exact sum: within half a step of each image plus the rounding to the storage type
    sa, _, _ = parse_image(ia, n); sb_, _, _ = parse_image(ib, n)
    g = np.arange(n) // 128
    err = np.abs(want.double().numpy() - (a.double() + b.double()).numpy())
    ulp = np.abs(want.double().numpy()) * (2.0 ** -8 if name == "bf16" else 2.0 ** -11 if name == "f16" else 2.0 ** -24)
    assert np.all(err <= (sa[g] + sb_[g]) * 0.5 * 1.001 + ulp + 1e-12)


# ------------------------------------------------------------------ GPU

def _coded_sum(dt, code, a, b):
    """The coded all-reduce's result (CPU restatement) of two fp32 arrays stored as `dt`, with the uncoded one."""
    A, B = torch.from_numpy(a).to(dt), torch.from_numpy(b).to(dt)
    n = A.numel()
    out = oracle.q8_sum(code, oracle.q8_encode(code, bits(A)), oracle.q8_encode(code, bits(B)), n)
    outf = torch.from_numpy(out.view(np.int16)).view(dt).float().numpy() if code != 0 else out.astype(np.float32)
    return outf, A.float().numpy(), B.float().numpy(), (A + B).float().numpy()


def test_codec_accuracy_metric_on_the_bench_distributions():
    """The codec's own accuracy metric (relative L2 error / SNR against the exact sum), on the prefill distribution
    with and without its 0.1 % outliers, on N(0,1) and on U[-4,4].  The figures the documentation quotes are pinned
    here: without outliers the coded sum is within 0.7 % of the exact one (44 dB; the uncoded bf16 sum: 0.18 %); with
    one element in a thousand at +-8 a fifth of the groups is stretched and the error on the other 99.8 % of the
    elements is 14-19 % (16 dB), although the whole-tensor figure still reads 1.3 % because the outliers carry the norm."""
    from libtbvcoll_amd import codec_metric
    n = 1 << 20
    got = {}
    for name, gen, cut in codec_metric.distributions(synth):
        outf, a, b, unc = _coded_sum(torch.bfloat16, 2, gen(100, n), gen(101, n))
        got[name] = codec_metric.accuracy(outf, a, b, cut, unc)
    with_out, clean, normal, uni = (got[k] for k, _, _ in codec_metric.distributions(synth))
    for m in (clean, normal, uni):
        assert m["stretched_group_frac"] == 0.0 and m["rel_l2"] == m["rel_l2_typical"]
        assert 0.002 < m["rel_l2"] < 0.007 and m["snr_db"] > 43.0
        assert 0.0015 < m["rel_l2_uncoded"] < 0.0021                  # bf16 rounding of the exact sum: 2^-9 / sqrt(3)
    assert 0.0015 < with_out["outlier_element_frac"] < 0.0025         # 0.1 % per operand
    assert 0.19 < with_out["stretched_group_frac"] < 0.25             # 1 - (1 - 0.001)^256
    assert 0.010 < with_out["rel_l2"] < 0.016                         # dominated by the outliers' own magnitude
    assert 0.14 < with_out["rel_l2_typical"] < 0.19                   # what the other elements see
    assert 0.30 < with_out["rel_l2_typical_in_stretched"] < 0.40 and with_out["rel_l2_typical_in_clean"] < 0.007
    assert with_out["max_abs_err"] <= 2 * 16.04 / 255 / 2 + 0.01      # two operands, half a step of a stretched group each
    # closed form of the clean case: uniform quantisation noise of both operands, step = range / 255
    g = torch.from_numpy(synth.normal(100, n, std=0.02)).to(torch.bfloat16).float().numpy().reshape(-1, 128)
    step = (g.max(1) - g.min(1)) / 255.0
    predicted = np.sqrt(2 * np.mean(step ** 2) / 12.0) / np.sqrt(2 * 0.02 ** 2)
    assert abs(clean["rel_l2"] - predicted) / predicted < 0.15


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("n", [2048, 8 * 1000 + 8, 1 << 20, (8 << 20) + 4096 + 128])
def test_codec_kernels_byte_exact(name, n):
    from gpu_util import say
    from libtbvcoll_amd import tbvcoll
    dt, code = DTS[name]
    esz = 4 if name == "f32" else 2
    lib = tbvcoll.load()
    a = torch.from_numpy(synth.normal(5 + n % 100, n) * 0.02).to(dt); b = torch.from_numpy(synth.uniform(6 + n % 100, n)).to(dt)
    a[::1000] = 8.0
    A, B = a.cuda(), b.cuda()
    nb = n * esz
    ib = lib.tbv_emu_codec_image_bytes(nb, code)
    assert ib == oracle.q8_encode(code, bits(a[:1])).size * ((n + 2047) // 2048)
    IA = torch.zeros(ib, dtype=torch.uint8, device="cuda"); IB = torch.full((ib,), 255, dtype=torch.uint8, device="cuda")
    out = torch.empty_like(A)
    st = torch.cuda.current_stream().cuda_stream
    say("codec kernels", name, n)
    assert lib.tbv_emu_run_quant(IA.data_ptr(), A.data_ptr(), nb, code, st) == 0
    assert lib.tbv_emu_run_quant(IB.data_ptr(), B.data_ptr(), nb, code, st) == 0
    assert lib.tbv_emu_run_sum_quant(out.data_ptr(), IA.data_ptr(), IB.data_ptr(), nb, code, st) == 0
    torch.cuda.synchronize()
    wa, wb = oracle.q8_encode(code, bits(a)), oracle.q8_encode(code, bits(b))
    assert np.array_equal(IA.cpu().numpy(), wa)
    assert np.array_equal(IB.cpu().numpy(), wb)
    assert np.array_equal(bits(out), oracle.q8_sum(code, wa, wb, n))


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["default", "stream_gate", "host_wire", "nslot2", "streaming"])
def test_allreduce_with_codec(mode):
    """tbv_ar_allreduce with TBV_CODEC=1: above the threshold the bounce slot holds the int8 image and the result is
    decode + decode; below it, and for ragged byte counts, the call is the plain bit-exact sum."""
    import ctypes
    from gpu_util import say, session
    env = {"default": {}, "stream_gate": {"TBV_FUSEWAIT": 0, "TBV_DEFERSIG": 0}, "host_wire": {"TBV_WIRE": "host"},
           "nslot2": {"TBV_NSLOT": 2}, "streaming": {"TBV_STREAMING": 1}}[mode]
    hip = ctypes.CDLL("libamdhip64.so.7")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    with session(rails=2, cap=8 << 20, TBV_CODEC=1, TBV_CODEC_MIN=256 << 10, **env) as tbv:
        nslot = tbv.lib().tbv_emu_nslot()
        k = 0
        for name in ("bf16", "f16", "f32"):
            dt, code = DTS[name]
            esz = 4 if name == "f32" else 2
            for nb in (256 << 10, (1 << 20) + 4096, 8 << 20, 8192, (512 << 10) + 2):
                n = nb // esz
                nb = n * esz
                k += 1
                a = torch.from_numpy(synth.normal(20 + k, n) * 0.02).to(dt); b = torch.from_numpy(synth.normal(60 + k, n) * 0.02).to(dt)
                A, B = a.cuda(), b.cuda()
                out = torch.empty_like(A)
                tbv.stage_peer(B)
                say("codec allreduce", mode, name, nb)
                assert tbv.all_reduce(A, out)
                torch.cuda.synchronize()
                coded = nb >= (256 << 10) and nb % 16 == 0
                if coded:
                    wa, wb = oracle.q8_encode(code, bits(a)), oracle.q8_encode(code, bits(b))
                    assert np.array_equal(bits(out), oracle.q8_sum(code, wa, wb, n)), (name, nb)
                    img = torch.empty(wa.size, dtype=torch.uint8, device="cuda")
                    assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % nslot), wa.size, 3) == 0
                    assert np.array_equal(img.cpu().numpy(), wa)               # what travels is the image: 0.53 of a 2-byte payload
                    assert wa.size <= 0.54 * nb * (2 / esz) + 2176
                else:
                    assert np.array_equal(bits(out), oracle.sum_bits(code, bits(a), bits(b))), (name, nb)
        # mirror mode (the peer echoes this rank's image) and the early peer, in place
        a = torch.from_numpy(synth.normal(7, 1 << 20) * 0.02).to(torch.bfloat16); A = a.cuda()
        wa = oracle.q8_encode(2, bits(a))
        x = A.clone()
        assert tbv.all_reduce(x)
        torch.cuda.synchronize()
        assert np.array_equal(bits(x), oracle.q8_sum(2, wa, wa, a.numel()))
        b = torch.from_numpy(synth.normal(8, 1 << 20) * 0.02).to(torch.bfloat16)
        tbv.peer_resident(b.cuda())
        wb = oracle.q8_encode(2, bits(b))
        for _ in range(2 * nslot + 1):
            out = torch.empty_like(A)
            assert tbv.all_reduce(A, out)
        torch.cuda.synchronize()
        assert np.array_equal(bits(out), oracle.q8_sum(2, wa, wb, a.numel()))
        tbv.peer_resident(None)
        assert not tbv.err()


@pytest.mark.gpu
@pytest.mark.parametrize("one_launch", [1, 0])
def test_coded_step_with_the_peer_image_in_place(one_launch):
    """Early peer with the codec: by default the whole coded step is one kernel (quantise, decode both images, sum)
    that never reads its own image back; with TBV_MERGE=0 it is the quantise kernel followed by the dequantising
    sum.  Both must give the oracle's image in the bounce slot and the oracle's sum, out of place and in place,
    for sizes that end inside a superblock and inside a group."""
    import ctypes
    from gpu_util import say, session
    hip = ctypes.CDLL("libamdhip64.so.7")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    with session(rails=2, cap=8 << 20, TBV_CODEC=1, TBV_CODEC_MIN=64 << 10, TBV_MERGE=one_launch, TBV_NSLOT=3) as tbv:
        k = 0
        for name in ("bf16", "f16", "f32"):
            dt, code = DTS[name]
            esz = 4 if name == "f32" else 2
            # whole superblocks; a last superblock of 3 vectors; a last group of one vector; the cap
            for nb in (1 << 20, (1 << 20) + 48, (256 << 10) + 4096 + 16, 8 << 20):
                n = nb // esz
                k += 1
                a = torch.from_numpy(synth.normal(120 + k, n) * 0.02).to(dt); b = torch.from_numpy(synth.normal(160 + k, n) * 0.02).to(dt)
                A, B = a.cuda(), b.cuda()
                wa, wb = oracle.q8_encode(code, bits(a)), oracle.q8_encode(code, bits(b))
                want = oracle.q8_sum(code, wa, wb, n)
                tbv.peer_resident(B)
                for rep in range(4):                               # every ring slot, and one of them twice
                    out = torch.zeros_like(A)
                    say("coded step", "one launch" if one_launch else "two launches", name, nb, "rep", rep)
                    assert tbv.all_reduce(A, out)
                    torch.cuda.synchronize()
                    assert np.array_equal(bits(out), want), (name, nb, rep)
                    img = torch.empty(wa.size, dtype=torch.uint8, device="cuda")
                    assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), wa.size, 3) == 0
                    assert np.array_equal(img.cpu().numpy(), wa), (name, nb, rep, "image")
                x = A.clone()
                assert tbv.all_reduce(x)                           # in place
                torch.cuda.synchronize()
                assert np.array_equal(bits(x), want), (name, nb, "in place")
                assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), wa.size, 3) == 0
                assert np.array_equal(img.cpu().numpy(), wa), (name, nb, "image of the in-place call")
                tbv.peer_resident(None)
        # hand-made groups: min 0 and max 255 make the step exactly 1, so k + 0.5 lands on a rounding tie (to even) for
        # every k; a second kind of group holds a huge pair of values, which pushes everything else to the middle code
        ties = np.concatenate([[0.0, 255.0], np.arange(126) + 0.5]).astype(np.float32)
        spike = np.concatenate([[-1.0e38, 1.0e38], np.linspace(-1, 1, 126)]).astype(np.float32)
        pat = np.concatenate([ties, spike, ties[::-1], -ties])
        a = torch.from_numpy(np.tile(pat, 128)).to(torch.bfloat16); b = torch.from_numpy(np.tile(pat[::-1].copy(), 128)).to(torch.bfloat16)
        A, B = a.cuda(), b.cuda()
        wa, wb = oracle.q8_encode(2, bits(a)), oracle.q8_encode(2, bits(b))
        codes = wa[128:128 + 128]                                  # first group's codes: 0, 255, then the ties
        assert list(codes[:6]) == [0, 255, 0, 2, 2, 4], list(codes[:8])
        tbv.peer_resident(B)
        out = torch.zeros_like(A)
        say("coded step, hand-made groups")
        assert tbv.all_reduce(A, out)
        torch.cuda.synchronize()
        img = torch.empty(wa.size, dtype=torch.uint8, device="cuda")
        assert hip.hipMemcpy(img.data_ptr(), tbv.lib().tbv_emu_send_slot(tbv.seq() % 3), wa.size, 3) == 0
        assert np.array_equal(img.cpu().numpy(), wa), "image of the hand-made groups"
        assert np.array_equal(bits(out), oracle.q8_sum(2, wa, wb, a.numel())), "sum of the hand-made groups"
        tbv.peer_resident(None)
        assert not tbv.err()
