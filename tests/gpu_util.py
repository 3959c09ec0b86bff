"""Helpers shared by the GPU parity tests."""
import contextlib
import os
import sys

import numpy as np
import torch

from libtbvcoll_amd import synth, tbvcoll

TBV_KEYS = ("TBV_ASYNC", "TBV_GPUSIG", "TBV_KWAIT", "TBV_NSLOT", "TBV_CHUNK", "TBV_RAIL1MAX", "TBV_CPU", "TBV_WDOG",
            "TBV_TAG", "TBV_UNCACHED", "TBV_RAILSUM", "TBV_FUSE", "TBV_FUSEWAIT", "TBV_UNROLL", "TBV_GRIDCAP", "TBV_BLOCK",
            "TBV_PACKSIG", "TBV_DEFERSIG", "TBV_WIRE", "TBV_ONEKERNEL", "TBV_MERGE", "TBV_MERGEMAX", "TBV_STREAMING", "TBV_CODEC", "TBV_CODEC_MIN")
DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def say(*a):
    """Name the case before touching the GPU, flushed, so a lost box still tells which case ran."""
    print("[case]", *a, flush=True)
    sys.stdout.flush()


@contextlib.contextmanager
def session(rails=2, cap=4 << 20, **env):
    """(Re)initialise the library with the given TBV_* settings; tear it down afterwards."""
    tbvcoll.shutdown()
    for k in TBV_KEYS:
        os.environ.pop(k, None)
    env.setdefault("TBV_NSLOT", 4)
    env.setdefault("TBV_WDOG", 5)
    for k, v in env.items():
        os.environ[k] = str(v)
    say("init", "rails", rails, "cap", cap, env)
    tbvcoll.init(0, ",".join(f"rail{i}" for i in range(rails)), "", cap_bytes=cap)
    try:
        yield tbvcoll
    finally:
        torch.cuda.synchronize()
        tbvcoll.shutdown()
        for k in env:
            os.environ.pop(k, None)


def dev(x_np, dtype):
    """fp32 numpy -> tensor of `dtype` on the GPU (round to nearest even, done by torch on the CPU)."""
    return torch.from_numpy(x_np).to(dtype).cuda()


def bits_np(t):
    t = t.detach().contiguous().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy().view(np.uint32)


def same_bits(a, b):
    return np.array_equal(bits_np(a), bits_np(b))


def first_diff(a, b):
    x, y = bits_np(a).reshape(-1), bits_np(b).reshape(-1)
    bad = np.nonzero(x != y)[0]
    return None if bad.size == 0 else (int(bad[0]), int(bad.size), hex(int(x[bad[0]])), hex(int(y[bad[0]])))
