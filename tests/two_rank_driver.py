#!/usr/bin/env python3
"""One rank of a two-process run on one GPU, in the shape of the reference's own drivers
(step4/test_exact.py:9-35 and step4/test_stress.py:8-42): the module is imported as plain `tbvcoll`,
the rank comes from RANK, rank 1 gets rank 0's address in PEER_IP, and no call hands the library
the peer's payload.  Both ranks derive both inputs from seeds, so each can check its result against
the exact sum without a second collective.  Prints one JSON line.

    MODE=exact   every dtype x {57344, 229376, 1048576} bytes, cap 4 MiB, out of place on a temporary,
                 synchronised per call; compared with the storage-type add and the fp32 add
    MODE=stress  ITERS back-to-back out-of-place calls of BYTES bytes in DT without any synchronisation,
                 inputs and outputs kept, everything compared after one final synchronisation
"""
import json
import os
import sys

import torch

import tbvcoll      # the binding beside libtbvcoll.so, found through PYTHONPATH exactly as a reference driver finds its own

rank = int(os.environ["RANK"])
mode = os.environ.get("MODE", "exact")
torch.cuda.set_device(0)
DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def from_seed(seed, numel):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.rand(numel, generator=g, device="cuda", dtype=torch.float32) - 0.5) * 10


res = {"rank": rank, "mode": mode}
if mode == "exact":
    tbvcoll.init(rank, os.environ.get("DEVS", "rail0,rail1"), os.environ.get("PEER_IP", ""), port=int(os.environ["PORT"]), cap_bytes=4 << 20)
    cells = []
    for name, dt in DT.items():
        for nb in (57344, 229376, 1048576):
            numel = nb // (4 if dt == torch.float32 else 2)
            f0, f1 = from_seed(1234, numel), from_seed(1235, numel)
            mine = (f0 if rank == 0 else f1).to(dt)
            out = torch.empty_like(mine)
            assert tbvcoll.all_reduce(mine.clone(), out), (name, nb)
            torch.cuda.synchronize()
            same_dt = bool(torch.equal(out, f0.to(dt) + f1.to(dt)))
            same_32 = bool(torch.equal(out, (f0.to(dt).float() + f1.to(dt).float()).to(dt)))
            cells.append({"dtype": name, "bytes": nb, "same_dt": same_dt, "same_f32": same_32})
    # in place, and a call over the cap (declined: the caller would fall back)
    f0, f1 = from_seed(77, 1 << 19), from_seed(78, 1 << 19)
    x = (f0 if rank == 0 else f1).to(torch.bfloat16)
    assert tbvcoll.all_reduce(x)
    torch.cuda.synchronize()
    res["in_place_same"] = bool(torch.equal(x, f0.to(torch.bfloat16) + f1.to(torch.bfloat16)))
    res["over_cap_declined"] = tbvcoll.all_reduce(torch.zeros((4 << 20) // 2 + 8, dtype=torch.bfloat16, device="cuda")) is False
    res["cells"] = cells
    res["ok"] = all(c["same_dt"] and c["same_f32"] for c in cells) and res["in_place_same"] and res["over_cap_declined"]
else:
    nb = int(os.environ.get("BYTES", "57344"))
    iters = int(os.environ.get("ITERS", "500"))
    dt = DT[os.environ.get("DT", "bf16")]
    tbvcoll.init(rank, os.environ.get("DEVS", "rail0,rail1"), os.environ.get("PEER_IP", ""), port=int(os.environ["PORT"]),
                 cap_bytes=int(os.environ.get("CAP", str(nb))))
    numel = nb // (4 if dt == torch.float32 else 2)

    def inp(it, r):
        return from_seed(it * 2 + r, numel).to(dt)

    kept = []
    for it in range(iters):
        x = inp(it, rank)
        out = torch.empty_like(x)
        assert tbvcoll.all_reduce(x, out), it
        kept.append((x, out))                      # the input too: a reused allocation would fake a mismatch
    torch.cuda.synchronize()
    bad = [it for it, (_, out) in enumerate(kept) if not torch.equal(out, inp(it, 0) + inp(it, 1))]
    res.update({"bytes": nb, "iters": iters, "bad": len(bad), "first_bad": bad[0] if bad else None, "async": tbvcoll.is_async(),
                "ok": not bad})
res["err"] = tbvcoll.err()
res["ok"] = bool(res["ok"]) and not res["err"]
print("RESULT " + json.dumps(res), flush=True)
sys.exit(0 if res["ok"] else 1)
