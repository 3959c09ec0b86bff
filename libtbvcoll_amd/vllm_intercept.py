"""Route a tensor-parallel group's all-reduce through libtbvcoll.

Counterpart of the reference's vLLM patch (step3b/vllm_tp_bench.py:77-140): replace
`GroupCoordinator.all_reduce` of vLLM's `parallel_state` module so that calls of the
tensor-parallel group go through `tbv_ar_allreduce`, and everything the library
does not take (other groups, world size 1, unsupported dtype, non-contiguous
input, payload over the cap = rc -2) falls through to the original method, i.e.
to RCCL.  Behaviour kept from the reference:

  * the TP group is recognised by `unique_name`, resolved once through
    `get_tp_group()`;
  * initialisation is lazy (first TP call) unless `eager=True`;
  * the raw ctypes function is bound once; the current stream is read on every
    call (a cached stream handle goes stale when vLLM switches streams and
    corrupts results silently);
  * out-of-place: a fresh `empty_like` output per call;
  * rc 0 -> return the output; rc -2 -> count a fallback and call the original;
    any other rc -> RuntimeError;
  * counters: handled calls, fallbacks, Python-side seconds.

`output_hash` is the reference's end-to-end gate: sha256 over the generated token
ids of a round, first 16 hex digits (step3b/vllm_tp_bench.py:176-183); a run
through this library must print the same hash as a run through RCCL.

The module takes the `parallel_state` module as an argument, so it imports
neither vLLM nor anything else that is absent from this image.
"""
import hashlib
import time

import torch

from . import tbvcoll

_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


class Intercept:
    def __init__(self, ps, rank, devs, peer_ip="", port=18996, cap_bytes=8 << 20, eager=False, lib=tbvcoll):
        self.ps, self.rank, self.devs, self.peer_ip, self.port, self.cap_bytes = ps, rank, devs, peer_ip, port, cap_bytes
        self.lib = lib
        self.orig = ps.GroupCoordinator.all_reduce
        self.tp_name = None            # None: not resolved yet; False: no TP group
        self.fn = None
        self.cap = 0
        self.counters = {"n": 0, "fallback": 0, "py": 0.0}
        me = self

        def patched_all_reduce(group, input_):
            return me._all_reduce(group, input_)

        self.patched = patched_all_reduce
        ps.GroupCoordinator.all_reduce = patched_all_reduce
        if eager:
            self._init()

    def _init(self):
        self.lib.init(self.rank, self.devs, self.peer_ip if self.rank == 1 else "", port=self.port, cap_bytes=self.cap_bytes)
        self.fn = self.lib.raw_fn()
        self.cap = self.lib.cap()

    def _all_reduce(self, group, input_):
        if group.world_size == 1:
            return input_
        if self.tp_name is None:
            try:
                self.tp_name = self.ps.get_tp_group().unique_name
            except Exception:
                self.tp_name = False
        if self.tp_name and group.unique_name == self.tp_name:
            if self.fn is None:
                self._init()
            t0 = time.perf_counter()
            dt = _DT.get(input_.dtype)
            nb = input_.numel() * input_.element_size()
            if dt is not None and nb <= self.cap and input_.is_contiguous():
                out = torch.empty_like(input_)
                rc = self.fn(input_.data_ptr(), out.data_ptr(), nb, dt, torch.cuda.current_stream().cuda_stream)
                self.counters["py"] += time.perf_counter() - t0
                if rc == 0:
                    self.counters["n"] += 1
                    return out
                if rc != -2:
                    raise RuntimeError(f"tbv_ar_allreduce rc={rc}")
            else:
                self.counters["py"] += time.perf_counter() - t0
            self.counters["fallback"] += 1
        return self.orig(group, input_)

    def all_reduce_rmsnorm(self, group, input_, weight, eps):
        """The tensor-parallel all-reduce of `input_` and the RMSNorm of its result (what every decoder layer does
        next; the reference plans the fusion, reports/12_references.md:136): returns (reduced, normed).  Goes through
        `tbv_ar_allreduce_rmsnorm` when the library takes the call (TP group, supported dtype and layout, rows of at
        most 64 KiB, payload within the cap); otherwise the all-reduce goes the usual way (library or original) and the
        norm is computed here in fp32, the formula vLLM's own kernel implements.  The fused kernel's `normed` is
        within 2 ulp of that formula, so an output-hash comparison between a fused and an unfused run may differ."""
        if group.world_size > 1 and self.tp_name is None:
            try:
                self.tp_name = self.ps.get_tp_group().unique_name
            except Exception:
                self.tp_name = False
        fused = getattr(self.lib, "all_reduce_rmsnorm", None)
        if (fused is not None and group.world_size > 1 and self.tp_name and group.unique_name == self.tp_name
                and input_.dtype in _DT and input_.is_contiguous() and input_.dim() >= 1
                and weight.dtype is input_.dtype and weight.is_contiguous() and weight.numel() == input_.shape[-1]):
            if self.fn is None:
                self._init()
            t0 = time.perf_counter()
            out = torch.empty_like(input_)
            normed = fused(input_, weight, eps, out=out)
            self.counters["py"] += time.perf_counter() - t0
            if normed is not None:
                self.counters["n"] += 1
                self.counters["fused_norm"] = self.counters.get("fused_norm", 0) + 1
                return out, normed
        reduced = self._all_reduce(group, input_)
        x = reduced.float()
        normed = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)).to(reduced.dtype) * weight
        return reduced, normed

    def report(self):
        """Counters plus the library's per-call averages (resets the latter), as the reference prints at the end."""
        r = dict(self.counters)
        if self.fn is not None:
            pre, xfer, post, enq, drain, n = self.lib.stats5()
            r.update(mode="ASYNC" if self.lib.is_async() else "SYNC", xfer_us=xfer, enq_us=enq, drain_us=drain,
                     pre_us=pre, post_us=post,
                     wrapper_us=r["py"] / max(1, r["n"]) * 1e6 - enq)
        return r

    def uninstall(self):
        if self.ps.GroupCoordinator.all_reduce is self.patched:
            self.ps.GroupCoordinator.all_reduce = self.orig


def install(ps, rank, devs, peer_ip="", port=18996, cap_bytes=8 << 20, eager=False, lib=tbvcoll):
    """Patch `ps.GroupCoordinator.all_reduce`; returns the Intercept (call `.uninstall()` to undo)."""
    return Intercept(ps, rank, devs, peer_ip, port, cap_bytes, eager, lib)


def output_hash(token_id_lists):
    """sha256 over str(list(ids)) of every output of a round, first 16 hex digits."""
    blob = b"".join(bytes(str(list(ids)), "utf8") for ids in token_id_lists)
    return hashlib.sha256(blob).hexdigest()[:16]
