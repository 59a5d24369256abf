"""Python face of the swap engine (C++: cswap_amd/csrc/swap_engine.cpp).

``SwapEngine`` mirrors the reference's ``Execution`` object
(CSWAP+/Execution.h:38-446): ``pre`` kicks compression + the asynchronous copy
to pinned host memory for a tensor, ``post`` waits for that copy after the
layer's compute was launched; ``swap_in`` is the backward-side mirror the
reference keeps inside its patched autograd engine.
"""
from __future__ import annotations

import ctypes as C
import time

import torch

from ._lib import Choice, Costs, EngineConfig, TicketInfo, TicketTiming, check, lib
from .workloads import field_dims

AUTO, NONE, SPARSE, ZFP = -1, 2, 3, 6
AUTO_SPARSE = -3   # the selector for a tensor expected to be sparse: the compaction itself is its probe
POLICY_NAME = {NONE: "none", SPARSE: "sparse", ZFP: "zfp"}


def default_costs() -> Costs:
    c = Costs()
    lib().cswap_costs_default(C.byref(c))
    return c


def select(n: int, nnz: int, maxbits: int = 512, costs: Costs | None = None) -> Choice:
    ch = Choice()
    check(lib().cswap_select(n, nnz, maxbits, C.byref(costs) if costs is not None else None, C.byref(ch)),
          "cswap_select")
    return ch


def select_field(nx: int, ny: int, nz: int, nnz: int, maxbits: int = 512, costs: Costs | None = None) -> Choice:
    ch = Choice()
    check(lib().cswap_select_field(nx, ny, nz, nnz, maxbits, C.byref(costs) if costs is not None else None,
                                   C.byref(ch)), "cswap_select_field")
    return ch


class SwapEngine:
    def __init__(self, pinned_bytes: int = 1 << 30, device_bytes: int = 1 << 30, maxbits: int = 512,
                 process: int = 0, max_tickets: int = 256, costs: Costs | None = None, timing: bool = False):
        cfg = EngineConfig()
        lib().cswap_engine_config_default(C.byref(cfg))
        cfg.pinned_pool_bytes = pinned_bytes
        cfg.device_pool_bytes = device_bytes
        cfg.zfp_maxbits = maxbits
        cfg.process = process
        cfg.max_tickets = max_tickets
        if costs is not None:
            cfg.costs = costs
        cfg.timing = 1 if timing else 0
        self._h = C.c_void_p()
        check(lib().cswap_engine_create(C.byref(self._h), C.byref(cfg)), "cswap_engine_create")

    def close(self):
        if self._h:
            lib().cswap_engine_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def calibrate(self) -> Costs:
        c = Costs()
        check(lib().cswap_engine_calibrate(self._h, C.byref(c)), "cswap_engine_calibrate")
        return c

    # Execution::pre
    def pre(self, t: torch.Tensor, policy: int = AUTO) -> int:
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
            raise ValueError("expected a contiguous fp32 device tensor")
        nx, ny, nz = field_dims(t.shape)
        ticket = C.c_int(-1)
        check(lib().cswap_swap_out(self._h, t.data_ptr(), nx, ny, nz, policy,
                                   torch.cuda.current_stream().cuda_stream, C.byref(ticket)), "cswap_swap_out")
        return ticket.value

    # Execution::post
    def post(self, ticket: int) -> None:
        check(lib().cswap_swap_wait(self._h, ticket), "cswap_swap_wait")

    def swap_in(self, ticket: int, out: torch.Tensor) -> torch.Tensor:
        check(lib().cswap_swap_in(self._h, ticket, out.data_ptr(), torch.cuda.current_stream().cuda_stream),
              "cswap_swap_in")
        return out

    def tune(self, numel: int) -> int:
        """Measure the best ZVC chunk count for tensors of about ``numel`` elements
        (used from then on when the engine was created with ``process=0``)."""
        best = C.c_int(0)
        check(lib().cswap_engine_tune(self._h, numel, C.byref(best)), "cswap_engine_tune")
        return best.value

    def probe_count(self) -> int:
        """Counting passes with a host round trip the engine has run so far."""
        return lib().cswap_engine_probe_count(self._h)

    def process_for(self, numel: int) -> int:
        return lib().cswap_engine_process_for(self._h, numel)

    def prefetch(self, ticket: int) -> None:
        """Start the host-to-device copy of a swapped tensor ahead of its swap_in."""
        check(lib().cswap_swap_prefetch(self._h, ticket), "cswap_swap_prefetch")

    def release(self, ticket: int) -> None:
        check(lib().cswap_swap_release(self._h, ticket), "cswap_swap_release")

    def timing(self, ticket: int) -> TicketTiming:
        """Phase times of the ticket in microseconds, from the engine's own events
        (engines created with ``timing=True``); -1 = not finished yet."""
        t = TicketTiming()
        check(lib().cswap_swap_timing(self._h, ticket, C.byref(t)), "cswap_swap_timing")
        return t

    def info(self, ticket: int) -> TicketInfo:
        i = TicketInfo()
        check(lib().cswap_swap_info(self._h, ticket, C.byref(i)), "cswap_swap_info")
        return i


def _dummy_compute(a: torch.Tensor, b: torch.Tensor, reps: int) -> None:
    """Stand-in for the layer's kernels that run while the copy is in flight."""
    for _ in range(reps):
        torch.mm(a, b)


def bench_schedule(dev, batch: int = 128, seed: int = 0) -> dict:
    """Configuration 4: walk the VGG-16 activation schedule; per tensor, swap out
    (probe + select + compress + D2H on the copy stream, overlapped with a dummy
    compute stream) and back in, against the raw (policy 2) swap."""
    from .workloads import config4_schedule, config4_tensor

    sched = config4_schedule(batch)
    biggest = max(int(torch.tensor(e["shape"]).prod()) for e in sched) * 4
    eng = SwapEngine(pinned_bytes=2 * biggest + (64 << 20), device_bytes=2 * biggest + (64 << 20))
    costs = eng.calibrate()
    a = torch.randn(2048, 2048, device=dev)
    b = torch.randn(2048, 2048, device=dev)
    rows = []
    tot = {"auto": 0.0, "none": 0.0}
    worst = 0.0
    for e in sched:
        x = torch.from_numpy(config4_tensor(e, seed)).to(dev)
        out = torch.empty_like(x)
        lat = {}
        chosen = None
        for label, pol in (("none", NONE), ("auto", AUTO)):
            best = None
            for _ in range(5):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                tk = eng.pre(x, pol)
                _dummy_compute(a, b, 2)
                eng.post(tk)
                eng.swap_in(tk, out)
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                info = eng.info(tk)
                eng.release(tk)
                best = (t1 - t0) if best is None else min(best, t1 - t0)
            lat[label] = best * 1e3
            if label == "auto":
                chosen = info
        # dummy compute alone, to report how much of it the swap hides
        torch.cuda.synchronize()
        t0 = time.perf_counter(); _dummy_compute(a, b, 2); torch.cuda.synchronize()
        comp_ms = (time.perf_counter() - t0) * 1e3
        rows.append({"id": e["id"], "kind": e["kind"], "shape": list(e["shape"]), "MB": round(x.numel() * 4 / 1e6, 1),
                     "policy": POLICY_NAME[chosen.policy], "ratio": round(chosen.bytes_out / chosen.bytes_in, 4),
                     "none_ms": round(lat["none"], 3), "auto_ms": round(lat["auto"], 3),
                     "compute_ms": round(comp_ms, 3)})
        tot["auto"] += lat["auto"]; tot["none"] += lat["none"]
        if chosen.policy != NONE:
            worst = max(worst, lat["auto"] / lat["none"])
        del x, out
    eng.close()
    return {"costs": {k: round(getattr(costs, k), 2) for k, _ in Costs._fields_ if k.endswith(("gbs", "us"))},
            "total_none_ms": round(tot["none"], 2), "total_auto_ms": round(tot["auto"], 2),
            "worst_compressed_over_raw": round(worst, 3), "tensors": rows}


def bench_backward(dev, batch: int = 128, seed: int = 0, compute_reps: int = 2) -> dict:
    """Configuration 4, backward side: every swapped tensor of the schedule is
    already on the host; walk them in reverse (the order backward asks for them),
    each followed by a dummy layer backward on the compute stream.  Compared:
    raw tensors fetched on demand, compressed tensors fetched on demand, and
    compressed tensors with the next one prefetched under the current layer."""
    from .workloads import config4_schedule, config4_tensor

    sched = [e for e in config4_schedule(batch) if e["kind"] != "dense"]   # the swapped ones: ReLU and pool outputs
    total = sum(int(torch.tensor(e["shape"]).prod()) * 4 for e in sched)
    biggest = max(int(torch.tensor(e["shape"]).prod()) for e in sched) * 4
    eng = SwapEngine(pinned_bytes=total + (64 << 20), device_bytes=4 * biggest + (64 << 20))
    eng.calibrate()
    a = torch.randn(2048, 2048, device=dev)
    b = torch.randn(2048, 2048, device=dev)
    xs = [torch.from_numpy(config4_tensor(e, seed)).to(dev) for e in sched]
    outs = [torch.empty_like(x) for x in xs]
    res = {}
    for label, pol, ahead in (("raw_on_demand", NONE, 0), ("compressed_on_demand", AUTO, 0),
                              ("compressed_prefetch_1", AUTO, 1), ("raw_prefetch_1", NONE, 1)):
        best = None
        for _ in range(3):
            tks = []
            for x in xs:
                tk = eng.pre(x, pol)
                eng.post(tk)
                tks.append(tk)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            order = list(range(len(xs)))[::-1]
            if ahead:
                eng.prefetch(tks[order[0]])
            for k, i in enumerate(order):
                if k >= 2:
                    eng.release(tks[order[k - 2]])      # its decompression finished a layer ago
                for j in order[k + 1:k + 1 + ahead]:
                    eng.prefetch(tks[j])
                eng.swap_in(tks[i], outs[i])
                _dummy_compute(a, b, compute_reps)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            for i in order[-2:]:
                eng.release(tks[i])
            best = dt if best is None else min(best, dt)
        res[label + "_ms"] = round(best * 1e3, 2)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in xs:
        _dummy_compute(a, b, compute_reps)
    torch.cuda.synchronize()
    res["compute_only_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
    res["tensors"] = len(xs)
    res["MB"] = round(total / 1e6, 1)
    eng.close()
    return res
