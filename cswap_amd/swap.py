"""Python face of the swap engine (C++: cswap_amd/csrc/swap_engine.cpp).

``SwapEngine`` mirrors the reference's ``Execution`` object
(CSWAP+/Execution.h:38-446): ``pre`` kicks compression + the asynchronous copy
to pinned host memory for a tensor, ``post`` waits for that copy after the
layer's compute was launched; ``swap_in`` is the backward-side mirror the
reference keeps inside its patched autograd engine.
"""
from __future__ import annotations

import ctypes as C

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

    def set_maxbits(self, maxbits: int) -> None:
        """ZFP bits per 4x4x4 block for the swap-outs from now on (setRatio: CSWAP+/Execution.h:63;
        tensors already out come back with the rate they went out with)."""
        check(lib().cswap_engine_set_zfp_maxbits(self._h, maxbits), "cswap_engine_set_zfp_maxbits")

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
