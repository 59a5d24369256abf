"""Planner: which activations leave the device, and how, under a memory target.

Python face of ``cswap_planner_*`` with the method names the reference's model
drivers call on ``c10::GetPolicyMaker()`` (CSWAP+/inception-v3-cifar100.cpp:207-214,
CSWAP+/vgg16-cifar10.cpp:474-497, CSWAP+/resnet-cifar10.cpp:330): record one
profiled iteration with ``add_comptime`` / ``add_tensor`` / ``add_stepdep`` /
``add_omitid``, fix the target with ``init(ratio)``, then ``make_policy()`` (or the
raw-swap baseline ``capuchin()``) returns one action per tensor for
``Execution.policy`` and the predicted iteration time.  The reference's own
planner is not in its tree; the cost model here is this library's.
"""
from __future__ import annotations

import ctypes as C

from ._lib import Costs, PlanSummary, check, lib


class PolicyMaker:
    def __init__(self, costs: Costs | None = None, zfp_maxbits: int = 512):
        self._h = lib().cswap_planner_create(C.byref(costs) if costs is not None else None, zfp_maxbits)
        if not self._h:
            raise MemoryError("cswap_planner_create")
        self.summary = PlanSummary()
        self.begin_stage: list[int] = []

    def close(self) -> None:
        if self._h:
            lib().cswap_planner_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def reset(self) -> None:
        check(lib().cswap_planner_reset(self._h), "cswap_planner_reset")

    def set_backward_factor(self, factor: float) -> None:
        check(lib().cswap_planner_set_backward_factor(self._h, factor), "cswap_planner_set_backward_factor")

    # -- profile of one iteration (names as in the reference's drivers)
    def add_comptime(self, microseconds: float) -> None:
        check(lib().cswap_planner_add_comptime(self._h, microseconds), "cswap_planner_add_comptime")

    def add_tensor(self, index: int, nbytes: int) -> None:
        check(lib().cswap_planner_add_tensor(self._h, index, nbytes), "cswap_planner_add_tensor")

    def add_stepdep(self, dep) -> None:
        """``add_stepdep([pre.tensor_id, index])``: op ``index`` consumes tensor ``pre.tensor_id``."""
        check(lib().cswap_planner_add_stepdep(self._h, int(dep[0]), int(dep[1])), "cswap_planner_add_stepdep")

    def add_omitid(self, index: int) -> None:
        check(lib().cswap_planner_add_omitid(self._h, index), "cswap_planner_add_omitid")

    def set_field(self, index: int, nx: int, ny: int, nz: int) -> None:
        check(lib().cswap_planner_set_field(self._h, index, nx, ny, nz), "cswap_planner_set_field")

    def set_nnz(self, index: int, nnz: int) -> None:
        check(lib().cswap_planner_set_nnz(self._h, index, nnz), "cswap_planner_set_nnz")

    # -- planning
    def init(self, ratio: float) -> None:
        check(lib().cswap_planner_init(self._h, ratio), "cswap_planner_init")

    def _plan(self, fn, n: int):
        pol = (C.c_int * n)()
        beg = (C.c_int * n)()
        check(fn(self._h, pol, beg, n, C.byref(self.summary)), "cswap_planner plan")
        self.begin_stage = list(beg)
        return list(pol), self.summary.time_us

    def make_policy(self, n: int):
        """Returns (policy list for ``Execution.policy``, predicted iteration time in microseconds)."""
        return self._plan(lib().cswap_planner_make_policy, n)

    def capuchin(self, n: int):
        return self._plan(lib().cswap_planner_capuchin, n)
