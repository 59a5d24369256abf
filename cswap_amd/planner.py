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


# ------------------------------------------------------------------ the walk of the reference's drivers
def run_planned_iteration(engine, mods, x, policy, begin_stage, backward_factor: int = 2, check=None,
                          keep=None):
    """One iteration of the walk the reference's drivers do: forward with
    Execution.pre/post around every op, then the ops in reverse, each standing in
    for its backward by running ``backward_factor`` times, with the swapped input
    fetched back first and the next one prefetched.  ``keep`` (a dict) receives a
    clone of every tensor at the moment it is swapped out and ``check(id, tensor)``
    is called with every tensor fetched back (both for tests).  Returns seconds."""
    import time

    import torch

    from .execution import ACT, Execution

    exe = Execution(engine)
    exe.init_(len(mods) + 1)
    exe.policy[:len(policy)] = policy
    exe.begin_stage[:len(begin_stage)] = begin_stage
    acts = {}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    with torch.no_grad():
        exe.preforward()
        pre, pre_id = x, -1
        for i, m in enumerate(mods):
            exe.pre(pre, pre_id, ACT)
            out = m(pre)
            exe.post()
            if exe.swapped(pre_id):
                if keep is not None:
                    keep[pre_id] = pre.clone()
                acts[pre_id] = None           # the device copy may go: the storage is dropped here
            else:
                acts[pre_id] = pre
            pre, pre_id = out, i
        exe.postforward()
        # backward order: op i needs its input, tensor i-1
        order = [i - 1 for i in range(len(mods) - 1, 0, -1)]
        swapped = [t for t in order if exe.swapped(t)]
        k = 0
        if swapped:
            exe.prefetch(swapped[0])
        for i in range(len(mods) - 1, 0, -1):
            tid = i - 1
            if exe.swapped(tid):
                k += 1
                if k < len(swapped):
                    exe.prefetch(swapped[k])
                inp = exe.fetch(tid)
                if check is not None:
                    check(tid, inp)
            else:
                inp = acts[tid]
            for _ in range(backward_factor):
                mods[i](inp)
    torch.cuda.synchronize()
    return time.perf_counter() - t0
