"""Python mirror of the reference's swap scheduler ``class Execution``
(CSWAP+/Execution.h:38-446) over the swap engine; same semantics as the
header-only C++ mirror ``include/cswap_execution.hpp``.

Tensors are identified by the index of the op that produced them; tensor ``i``
is swapped out when the running op index reaches ``begin_stage[i]`` (default
``i + 1``, the op that consumes it) with the action ``policy[i]``: 0 keep,
2 raw swap, 3 ZVC, 6 ZFP, -1 selector.
"""
from __future__ import annotations

import torch

from . import swap

CONV, POOL, ACT, BN, FC, MASKFILL = range(6)   # Layer_type, CSWAP+/Execution.h:28-35


class Execution:
    def __init__(self, engine: "swap.SwapEngine"):
        self.engine = engine
        self.index = -1
        self.policy: list[int] = []
        self.begin_stage: list[int] = []
        self._tickets: dict[int, tuple[int, tuple]] = {}
        self._pending: list[int] = []

    def init_(self, n: int) -> None:
        self.policy = [0] * n
        self.begin_stage = [i + 1 for i in range(n)]

    def init(self) -> None:
        self.index = -1

    def preforward(self) -> None:
        self.init()

    def postforward(self) -> None:
        pass

    def pre(self, tensor, tensor_id=None, layer_type: int = ACT) -> None:
        """``pre(tensor, tensor_id)`` for an op with one input, or
        ``pre([(tensor, tensor_id), ...])`` for an op with several (concatenation,
        residual add; Execution.h:135-212): the op index advances once and every
        input whose ``begin_stage`` is this op goes out under its own policy."""
        inputs = [(tensor, tensor_id)] if isinstance(tensor, torch.Tensor) else list(tensor)
        self.index += 1
        self._pending = []
        for t, tid in inputs:
            if tid is None or tid < 0 or tid >= len(self.policy):
                continue
            pol = self.policy[tid]
            if self.index != self.begin_stage[tid] or pol in (0, 1) or tid in self._tickets:
                continue
            ticket = self.engine.pre(t, pol)
            self._tickets[tid] = (ticket, tuple(t.shape))
            self._pending.append(tid)

    def post(self) -> int:
        """Wait for the copies the matching ``pre`` started; returns the id of the
        op's output tensor (``x.tensor_id = index``, Execution.h:219)."""
        for tid in self._pending:
            self.engine.post(self._tickets[tid][0])
        self._pending = []
        return self.index

    def swapped(self, tensor_id: int) -> bool:
        return tensor_id in self._tickets

    def com_and_tran(self, tensor_id: int) -> int:
        if tensor_id not in self._tickets:
            return 0
        return self.engine.info(self._tickets[tensor_id][0]).policy

    def prefetch(self, tensor_id: int) -> None:
        """Start the inbound copy of a tensor that a later fetch() will ask for."""
        self.engine.prefetch(self._tickets[tensor_id][0])

    def fetch(self, tensor_id: int, out: torch.Tensor | None = None) -> torch.Tensor:
        ticket, shape = self._tickets.pop(tensor_id)
        if out is None:
            out = torch.empty(shape, dtype=torch.float32, device="cuda")
        self.engine.swap_in(ticket, out)
        self.engine.release(ticket)
        return out
