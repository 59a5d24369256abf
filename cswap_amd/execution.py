"""Python mirror of the reference's swap scheduler ``class Execution``
(CSWAP+/Execution.h:38-446) over the swap engine; same semantics as the
header-only C++ mirror ``include/cswap_execution.hpp``.

Tensors are identified by the index of the op that produced them; tensor ``i``
is dealt with when the running op index reaches ``begin_stage[i]`` (default
``i + 1``, the op that consumes it), in the reference's branch order:
``policy[i] == 1``, or ``policy_ == 4`` and a consumer that is not a convolution
-> dropped for recomputation, tag 1 (Execution.h:243); ``policy[i] == 2``, or a
convolution consumer and ``policy_ > 2`` (the vDNN and SuperNeurons modes) -> raw
swap (Execution.h:70); 3 -> ZVC (Execution.h:86); 6 -> ZFP (Execution.h:107);
-1 (added here) -> the selector decides, and a ZFP or raw decision is remembered
for the next ``recheck`` iterations so that they skip the probe.
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
        self.policy_ = 1            # 1 this scheme, 2 Capuchin, 3 vDNN, 4 SuperNeurons (Execution.h:420)
        self.recheck = 16           # iterations a remembered selector decision is reused; 0 = never
        self.memo_hits = 0
        self._tickets: dict[int, tuple[int, tuple]] = {}
        self._dropped: set[int] = set()
        self._memo: dict[int, list] = {}    # tensor id -> [numel, policy, uses]
        self._pending: list[int] = []

    def init_(self, n: int) -> None:
        self.policy = [0] * n
        self.begin_stage = [i + 1 for i in range(n)]

    def init(self) -> None:
        self.index = -1

    def setRatio(self, ratio: int) -> None:  # noqa: N802 (the reference's name, CSWAP+/Execution.h:63)
        """4 * ratio bits per 4x4x4 block for the ZFP swap-outs from now on (128: a quarter of fp32)."""
        self.engine.set_maxbits(4 * int(ratio))

    def preforward(self) -> None:
        self.init()
        self._dropped.clear()

    @staticmethod
    def action(entry: int, mode: int, layer_type: int) -> int:
        """0 keep, 1 drop, 2 raw swap, 3 ZVC, 6 ZFP, -1 selector
        (Execution.h:70,86,107,243)."""
        if entry == 1 or (mode == 4 and layer_type != CONV):
            return 1
        if entry == 2 or (layer_type == CONV and mode > 2):
            return swap.NONE
        return entry if entry in (swap.SPARSE, swap.ZFP, swap.AUTO) else 0

    def forget(self) -> None:
        self._memo.clear()

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
            if self.index != self.begin_stage[tid] or tid in self._tickets or tid in self._dropped:
                continue
            act = self.action(self.policy[tid], self.policy_, layer_type)
            if act == 0:
                continue
            if act == 1:
                self._dropped.add(tid)
                continue
            remember = False
            if act == swap.AUTO and self.recheck > 0:
                m = self._memo.get(tid)
                if m and m[0] == t.numel() and m[2] < self.recheck and m[1] in (swap.ZFP, swap.NONE):
                    act = m[1]
                    m[2] += 1
                    self.memo_hits += 1
                else:
                    remember = True
                    if m and m[0] == t.numel() and m[1] == swap.SPARSE:
                        act = swap.AUTO_SPARSE   # the selector, with the compaction itself as its probe
            ticket = self.engine.pre(t, act)
            if remember:
                self._memo[tid] = [t.numel(), self.engine.info(ticket).policy, 0]
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

    def dropped(self, tensor_id: int) -> bool:
        return tensor_id in self._dropped

    def com_and_tran(self, tensor_id: int) -> int:
        if tensor_id in self._dropped:
            return 1
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
