"""Activation swapping for stock PyTorch-ROCm through saved-tensor hooks.

The reference swaps the inputs of selected layers out during forward and back
in during backward from inside a patched autograd engine (``com_and_tran``,
``storage_impl_`` fields on ``Node``; CSWAP+/Execution.h:260-262,278-282,297-299).
On an unpatched torch the same points are ``torch.autograd.graph.saved_tensors_hooks``:
``pack`` (a tensor is saved for backward) = ``Execution::pre`` and, one pack later,
``Execution::post``; ``unpack`` (backward needs it) = the swap-in + decompress.

    eng = SwapEngine(...)
    with swap_saved_tensors(eng, policy=AUTO, min_bytes=1 << 20):
        loss = model(x).sum()
    loss.backward()
"""
from __future__ import annotations

import torch

from . import swap


class _Handle:
    __slots__ = ("ticket", "shape", "keep")

    def __init__(self, ticket, shape, keep):
        self.ticket, self.shape, self.keep = ticket, shape, keep


class swap_saved_tensors(torch.autograd.graph.saved_tensors_hooks):
    """Swap eligible saved activations (contiguous fp32 device tensors of at
    least ``min_bytes``) through ``engine``; everything else is saved as usual.

    The outbound copy of tensor i overlaps with whatever the compute stream does
    until tensor i+1 is packed, at which point its completion is awaited and the
    device copy is let go (the reference does the same one layer later,
    CSWAP+/vgg16-cifar10.cpp:221-228)."""

    def __init__(self, engine: "swap.SwapEngine", policy: int = swap.AUTO, min_bytes: int = 1 << 20):
        self.engine = engine
        self.policy = policy
        self.min_bytes = min_bytes
        self._pending = None       # handle whose outbound copy may still be in flight
        self._to_release = []      # tickets whose swap-in has been launched
        self.stats = {"swapped": 0, "bytes_in": 0, "bytes_out": 0, "kept": 0}
        super().__init__(self._pack, self._unpack)

    # -- forward side
    def _settle(self):
        h = self._pending
        if h is not None:
            self.engine.post(h.ticket)   # Execution::post: copy done, device memory may go
            h.keep = None
            self._pending = None

    def _pack(self, t: torch.Tensor):
        eligible = (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.dim() >= 1
                    and t.numel() * 4 >= self.min_bytes and not isinstance(t, torch.nn.Parameter)
                    and not t.is_leaf)
        if not eligible:
            self.stats["kept"] += 1
            return t
        self._settle()
        self._drain()
        ticket = self.engine.pre(t.detach(), self.policy)
        info = self.engine.info(ticket)
        self.stats["swapped"] += 1
        self.stats["bytes_in"] += info.bytes_in
        self.stats["bytes_out"] += info.bytes_out
        h = _Handle(ticket, tuple(t.shape), t)   # keep the device copy alive until the copy finished
        self._pending = h
        return h

    # -- backward side
    def _drain(self):
        for tk in self._to_release:
            self.engine.release(tk)
        self._to_release.clear()

    def _unpack(self, h):
        if not isinstance(h, _Handle):
            return h
        if self._pending is h:
            self._settle()
        self._drain()
        out = torch.empty(h.shape, dtype=torch.float32, device="cuda")
        self.engine.swap_in(h.ticket, out)
        self._to_release.append(h.ticket)   # released once the next swap-in is issued (or at close)
        return out

    def close(self):
        """Wait for and release everything still held; call after backward."""
        self._settle()
        torch.cuda.synchronize()
        self._drain()
