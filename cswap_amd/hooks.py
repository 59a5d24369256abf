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
from ._lib import CswapError

E_NOMEM = -4   # CSWAP_E_NOMEM
KEEP = 0       # the reference's policy code for "stays on the device" (only with ``only``)


class _Handle:
    __slots__ = ("ticket", "shape", "keep", "key", "refs", "out", "raw")

    def __init__(self, ticket, shape, keep, key, raw):
        self.ticket, self.shape, self.keep, self.key = ticket, shape, keep, key
        self.raw = raw       # swapped out as it is: the outbound copy reads the tensor itself
        self.refs = 1        # how many autograd nodes saved this tensor
        self.out = None      # the swapped-in tensor while further nodes still have to ask for it


class _Ref:
    """What autograd holds for one saved tensor: the swapped tensor and the shape
    this node saw it in (a matmul saves a [b, h, s, s] tensor as [b*h, s, s])."""
    __slots__ = ("handle", "shape")

    def __init__(self, handle, shape):
        self.handle, self.shape = handle, shape


class swap_saved_tensors(torch.autograd.graph.saved_tensors_hooks):
    """Swap eligible saved activations (contiguous fp32 device tensors of at
    least ``min_bytes``) through ``engine``; everything else is saved as usual.

    The outbound copy of a tensor overlaps with whatever the compute stream does
    next.  The last ``depth`` tensors packed keep their device copy; packing one
    more lets the oldest go.  A tensor that went out raw is read by its copy, so
    that first waits for the copy (the reference waits one layer later,
    CSWAP+/vgg16-cifar10.cpp:221-228, i.e. depth 1); a compressed tensor's copy
    reads the engine's staging block, so its device tensor simply goes, stream
    ordered behind the compression, and the host waits for nothing: the forward
    pass runs ahead of the link as far as the staging pool has room (the engine
    takes blocks back as their copies finish and makes a request wait only when
    the pool is full).

    A tensor that several nodes save (the output of a ReLU is saved by the ReLU
    and by the convolution or pooling that consumes it; attention probabilities by
    the softmax and by the matmul, there reshaped) is swapped once: while its
    device copy is still held, packing the same contiguous bytes (address, element
    count, version) again refers to the same swap, and backward hands the one
    swapped-in tensor, viewed in each node's shape, to every node that asks for it.

    The last ``depth`` tensors of the forward pass are still on the device when it
    ends and are the first that backward asks for: they are handed back as they
    are, without a transfer.  The compressed tensors before them whose outbound
    copies are still queued have their payloads in the staging pool, and the
    engine decompresses those from there, again without the link.

    Backward asks for the tensors in roughly the reverse of the order they were
    packed in, so each unpack also starts the inbound copy of the ``prefetch``
    tensors packed just before the one it returns (one context serves one forward
    and one backward pass: a swapped tensor is handed back once per node that saved
    it and its host copy is released right after): their transfer then runs on
    the copy stream under the backward kernels of the current layer.  (VGG-16 at
    batch 128 on one MI355X: looking two tensors ahead keeps the link busy through
    layers whose backward is short; deeper look-ahead gains nothing more.)

    ``memo``: a dict the caller keeps from one training iteration to the next.  With
    ``policy=AUTO`` the selector probes every tensor (a counting pass and a host
    round trip, CSWAP+/Execution.h:92 has the same one); the k-th swapped tensor of
    an iteration is the same activation every time, so its decision is remembered
    under (k, element count).  A remembered "ZFP" or "raw" is passed to the engine
    as an explicit policy and costs no probe; a remembered "ZVC" goes in as
    ``AUTO_SPARSE``: the one-kernel compaction runs first and its count is the
    selector's probe, so the choice is confirmed every time.  After ``recheck`` uses
    a ZFP or raw entry is probed again, so a layer whose sparsity drifts is noticed.

    ``only``: when set to a tensor, nothing but that tensor (the same contiguous
    bytes) is swapped while the hooks are active.  Other eligible tensors saved in
    the meantime (a ReLU saves its output, which is the next layer's input) are
    held as they are and remembered: ``swap_named`` swaps such a tensor out later,
    for every node that saved it, once the caller says how.  ``policy`` and
    ``only`` may be changed between two activations of the same context, which is
    how the per-layer calls of ``cswap_amd.torch_names`` drive one context per
    iteration."""

    def __init__(self, engine: "swap.SwapEngine", policy: int = swap.AUTO, min_bytes: int = 1 << 20,
                 prefetch: int = 2, depth: int = 2, memo: dict | None = None, recheck: int = 16,
                 only: torch.Tensor | None = None):
        self.engine = engine
        self.policy = policy
        self.only = only
        self.min_bytes = min_bytes
        self.prefetch = prefetch
        self.depth = max(1, depth)
        self.memo = memo
        self.recheck = max(1, recheck)
        self._position = 0         # swaps attempted so far in this context
        self._order = []           # handles in pack order
        self._fetched = set()      # tickets already swapped in or being prefetched
        self._released = set()
        self._pending = []         # handles whose outbound copy may still be in flight, oldest first
        self._live = {}            # key -> handle, only while the handle holds its device tensor
        self._to_release = []      # handles whose swap-in has been launched
        self.stats = {"swapped": 0, "bytes_in": 0, "bytes_out": 0, "kept": 0, "shared": 0}
        super().__init__(self._pack, self._unpack)

    # -- forward side
    def _settle(self, keep_in_flight: int = 0):
        """Wait for the oldest outbound copies until at most ``keep_in_flight`` are left."""
        while len(self._pending) > keep_in_flight:
            h = self._pending.pop(0)
            if h.raw:
                self.engine.post(h.ticket)   # Execution::post: copy done, device memory may go
            h.keep = None
            self._live.pop(h.key, None)

    @staticmethod
    def _key(t: torch.Tensor):
        return (t.data_ptr(), t.numel(), t._version)

    def _eligible(self, t: torch.Tensor) -> bool:
        return (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.dim() >= 1
                and t.numel() * 4 >= self.min_bytes and not isinstance(t, torch.nn.Parameter)
                and not t.is_leaf)

    def _pack(self, t: torch.Tensor):
        if not self._eligible(t):
            self.stats["kept"] += 1
            return t
        key = self._key(t)
        h = self._live.get(key)
        if h is not None:                # same tensor saved by another node: one swap serves both
            h.refs += 1
            self.stats["shared"] += 1
            return _Ref(h, tuple(t.shape))
        if self.only is not None and (self.policy == KEEP or not (t.data_ptr() == self.only.data_ptr()
                                                                  and t.numel() == self.only.numel())):
            # not the tensor this activation is for (or that one is to stay): held as it is, until
            # swap_named says otherwise
            h = _Handle(None, tuple(t.shape), t, key, False)
            self._live[key] = h
            self.stats["held"] = self.stats.get("held", 0) + 1
            return _Ref(h, tuple(t.shape))
        h = _Handle(None, tuple(t.shape), t, key, False)
        return _Ref(h, tuple(t.shape)) if self._swap_out(t, h) else t

    def swap_named(self, t: torch.Tensor) -> bool:
        """Swaps out, with the current ``policy``, a tensor that was saved and held while the hooks
        were active for another one.  False if ``t`` is not such a tensor (nobody has saved it yet:
        the pack hook will see it) or could not go out."""
        h = self._live.get(self._key(t)) if self._eligible(t) else None
        if h is None or h.ticket is not None or self.policy == KEEP:
            return False
        return self._swap_out(t, h)

    def _swap_out(self, t: torch.Tensor, h) -> bool:
        """Starts the swap-out of t for handle h (which holds t); False if it has to stay on the device."""
        self._settle(self.depth - 1)
        self._drain()
        policy, slot = self.policy, (self._position, t.numel())
        self._position += 1
        if self.memo is not None and self.policy == swap.AUTO:
            known = self.memo.get(slot)
            if known is not None and known[0] in (swap.ZFP, swap.NONE) and known[1] < self.recheck:
                policy = known[0]
                self.memo[slot] = (known[0], known[1] + 1)
                self.stats["memo_hits"] = self.stats.get("memo_hits", 0) + 1
            elif known is not None and known[0] == swap.SPARSE:
                # still the selector's call, but with the compaction itself as its probe: the payload
                # is made by the time the count is known, and the count confirms the choice every time
                policy = swap.AUTO_SPARSE
                self.stats["memo_sparse"] = self.stats.get("memo_sparse", 0) + 1
        try:
            try:
                ticket = self.engine.pre(t.detach(), policy)
            except CswapError as err:
                if err.code != E_NOMEM or policy == self.policy:
                    raise
                policy = self.policy     # no staging room for the remembered codec: let the selector degrade it
                ticket = self.engine.pre(t.detach(), policy)
        except CswapError as err:
            if err.code != E_NOMEM:
                raise
            self.stats["kept_no_room"] = self.stats.get("kept_no_room", 0) + 1
            return False                 # pinned pool, staging pool or tickets exhausted: the tensor stays on the device
        info = self.engine.info(ticket)
        if self.memo is not None and policy in (swap.AUTO, swap.AUTO_SPARSE):
            self.memo[slot] = (info.policy, 0)
        self.stats["swapped"] += 1
        self.stats["bytes_in"] += info.bytes_in
        self.stats["bytes_out"] += info.bytes_out
        by = self.stats.setdefault("by_policy", {})
        name = {swap.NONE: "raw", swap.SPARSE: "zvc", swap.ZFP: "zfp"}.get(info.policy, str(info.policy))
        by[name] = by.get(name, 0) + 1
        h.ticket = ticket
        h.raw = info.policy == swap.NONE     # h.keep holds the device copy alive for now
        self._pending.append(h)
        self._live[h.key] = h
        self._order.append(h)
        return True

    # -- backward side
    def _drain(self):
        for h in self._to_release:
            self.engine.release(h.ticket)
            self._released.add(h.ticket)
        self._to_release.clear()

    def _unpack(self, ref):
        if not isinstance(ref, _Ref):
            return ref
        h = ref.handle
        if h.out is not None:            # another node already had it swapped in
            out = h.out
            h.refs -= 1
            if h.refs <= 0:
                h.out = None
            return out.view(ref.shape)
        if h.ticket is None:             # held, and never named for a swap: it is where it was
            out = h.keep.detach()
            h.refs -= 1
            if h.refs <= 0:
                h.keep = None
                self._live.pop(h.key, None)
            return out.view(ref.shape)
        self._drain()
        if h.keep is not None:           # still on the device: its outbound copy was one of the last in flight
            out = h.keep.detach()
            h.keep = None
            self._pending.remove(h)
            self._live.pop(h.key, None)
            self.stats["resident"] = self.stats.get("resident", 0) + 1
        else:
            out = torch.empty(h.shape, dtype=torch.float32, device="cuda")
            self.engine.swap_in(h.ticket, out)
        self._fetched.add(h.ticket)
        self._to_release.append(h)       # released once the next swap-in is issued (or at close)
        h.refs -= 1
        if h.refs > 0:
            h.out = out
        self._prefetch_before(h)
        return out.view(ref.shape)

    def _prefetch_before(self, h):
        """Start the inbound copies of the tensors packed just before ``h``."""
        if self.prefetch <= 0 or h not in self._order:
            return
        i = self._order.index(h)
        started = 0
        for g in reversed(self._order[:i]):
            if started >= self.prefetch:
                break
            if g.ticket in self._fetched or g.keep is not None:
                continue
            try:
                self.engine.prefetch(g.ticket)
            except CswapError as err:
                if err.code != E_NOMEM:
                    raise
                break                      # staging pool full: the swap-in will fetch it on demand
            self._fetched.add(g.ticket)
            self.stats["prefetched"] = self.stats.get("prefetched", 0) + 1
            started += 1

    def close(self):
        """Wait for and release everything still held; call after backward."""
        self._settle()
        torch.cuda.synchronize()
        self._drain()
        for h in self._order:              # saved but never asked for by backward
            h.out = None
            if h.ticket not in self._released:
                self.engine.release(h.ticket)
                self._released.add(h.ticket)
        self._order.clear()
        for h in self._live.values():      # held and never swapped
            h.keep = None
        self._live.clear()
