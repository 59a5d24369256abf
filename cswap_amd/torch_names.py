"""The five calls the reference's patched torch offers to Python model code, on stock
PyTorch-ROCm and with the reference's argument meaning:

    torch.cswapinit_()            once, after the model is on the device   (CIFAR10/cifar10.py:86)
    torch.cswapsetratio(ratio)    ZFP rate: 4 * ratio bits per 4x4x4 block (CIFAR10/cifar10.py:106)
    torch.cswapinit()             at the top of every forward pass         (CIFAR10/models/vgg.py:23)
    torch.cswappre(t, type)       before the layer that consumes t         (CIFAR10/models/vgg.py:43)
    torch.cswappost(t, out, type) after it                                 (CIFAR10/models/vgg.py:45)

``type`` is the reference's policy code (CSWAP+/Execution.h:70,86,107; the comment at
CIFAR10/models/vgg.py:41): 0 keeps ``t`` on the device, 2 swaps it out as it is, 3 as
zero-value compaction, 6 as fixed-rate ZFP; -1, which the reference does not have, asks
the selector.  In the reference these reach ``Execution::init_/init/pre/post`` and
``setRatio`` (CSWAP+/Execution.h:42-133,217-310) and the swap-in happens inside its
patched autograd engine; here ``cswappre`` switches saved-tensor hooks on for exactly
the tensor ``t`` and ``cswappost`` switches them off again, so that the copy autograd
keeps of ``t`` for backward is the one that goes out, and backward's request for it is
the swap-in (``cswap_amd.hooks``).  A tensor that the layer before had already saved (a
ReLU keeps its output) goes out for that node as well, so its device memory does go.
A tensor that no node saves (the input of a ReLU) is not swapped: stock autograd frees
it by itself as soon as the layer has run.  As in the reference, the outbound copy of a tensor
is waited for one layer later, and nothing is swapped while autograd is not recording.

``install()`` puts the five names on the ``torch`` module, so that a model file written
for the reference runs unchanged; they can also be called from here directly.
"""
from __future__ import annotations

import torch

from . import swap
from .hooks import swap_saved_tensors

KEEP, RAW, ZVC, ZFP, SELECT = 0, swap.NONE, swap.SPARSE, swap.ZFP, swap.AUTO
_CODES = {KEEP, RAW, ZVC, ZFP, SELECT}


class _State:
    engine = None       # cswapinit_
    owns_engine = False
    ctx = None          # one saved-tensor-hooks context per forward + backward pass (cswapinit)
    active = False      # between a cswappre that switched the hooks on and its cswappost
    memo = None         # the selector's decisions, kept from one iteration to the next
    min_bytes = 0
    prefetch = 2


_S = _State()


def _engine():
    if _S.engine is None:
        raise RuntimeError("cswapinit_() has not been called")
    return _S.engine


def cswapinit_(pinned_bytes: int = 4 << 30, device_bytes: int = 1 << 30, engine: "swap.SwapEngine | None" = None,
               calibrate: bool = True, min_bytes: int = 0, prefetch: int = 2) -> "swap.SwapEngine":
    """Execution::init_ (CSWAP+/Execution.h:46-64): the copy streams, the pinned pool the swapped
    tensors live in, the staging pool for compressed payloads, and the reference's starting rate
    (setRatio(128): 8 bits per value).  ``engine`` hands in one that already exists instead."""
    cswapclose()
    if engine is None:
        engine = swap.SwapEngine(pinned_bytes=pinned_bytes, device_bytes=device_bytes, maxbits=512)
        _S.owns_engine = True
        if calibrate:
            engine.calibrate()
    _S.engine = engine
    _S.memo = {}
    _S.min_bytes = min_bytes
    _S.prefetch = prefetch
    return engine


def cswapsetratio(ratio: int) -> None:
    """setRatio (CSWAP+/Execution.h:63): 4 * ratio bits per block of 64 values, 128 = a quarter
    of the fp32 size.  Tensors that are already out come back with the rate they went out with."""
    ratio = int(ratio)
    if not 4 <= ratio <= 1024:
        raise ValueError("ratio must be in 4..1024 (16..4096 bits per 4x4x4 block)")
    _engine().set_maxbits(4 * ratio)


def cswapinit() -> None:
    """Execution::init (CSWAP+/Execution.h:42-45), at the top of a forward pass: whatever the
    previous pass still holds is released and the tensor index starts again."""
    eng = _engine()
    _finish_pass()
    # depth 1: the copy of a tensor that went out raw is waited for when the next one is packed,
    # one layer later, as in the reference (CSWAP+/vgg16-cifar10.cpp:221-228)
    _S.ctx = swap_saved_tensors(eng, policy=SELECT, min_bytes=_S.min_bytes, prefetch=_S.prefetch, depth=1,
                                memo=_S.memo)


def cswappre(t: torch.Tensor, type: int = KEEP) -> None:  # noqa: A002 (the reference's argument name)
    """Execution::pre (CSWAP+/Execution.h:65-133) for the layer input ``t``."""
    type = int(type)
    if type not in _CODES:
        raise ValueError(f"unknown policy code {type}: 0 keep, 2 raw, 3 ZVC, 6 ZFP, -1 selector")
    if _S.active:
        raise RuntimeError("cswappre without the cswappost of the call before it")
    if _S.ctx is None:
        cswapinit()
    if not torch.is_grad_enabled():
        return                      # nothing is saved for backward: nothing to swap
    # The hooks are on for every layer, also one whose input stays (code 0) or has no grad_fn
    # (Execution::pre leaves such a tensor alone, Execution.h:69; so do the hooks): what the layer
    # saves besides its input -- a ReLU saves its output -- is the input of a later layer, and has
    # to be known to the context by the time that layer's cswappre names it.
    ctx = _S.ctx
    ctx.policy = type
    ctx.only = t
    ctx.swap_named(t)               # t was saved by the layer that made it: it goes out for that node too
    ctx.__enter__()
    _S.active = True


def cswappost(t: torch.Tensor, out: torch.Tensor | None = None, type: int = KEEP) -> None:  # noqa: A002
    """Execution::post (CSWAP+/Execution.h:217-310) after the layer has been called."""
    if not _S.active:
        return
    ctx = _S.ctx
    ctx.__exit__(None, None, None)
    ctx.only = None
    _S.active = False


def stats() -> dict:
    """What the current pass has swapped so far (see swap_saved_tensors.stats)."""
    return dict(_S.ctx.stats) if _S.ctx is not None else {}


def _finish_pass() -> None:
    if _S.active:
        cswappost(None)
    if _S.ctx is not None:
        _S.ctx.close()
        _S.ctx = None


def cswapclose() -> None:
    """Releases everything (no counterpart in the reference, whose process simply ends)."""
    if _S.engine is not None:
        _finish_pass()
        if _S.owns_engine:
            _S.engine.close()
    _S.engine, _S.owns_engine, _S.memo = None, False, None


_NAMES = {"cswapinit_": cswapinit_, "cswapinit": cswapinit, "cswapsetratio": cswapsetratio,
          "cswappre": cswappre, "cswappost": cswappost}


def install(module=torch) -> None:
    """``torch.cswappre`` and the other four, for model files written against the reference."""
    for name, fn in _NAMES.items():
        setattr(module, name, fn)


def uninstall(module=torch) -> None:
    for name, fn in _NAMES.items():
        if getattr(module, name, None) is fn:
            delattr(module, name)
