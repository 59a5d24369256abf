"""Torch-facing glue over the C ABI (device memory and streams only).

Names follow the reference's call sites: ``compress`` / ``decompress`` /
``setRatio`` (CSWAP+/Execution.h:63,113), ``cuda_compress`` /
``cuda_decompress`` (CSWAP+/zfp/cuZFP.h:11-12) and the four ZVC launchers
(CSWAP+/zfp/compression.cuh:4-9).  Every function launches on torch's current
stream and returns without synchronising.
"""
from __future__ import annotations

import torch

from ._lib import check, lib
from .workloads import field_dims

PROCESS = 512 * 32  # CSWAP+/Execution.h:50-52


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need_f32_cuda(t: torch.Tensor) -> None:
    if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
        raise ValueError("expected a contiguous fp32 tensor in device memory")


# ------------------------------------------------------------------- ZFP
def zfp_stream_bytes(nx: int, ny: int, nz: int, maxbits: int) -> int:
    return lib().cswap_zfp_stream_bytes(nx, ny, nz, maxbits)


def zfp_stream_capacity(nx: int, ny: int, nz: int, maxbits: int) -> int:
    return lib().cswap_zfp_stream_capacity(nx, ny, nz, maxbits)


# zfp_type of a field by torch dtype (zfp_type_int32 = 1, int64 = 2, float = 3, double = 4)
_ZFP_KIND = {torch.float32: "f32", torch.int32: "i32", torch.float64: "f64", torch.int64: "i64"}


def _need_field(t: torch.Tensor) -> str:
    kind = _ZFP_KIND.get(t.dtype)
    if kind is None:
        raise TypeError(f"ZFP codes float32, float64, int32 and int64 fields, not {t.dtype}")
    if kind == "f32":
        _need_f32_cuda(t)
    elif not (t.is_cuda and t.is_contiguous()):
        raise TypeError(f"expected a contiguous {t.dtype} CUDA tensor")
    return kind


def cuda_compress(t: torch.Tensor, maxbits: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """Fixed-rate ZFP of ``t`` viewed as the field (nx=last dim, ny=second to
    last, nz=rest); the scalar type follows the tensor's dtype, as the reference
    dispatches on ``field->type`` (CSWAP+/zfp/cuZFP.cu:389-423).  Returns the
    stream as a uint8 device tensor."""
    kind = _need_field(t)
    nx, ny, nz = field_dims(t.shape)
    cap = zfp_stream_capacity(nx, ny, nz, maxbits)
    if out is None:
        out = torch.empty(cap, dtype=torch.uint8, device=t.device)
    elif out.numel() * out.element_size() < cap:
        raise ValueError("stream buffer too small")
    if kind == "f32":
        check(lib().cswap_zfp_compress_f32(t.data_ptr(), nx, ny, nz, 0, 0, 0, maxbits, out.data_ptr(), _stream()),
              "cswap_zfp_compress_f32")
    else:
        name = f"cswap_zfp_compress_{kind}_nd"
        check(getattr(lib(), name)(t.data_ptr(), 3, nx, ny, nz, 0, 0, 0, maxbits, out.data_ptr(), _stream()), name)
    return out


def cuda_decompress(stream: torch.Tensor, shape, maxbits: int, out: torch.Tensor | None = None,
                    dtype=torch.float32) -> torch.Tensor:
    nx, ny, nz = field_dims(shape)
    if out is None:
        out = torch.empty(tuple(shape), dtype=dtype, device=stream.device)
    kind = _need_field(out)
    if stream.numel() * stream.element_size() < zfp_stream_capacity(nx, ny, nz, maxbits):
        raise ValueError("stream buffer too small")
    if kind == "f32":
        check(lib().cswap_zfp_decompress_f32(stream.data_ptr(), nx, ny, nz, 0, 0, 0, maxbits, out.data_ptr(),
                                             _stream()), "cswap_zfp_decompress_f32")
    else:
        name = f"cswap_zfp_decompress_{kind}_nd"
        check(getattr(lib(), name)(stream.data_ptr(), 3, nx, ny, nz, 0, 0, 0, maxbits, out.data_ptr(), _stream()),
              name)
    return out


_rate_maxbits = 512  # 8 bits/value in 3-D


def setRatio(ratio: int) -> None:
    """``setRatio(128)`` in the reference selects 1/4 size, i.e. 8 bits/value
    (CSWAP+/Execution.h:63, CIFAR10/cifar10.py:103-106): maxbits = 4 * ratio."""
    global _rate_maxbits
    if ratio <= 0 or 4 * ratio > 4096:
        raise ValueError("ratio out of range")
    _rate_maxbits = 4 * ratio


def compress(t: torch.Tensor) -> torch.Tensor:
    return cuda_compress(t, _rate_maxbits)


def decompress(stream: torch.Tensor, shape) -> torch.Tensor:
    return cuda_decompress(stream, shape, _rate_maxbits)


# ------------------------------------------------------------------- ZVC
def zvc_geometry(n: int, process: int = PROCESS):
    L = lib()
    return (L.cswap_zvc_chunk_elems(n, process), L.cswap_zvc_chunk_words(n, process),
            L.cswap_zvc_active_chunks(n, process))


def PreGPUcompression(t: torch.Tensor, valueIndex: torch.Tensor, process: int = PROCESS) -> None:
    _need_f32_cuda(t)
    check(lib().cswap_zvc_count(t.data_ptr(), t.numel(), process, valueIndex.data_ptr(), _stream()),
          "cswap_zvc_count")


def PreAcc(valueIndex: torch.Tensor, kernel_size: int, num: torch.Tensor) -> None:
    check(lib().cswap_zvc_scan(valueIndex.data_ptr(), kernel_size, num.data_ptr(), _stream()), "cswap_zvc_scan")


def GPUcompression(t: torch.Tensor, compressedList: torch.Tensor, compressedValueIndex: torch.Tensor,
                   compressedBinIndex: torch.Tensor, process: int = PROCESS) -> None:
    _need_f32_cuda(t)
    check(lib().cswap_zvc_compact(t.data_ptr(), t.numel(), process, compressedValueIndex.data_ptr(),
                                  compressedList.data_ptr(), compressedBinIndex.data_ptr(), _stream()),
          "cswap_zvc_compact")


def GPUdecompression(values: torch.Tensor, dest: torch.Tensor, mask: torch.Tensor, beginIndex: torch.Tensor,
                     process: int = PROCESS) -> None:
    _need_f32_cuda(dest)
    check(lib().cswap_zvc_expand(values.data_ptr(), mask.data_ptr(), beginIndex.data_ptr(), dest.numel(),
                                 process, dest.data_ptr(), _stream()), "cswap_zvc_expand")


def zvc_compress(t: torch.Tensor, process: int = PROCESS, fused: bool = False):
    """count + scan + compact without a host round trip (``fused``: in a single
    pass over the tensor).  Returns
    (values[n] (first nnz valid), mask uint32[W*process], begin int32[process], nnz int32[1])."""
    _need_f32_cuda(t)
    n = t.numel()
    dev = t.device
    _, W, _ = zvc_geometry(n, process)
    values = torch.empty(n, dtype=torch.float32, device=dev)
    mask = torch.empty(W * process, dtype=torch.int32, device=dev)
    begin = torch.zeros(process, dtype=torch.int32, device=dev)
    nnz = torch.zeros(1, dtype=torch.int32, device=dev)
    if fused:
        ws = zvc_workspace(process, dev)
        check(lib().cswap_zvc_compress_fused(t.data_ptr(), n, process, ws.data_ptr(), begin.data_ptr(),
                                             nnz.data_ptr(), values.data_ptr(), mask.data_ptr(), _stream()),
              "cswap_zvc_compress_fused")
    else:
        check(lib().cswap_zvc_compress(t.data_ptr(), n, process, begin.data_ptr(), nnz.data_ptr(),
                                       values.data_ptr(), mask.data_ptr(), _stream()), "cswap_zvc_compress")
    return values, mask, begin, nnz


def zvc_workspace(process: int = PROCESS, device=None) -> torch.Tensor:
    """A workspace for the single-pass compression, allocated and prepared
    (cswap_zvc_workspace_clear) on the current stream."""
    ws = torch.empty(lib().cswap_zvc_workspace_bytes(process), dtype=torch.uint8,
                     device=device if device is not None else torch.device("cuda"))
    check(lib().cswap_zvc_workspace_clear(ws.data_ptr(), process, _stream()), "cswap_zvc_workspace_clear")
    return ws


def probe_nnz(t: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    _need_f32_cuda(t)
    if out is None:
        out = torch.empty(1, dtype=torch.int64, device=t.device)
    check(lib().cswap_probe_nnz(t.data_ptr(), t.numel(), out.data_ptr(), _stream()), "cswap_probe_nnz")
    return out
