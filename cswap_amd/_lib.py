"""Loads ``libcswap_hip.so`` and declares its C ABI for ctypes.

There is no fallback: if the library is missing or fails to load, importing the
functions raises, so nothing can silently run on a CPU path.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcswap_hip.so")


class CswapError(RuntimeError):
    def __init__(self, code: int, what: str):
        self.code = code
        super().__init__(f"{what}: {lib().cswap_strerror(code).decode()} (code {code}, "
                         f"hipError {lib().cswap_last_hip_error()})")


_lib = None

vp, sz, pd, u, i32 = C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_uint, C.c_int

_SIGNATURES = {
    "cswap_strerror": (C.c_char_p, [i32]),
    "cswap_last_hip_error": (i32, []),
    "cswap_abi_version": (i32, []),
    "cswap_zfp_stream_bytes": (sz, [sz, sz, sz, u]),
    "cswap_zfp_stream_capacity": (sz, [sz, sz, sz, u]),
    "cswap_zfp_compress_f32": (i32, [vp, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zfp_decompress_f32": (i32, [vp, sz, sz, sz, pd, pd, pd, u, vp, vp]),
    "cswap_zvc_chunk_elems": (i32, [i32, i32]),
    "cswap_zvc_chunk_words": (i32, [i32, i32]),
    "cswap_zvc_active_chunks": (i32, [i32, i32]),
    "cswap_zvc_mask_bytes": (sz, [i32, i32]),
    "cswap_zvc_count": (i32, [vp, i32, i32, vp, vp]),
    "cswap_zvc_scan": (i32, [vp, i32, vp, vp]),
    "cswap_zvc_compact": (i32, [vp, i32, i32, vp, vp, vp, vp]),
    "cswap_zvc_expand": (i32, [vp, vp, vp, i32, i32, vp, vp]),
    "cswap_zvc_compress": (i32, [vp, i32, i32, vp, vp, vp, vp, vp]),
    "cswap_probe_nnz": (i32, [vp, sz, vp, vp]),
}


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m cswap_amd.build` "
                "(there is no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            f = getattr(L, name)  # AttributeError if the symbol is not exported
            f.restype = res
            f.argtypes = args
        _lib = L
    return _lib


def declared_symbols():
    return sorted(_SIGNATURES)


def check(code: int, what: str) -> None:
    if code != 0:
        raise CswapError(code, what)
