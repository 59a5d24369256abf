"""The C-ABI library must load and export every symbol include/cswap_hip.h
declares (no compute calls: this runs without a GPU)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_in_header():
    names = set()
    for fn in os.listdir(os.path.join(ROOT, "include")):
        if not fn.endswith(".h"):
            continue
        text = open(os.path.join(ROOT, "include", fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        for m in re.finditer(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text):
            name = m.group(1)
            if name.startswith("cswap_") or name in REFERENCE_NAMES:
                names.add(name)
    return names


REFERENCE_NAMES = {"PreGPUcompression", "PreAcc", "GPUcompression", "GPUdecompression", "cuda_compress",
                   "cuda_decompress", "compress", "decompress", "setRatio"}


def test_library_exports_every_declared_symbol():
    from cswap_amd import _lib

    L = _lib.lib()
    names = declared_in_header()
    assert len(names) >= 15
    for n in sorted(names):
        assert hasattr(L, n), f"{n} declared in include/ but not exported"
    for n in _lib.declared_symbols():
        assert n in names, f"{n} bound by the loader but not declared in include/"


def test_host_only_entry_points():
    from cswap_amd import _lib

    L = _lib.lib()
    assert L.cswap_abi_version() >= 1
    assert L.cswap_zfp_stream_bytes(32, 32, 4096, 512) == 4194304
    assert L.cswap_zfp_stream_capacity(2, 2, 5, 288) == ((2 * 288 + 63) // 64) * 8
    assert L.cswap_zfp_stream_bytes(2, 2, 5, 288) == (2 * 288 // 64) * 8
    assert L.cswap_zvc_mask_bytes(128 * 256 * 16 * 16, 16384) == 128 * 256 * 16 * 16 // 8
    assert (L.cswap_zvc_chunk_elems(1_000_003, 16384), L.cswap_zvc_chunk_words(1_000_003, 16384),
            L.cswap_zvc_active_chunks(1_000_003, 16384)) == (62, 2, 16130)
    assert L.cswap_strerror(-1) == b"invalid argument"


def test_argument_errors_do_not_launch():
    from cswap_amd import _lib

    L = _lib.lib()
    assert L.cswap_zfp_compress_f32(None, 4, 4, 4, 0, 0, 0, 512, None, None) == -1
    assert L.cswap_zfp_decompress_f32(None, 4, 4, 4, 0, 0, 0, 512, None, None) == -1
    assert L.cswap_zvc_count(None, 10, 16384, None, None) == -1
    assert L.cswap_probe_nnz(None, 0, None, None) == -1


def test_pipeline_kernel_grid_fits_its_scanner_on_any_part():
    """The ZVC pipeline kernel runs one data workgroup per compute unit but one, never more than
    there are tiles, and never more than the 256 tiles its one scanner wavefront serves per step:
    on a part with more compute units than that, the tiles beyond would wait for an offset that
    never comes.  The grid is computed on the host, so parts this build never runs on can be
    asked about."""
    from cswap_amd import _lib

    f = _lib.lib().cswap_test_zvc_stream_groups
    assert f(10000, 256) == 255          # MI355X
    assert f(10000, 304) == 256          # more compute units than the scanner serves per step
    assert f(10000, 1024) == 256
    assert f(100, 256) == 100            # fewer tiles than compute units
    assert f(5, 304) == 5
    assert f(10000, 2) == 1 and f(10000, 1) == 0
