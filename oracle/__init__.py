"""ctypes front end of the CPU checker (``oracle/cswap_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; the shipped package never imports
it.  Every function below is a thin numpy wrapper around the C function of the
same name; the C file cites the reference lines each one restates.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
PROCESS = 512 * 32  # reference launch geometry, CSWAP+/Execution.h:50-52


def build(ref: bool = True) -> None:
    """Compile the checker (and, where the reference sources exist, the
    reference's own host-side C into ``oracle/_ref``)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "all"])
    if ref:
        subprocess.check_call(["make", "-s", "-C", _HERE, "ref"])


def _load(name: str) -> C.CDLL:
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build(ref=False)
    return C.CDLL(path)


def _sig(lib: C.CDLL) -> C.CDLL:
    vp, sz, pd, u, i = C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_uint, C.c_int
    lib.orc_threads.restype = i
    lib.orc_zfp_stream_bytes3.restype = sz
    lib.orc_zfp_stream_bytes3.argtypes = [sz, sz, sz, u]
    lib.orc_zfp_encode3_f32.restype = sz
    lib.orc_zfp_encode3_f32.argtypes = [vp, sz, sz, sz, pd, pd, pd, u, vp]
    lib.orc_zfp_decode3_f32.restype = None
    lib.orc_zfp_decode3_f32.argtypes = [vp, sz, sz, sz, pd, pd, pd, u, vp]
    lib.orc_zfp_stream_bytes2.restype = sz
    lib.orc_zfp_stream_bytes2.argtypes = [sz, sz, u]
    lib.orc_zfp_stream_bytes1.restype = sz
    lib.orc_zfp_stream_bytes1.argtypes = [sz, u]
    lib.orc_zfp_encode2_f32.restype = sz
    lib.orc_zfp_encode2_f32.argtypes = [vp, sz, sz, pd, pd, u, vp]
    lib.orc_zfp_decode2_f32.restype = None
    lib.orc_zfp_decode2_f32.argtypes = [vp, sz, sz, pd, pd, u, vp]
    lib.orc_zfp_encode1_f32.restype = sz
    lib.orc_zfp_encode1_f32.argtypes = [vp, sz, pd, u, vp]
    lib.orc_zfp_decode1_f32.restype = None
    lib.orc_zfp_decode1_f32.argtypes = [vp, sz, pd, u, vp]
    lib.orc_perm2.argtypes = [vp]
    lib.orc_zfp_encode_i32.restype = sz
    lib.orc_zfp_encode_i32.argtypes = [vp, i, sz, sz, sz, pd, pd, pd, u, vp]
    lib.orc_zfp_decode_i32.restype = None
    lib.orc_zfp_decode_i32.argtypes = [vp, i, sz, sz, sz, pd, pd, pd, u, vp]
    lib.orc_zfp_encode_64.restype = sz
    lib.orc_zfp_encode_64.argtypes = [vp, i, i, sz, sz, sz, pd, pd, pd, u, vp]
    lib.orc_zfp_decode_64.restype = None
    lib.orc_zfp_decode_64.argtypes = [vp, i, i, sz, sz, sz, pd, pd, pd, u, vp]
    lib.orc_zfp_encode_block_f32.restype = None
    lib.orc_zfp_encode_block_f32.argtypes = [vp, u, sz, vp]
    lib.orc_zfp_decode_block_f32.restype = None
    lib.orc_zfp_decode_block_f32.argtypes = [vp, u, sz, vp]
    lib.orc_fwd_lift.argtypes = [vp, pd]
    lib.orc_inv_lift.argtypes = [vp, pd]
    lib.orc_fwd_xform3.argtypes = [vp]
    lib.orc_inv_xform3.argtypes = [vp]
    lib.orc_int2uint.restype = C.c_uint32
    lib.orc_int2uint.argtypes = [C.c_int32]
    lib.orc_uint2int.restype = C.c_int32
    lib.orc_uint2int.argtypes = [C.c_uint32]
    lib.orc_perm3.argtypes = [vp]
    lib.orc_block_emax.restype = i
    lib.orc_block_emax.argtypes = [vp]
    lib.orc_fwd_cast.argtypes = [vp, vp, i]
    for f in ("orc_zvc_chunk_elems", "orc_zvc_chunk_words", "orc_zvc_active_chunks"):
        getattr(lib, f).restype = i
        getattr(lib, f).argtypes = [i, i]
    lib.orc_zvc_mask_bytes.restype = sz
    lib.orc_zvc_mask_bytes.argtypes = [i, i]
    lib.orc_zvc_count.argtypes = [i, i, vp, vp]
    lib.orc_zvc_preacc.argtypes = [vp, i, vp]
    lib.orc_zvc_compress.argtypes = [i, i, vp, vp, vp, vp]
    lib.orc_zvc_decompress.argtypes = [vp, vp, vp, i, i, vp]
    lib.orc_zvc_decompress_reference_writes.argtypes = [vp, vp, vp, i, i, vp]
    return lib


_libs: dict = {}


def lib(omp: bool = False) -> C.CDLL:
    name = "liboracle_omp.so" if omp else "liboracle.so"
    if name not in _libs:
        _libs[name] = _sig(_load(name))
    return _libs[name]


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


# --------------------------------------------------------------------------- ZFP

def zfp_stream_bytes(nx: int, ny: int, nz: int, maxbits: int) -> int:
    return lib().orc_zfp_stream_bytes3(nx, ny, nz, maxbits)


def zfp_stream_words_alloc(nx: int, ny: int, nz: int, maxbits: int) -> int:
    blocks = ((nx + 3) // 4) * ((ny + 3) // 4) * ((nz + 3) // 4)
    return (blocks * maxbits + 63) // 64


def zfp_encode3(field: np.ndarray, maxbits: int, omp: bool = False) -> np.ndarray:
    """field: C-contiguous fp32 array of shape (nz, ny, nx).  Returns the
    stream as uint64 words (length = ceil(blocks*maxbits/64))."""
    assert field.dtype == np.float32 and field.ndim == 3 and field.flags.c_contiguous
    nz, ny, nx = field.shape
    out = np.zeros(zfp_stream_words_alloc(nx, ny, nz, maxbits) + 1, dtype=np.uint64)
    lib(omp).orc_zfp_encode3_f32(_p(field), nx, ny, nz, 0, 0, 0, maxbits, _p(out))
    return out[:-1]


def zfp_decode3(stream: np.ndarray, shape, maxbits: int, omp: bool = False) -> np.ndarray:
    nz, ny, nx = shape
    s = np.zeros(zfp_stream_words_alloc(nx, ny, nz, maxbits) + 1, dtype=np.uint64)
    w = np.ascontiguousarray(stream).view(np.uint64)
    s[: w.size] = w
    out = np.zeros(shape, dtype=np.float32)
    lib(omp).orc_zfp_decode3_f32(_p(s), nx, ny, nz, 0, 0, 0, maxbits, _p(out))
    return out


def zfp_encode_nd(field: np.ndarray, maxbits: int) -> np.ndarray:
    """1-D (nx,), 2-D (ny,nx) or 3-D (nz,ny,nx) C-contiguous fp32 field -> stream words."""
    assert field.dtype == np.float32 and field.flags.c_contiguous
    if field.ndim == 3:
        return zfp_encode3(field, maxbits)
    shp = field.shape
    blocks = int(np.prod([(n + 3) // 4 for n in shp]))
    out = np.zeros((blocks * maxbits + 63) // 64 + 1, dtype=np.uint64)
    if field.ndim == 2:
        lib().orc_zfp_encode2_f32(_p(field), shp[1], shp[0], 0, 0, maxbits, _p(out))
    else:
        lib().orc_zfp_encode1_f32(_p(field), shp[0], 0, maxbits, _p(out))
    return out[:-1]


def zfp_decode_nd(stream: np.ndarray, shape, maxbits: int) -> np.ndarray:
    shape = tuple(shape)
    if len(shape) == 3:
        return zfp_decode3(stream, shape, maxbits)
    blocks = int(np.prod([(n + 3) // 4 for n in shape]))
    s = np.zeros((blocks * maxbits + 63) // 64 + 1, dtype=np.uint64)
    w = np.ascontiguousarray(stream).view(np.uint64)
    s[: w.size] = w
    out = np.zeros(shape, dtype=np.float32)
    if len(shape) == 2:
        lib().orc_zfp_decode2_f32(_p(s), shape[1], shape[0], 0, 0, maxbits, _p(out))
    else:
        lib().orc_zfp_decode1_f32(_p(s), shape[0], 0, maxbits, _p(out))
    return out


def _dims3(shape):
    shape = tuple(shape)
    nx = shape[-1]
    ny = shape[-2] if len(shape) >= 2 else 1
    nz = shape[-3] if len(shape) >= 3 else 1
    return len(shape), nx, ny, nz


def zfp_encode_i32(field: np.ndarray, maxbits: int) -> np.ndarray:
    """1-D, 2-D or 3-D C-contiguous int32 field (x fastest) -> stream words."""
    assert field.dtype == np.int32 and field.flags.c_contiguous and 1 <= field.ndim <= 3
    dims, nx, ny, nz = _dims3(field.shape)
    blocks = int(np.prod([(n + 3) // 4 for n in field.shape]))
    out = np.zeros((blocks * maxbits + 63) // 64 + 1, dtype=np.uint64)
    lib().orc_zfp_encode_i32(_p(field), dims, nx, ny, nz, 0, 0, 0, maxbits, _p(out))
    return out[:-1]


def zfp_decode_i32(stream: np.ndarray, shape, maxbits: int) -> np.ndarray:
    dims, nx, ny, nz = _dims3(shape)
    blocks = int(np.prod([(n + 3) // 4 for n in shape]))
    s = np.zeros((blocks * maxbits + 63) // 64 + 1, dtype=np.uint64)
    w = np.ascontiguousarray(stream).view(np.uint64)
    s[: w.size] = w
    out = np.zeros(tuple(shape), dtype=np.int32)
    lib().orc_zfp_decode_i32(_p(s), dims, nx, ny, nz, 0, 0, 0, maxbits, _p(out))
    return out


def zfp_encode_64(field: np.ndarray, maxbits: int) -> np.ndarray:
    """1-D, 2-D or 3-D C-contiguous float64 or int64 field (x fastest) -> stream words."""
    assert field.dtype in (np.float64, np.int64) and field.flags.c_contiguous and 1 <= field.ndim <= 3
    dims, nx, ny, nz = _dims3(field.shape)
    blocks = int(np.prod([(n + 3) // 4 for n in field.shape]))
    out = np.zeros((blocks * maxbits + 63) // 64 + 1, dtype=np.uint64)
    lib().orc_zfp_encode_64(_p(field), int(field.dtype == np.int64), dims, nx, ny, nz, 0, 0, 0, maxbits, _p(out))
    return out[:-1]


def zfp_decode_64(stream: np.ndarray, shape, maxbits: int, dtype) -> np.ndarray:
    dtype = np.dtype(dtype)
    assert dtype in (np.float64, np.int64)
    dims, nx, ny, nz = _dims3(shape)
    blocks = int(np.prod([(n + 3) // 4 for n in shape]))
    s = np.zeros((blocks * maxbits + 63) // 64 + 1, dtype=np.uint64)
    w = np.ascontiguousarray(stream).view(np.uint64)
    s[: w.size] = w
    out = np.zeros(tuple(shape), dtype=dtype)
    lib().orc_zfp_decode_64(_p(s), int(dtype == np.int64), dims, nx, ny, nz, 0, 0, 0, maxbits, _p(out))
    return out


def zfp_encode_block(block64: np.ndarray, maxbits: int) -> np.ndarray:
    b = np.ascontiguousarray(block64, dtype=np.float32).reshape(64)
    out = np.zeros((maxbits + 63) // 64 + 1, dtype=np.uint64)
    lib().orc_zfp_encode_block_f32(_p(b), maxbits, 0, _p(out))
    return out[:-1]


def zfp_decode_block(words: np.ndarray, maxbits: int) -> np.ndarray:
    s = np.zeros((maxbits + 63) // 64 + 1, dtype=np.uint64)
    s[: words.size] = words
    out = np.zeros(64, dtype=np.float32)
    lib().orc_zfp_decode_block_f32(_p(s), maxbits, 0, _p(out))
    return out


def fwd_lift(v) -> np.ndarray:
    a = np.array(v, dtype=np.int32).copy()
    lib().orc_fwd_lift(_p(a), 1)
    return a


def inv_lift(v) -> np.ndarray:
    a = np.array(v, dtype=np.int32).copy()
    lib().orc_inv_lift(_p(a), 1)
    return a


def fwd_xform3(b) -> np.ndarray:
    a = np.array(b, dtype=np.int32).reshape(64).copy()
    lib().orc_fwd_xform3(_p(a))
    return a


def inv_xform3(b) -> np.ndarray:
    a = np.array(b, dtype=np.int32).reshape(64).copy()
    lib().orc_inv_xform3(_p(a))
    return a


def perm3() -> np.ndarray:
    a = np.zeros(64, dtype=np.uint8)
    lib().orc_perm3(_p(a))
    return a


def block_emax(b) -> int:
    a = np.ascontiguousarray(b, dtype=np.float32).reshape(64)
    return lib().orc_block_emax(_p(a))


def fwd_cast(b, emax: int) -> np.ndarray:
    a = np.ascontiguousarray(b, dtype=np.float32).reshape(64)
    o = np.zeros(64, dtype=np.int32)
    lib().orc_fwd_cast(_p(o), _p(a), emax)
    return o


# --------------------------------------------------------------------------- ZVC

def zvc_geometry(n: int, process: int = PROCESS):
    L = lib()
    return (L.orc_zvc_chunk_elems(n, process), L.orc_zvc_chunk_words(n, process),
            L.orc_zvc_active_chunks(n, process))


def zvc_compress(x: np.ndarray, process: int = PROCESS, omp: bool = False):
    """Returns (values[nnz], mask[W*process] uint32, begin[process] int32, nnz).
    Mask words and begin entries the reference leaves unwritten are zero."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    n = x.size
    L = lib(omp)
    _, W, K = zvc_geometry(n, process)
    begin = np.zeros(process, dtype=np.int32)
    L.orc_zvc_count(n, process, _p(x), _p(begin))
    num = np.zeros(1, dtype=np.int32)
    L.orc_zvc_preacc(_p(begin), K, _p(num))
    nnz = int(num[0])
    values = np.zeros(max(nnz, 1), dtype=np.float32)
    mask = np.zeros(W * process, dtype=np.uint32)
    L.orc_zvc_compress(n, process, _p(x), _p(values), _p(begin), _p(mask))
    return values[:nnz], mask, begin, nnz


def zvc_count(x: np.ndarray, process: int = PROCESS) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    c = np.zeros(process, dtype=np.int32)
    lib().orc_zvc_count(x.size, process, _p(x), _p(c))
    return c


def zvc_decompress(values, mask, begin, n: int, process: int = PROCESS,
                   omp: bool = False, reference_writes: bool = False) -> np.ndarray:
    values = np.ascontiguousarray(values, dtype=np.float32)
    if values.size == 0:
        values = np.zeros(1, dtype=np.float32)
    mask = np.ascontiguousarray(mask, dtype=np.uint32)
    begin = np.ascontiguousarray(begin, dtype=np.int32)
    out = np.zeros(n, dtype=np.float32)
    L = lib(omp)
    f = L.orc_zvc_decompress_reference_writes if reference_writes else L.orc_zvc_decompress
    f(_p(values), _p(mask), _p(begin), n, process, _p(out))
    return out


# --------------------------------------------------------------------------- _ref

def ref_host_lib():
    """The reference's own host-side C (bit stream + stream sizing), built by
    ``make -C oracle ref`` from /root/reference where that exists; None otherwise."""
    path = os.path.join(_HERE, "_ref", "libzfp_host_ref.so")
    if not os.path.exists(path):
        return None
    return C.CDLL(path)
