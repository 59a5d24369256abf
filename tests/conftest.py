import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden.npz"))


@pytest.fixture(scope="session")
def golden_12d():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden_12d.npz"))


@pytest.fixture(scope="session")
def golden_i32():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden_i32.npz"))


@pytest.fixture(scope="session")
def golden_64():
    import numpy as np

    return np.load(os.path.join(ROOT, "tests", "golden", "zfp_golden_64.npz"))


@pytest.fixture(scope="session")
def digests():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "zfp_digests.json")) as fh:
        return json.load(fh)


def golden_cases(g):
    """Yield (name, rate, maxbits, field, stream_bytes, decoded) for every fixture."""
    import numpy as np

    names = sorted({k.split("/")[0] for k in g.files})
    for n in names:
        f = g[n + "/in"]
        for k in sorted(g.files):
            if k.startswith(n + "/r") and k.endswith("/stream"):
                rate = float(k.split("/")[1][1:])
                maxbits = int(np.floor(4 ** f.ndim * rate + 0.5))   # bits per block of 4^d values
                yield n, rate, maxbits, f, g[k], g[k[: -len("stream")] + "dec"]


def libzfp():
    """The stock zfp 0.5.5 library of the build image (the codec version the
    reference snapshots, CSWAP+/zfp/version.h:9-15; not part of the reference tree),
    if this machine has it."""
    import ctypes as C
    import ctypes.util
    import os

    for cand in ("/opt/conda/lib/libzfp.so.0.5.5", ctypes.util.find_library("zfp")):
        if cand and (os.path.exists(cand) or "/" not in cand):
            try:
                L = C.CDLL(cand)
            except OSError:
                continue
            L.stream_open.restype = C.c_void_p
            L.stream_open.argtypes = [C.c_void_p, C.c_size_t]
            L.stream_close.argtypes = [C.c_void_p]
            L.zfp_stream_open.restype = C.c_void_p
            L.zfp_stream_open.argtypes = [C.c_void_p]
            L.zfp_stream_close.argtypes = [C.c_void_p]
            L.zfp_stream_set_rate.restype = C.c_double
            L.zfp_stream_set_rate.argtypes = [C.c_void_p, C.c_double, C.c_int, C.c_uint, C.c_int]
            L.zfp_stream_rewind.argtypes = [C.c_void_p]
            L.zfp_field_3d.restype = C.c_void_p
            L.zfp_field_3d.argtypes = [C.c_void_p, C.c_int, C.c_uint, C.c_uint, C.c_uint]
            L.zfp_field_free.argtypes = [C.c_void_p]
            L.zfp_compress.restype = C.c_size_t
            L.zfp_compress.argtypes = [C.c_void_p, C.c_void_p]
            L.zfp_decompress.restype = C.c_size_t
            L.zfp_decompress.argtypes = [C.c_void_p, C.c_void_p]
            for fn in ("zfp_field_1d", "zfp_field_2d"):
                getattr(L, fn).restype = C.c_void_p
            L.zfp_field_1d.argtypes = [C.c_void_p, C.c_int, C.c_uint]
            L.zfp_field_2d.argtypes = [C.c_void_p, C.c_int, C.c_uint, C.c_uint]
            return L
    return None


def libzfp_round_trip(Z, f, rate):
    """Compress and decompress the numpy field f (1-3 dims, x fastest) with the zfp
    library at the given rate: (maxbits, stream bytes, decoded field)."""
    import ctypes as C

    import numpy as np

    ztype = {"float32": 3, "int32": 1, "float64": 4, "int64": 2}[f.dtype.name]
    dims = f.ndim
    nz, ny, nx = (1,) * (3 - dims) + f.shape

    def field(arr):
        if dims == 3:
            return Z.zfp_field_3d(arr.ctypes.data, ztype, nx, ny, nz)
        if dims == 2:
            return Z.zfp_field_2d(arr.ctypes.data, ztype, nx, ny)
        return Z.zfp_field_1d(arr.ctypes.data, ztype, nx)

    buf = np.zeros(f.nbytes + 4096, dtype=np.uint8)
    bs = Z.stream_open(buf.ctypes.data, buf.size)
    zs = Z.zfp_stream_open(bs)
    Z.zfp_stream_set_rate(zs, rate, ztype, dims, 0)
    maxbits = int((C.c_uint * 4).from_address(zs)[1])           # zfp_stream: minbits, maxbits, maxprec, minexp
    fi = field(f)
    Z.zfp_stream_rewind(zs)
    n = Z.zfp_compress(zs, fi)
    assert n > 0
    out = np.empty_like(f)
    fo = field(out)
    Z.zfp_stream_rewind(zs)
    Z.zfp_decompress(zs, fo)
    Z.zfp_field_free(fi)
    Z.zfp_field_free(fo)
    Z.zfp_stream_close(zs)
    Z.stream_close(bs)
    return maxbits, buf[:n].copy(), out


def mid_size_field(kind, shape, rate):
    import numpy as np

    npdt = {"f32": np.float32, "i32": np.int32, "f64": np.float64, "i64": np.int64}[kind]
    rng = np.random.default_rng(len(shape) * 1000 + int(rate))
    smooth = np.cumsum(rng.standard_normal(shape), axis=-1)
    if kind[0] == "i":
        return np.ascontiguousarray((smooth * (1 << (20 if kind == "i32" else 40))).astype(npdt))
    return np.ascontiguousarray(smooth.astype(npdt))


MID_SIZE_CASES = [((33, 47, 65), 8.0), ((64, 64, 64), 16.0), ((300, 257), 12.0), ((70001,), 10.0), ((9, 130, 130), 3.0)]
