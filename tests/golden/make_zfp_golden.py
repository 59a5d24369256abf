#!/usr/bin/env python3
"""Regenerates the ZFP golden fixtures in this directory.

The generator is the stock zfp 0.5.5 command-line codec that ships with the
build image (``/opt/conda/bin/zfp``, serial execution policy).  It is the same
codec version the reference snapshots (CSWAP+/zfp/version.h:9-15) and is not
part of the reference tree.  It is only needed to *re*generate; the tests read
the committed ``zfp_golden.npz`` / ``zfp_digests.json``.

    python tests/golden/make_zfp_golden.py

Fixture contents
  zfp_golden.npz   small 3-D fields: ``<name>/in`` fp32 (nz,ny,nx), and per rate
                   ``<name>/r<rate>/stream`` (uint8) and ``<name>/r<rate>/dec``.
  zfp_golden_12d.npz  the same for 2-D (ny,nx) and 1-D (nx,) fields.
  zfp_golden_i32.npz  int32 fields of 1, 2 and 3 dimensions (``-t i32``); written
                   alone by ``make_zfp_golden.py --i32``.
  zfp_golden_64.npz   float64 (``-d``) and int64 (``-t i64``) fields of 1, 2 and 3
                   dimensions; written alone by ``make_zfp_golden.py --w64``.
  zfp_digests.json SHA-256 of input, stream and decoded output for the large
                   seeded configurations (inputs are re-created from the seed).
"""
import hashlib
import json
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ZFP = os.environ.get("ZFP_CLI", "/opt/conda/bin/zfp")

sys.path.insert(0, os.path.join(HERE, "..", ".."))
from cswap_amd.workloads import config1_field, config3_fields  # noqa: E402


def run_zfp(field: np.ndarray, rate: float):
    """field: (nz, ny, nx), (ny, nx) or (nx,) -- x is always the fastest axis."""
    dims = [str(n) for n in reversed(field.shape)]
    dt, flag = {"int32": ("<i4", ["-t", "i32"]), "float32": ("<f4", ["-f"]),
                "int64": ("<i8", ["-t", "i64"]), "float64": ("<f8", ["-d"])}[field.dtype.name]
    with tempfile.TemporaryDirectory() as d:
        fi, fz, fo = (os.path.join(d, n) for n in ("in.raw", "out.zfp", "out.raw"))
        field.astype(dt).tofile(fi)
        subprocess.check_call([ZFP, "-q", *flag, f"-{field.ndim}", *dims, "-r", repr(rate),
                               "-i", fi, "-z", fz, "-o", fo])
        stream = np.fromfile(fz, dtype=np.uint8)
        dec = np.fromfile(fo, dtype=dt).reshape(field.shape)
    return stream, dec


def int_fields():
    rng = np.random.default_rng(777)
    f = {}
    f["i3_rand_8x8x8"] = rng.integers(-2**20, 2**20, (8, 8, 8)).astype(np.int32)
    f["i3_partial_7x5x6"] = rng.integers(-1000, 1000, (7, 5, 6)).astype(np.int32)
    f["i3_wide_4x4x8"] = rng.integers(-2**30, 2**30, (4, 4, 8)).astype(np.int32)
    z = rng.integers(-500, 500, (8, 8, 8)).astype(np.int32)
    z[0:4, 0:4, 0:4] = 0
    z[4:8, 4:8, 4:8] = 12345
    f["i3_zero_const_blocks"] = z
    g = np.arange(12)
    zz, yy, xx = np.meshgrid(g, g, g, indexing="ij")
    f["i3_smooth_12"] = (1e6 * np.exp(-((xx - 5) ** 2 + (yy - 6) ** 2 + (zz - 4) ** 2) / 30)).astype(np.int32)
    f["i3_nx2_ny2_8x2x2"] = rng.integers(-2**15, 2**15, (8, 2, 2)).astype(np.int32)
    f["i3_single"] = np.array([[[-77]]], dtype=np.int32)
    f["i2_rand_8x12"] = rng.integers(-2**24, 2**24, (8, 12)).astype(np.int32)
    f["i2_partial_7x9"] = rng.integers(-99, 99, (7, 9)).astype(np.int32)
    f["i2_smooth_20x20"] = (1e5 * np.exp(-((g[None, :8] - 3) ** 2 + (g[:8, None] - 4) ** 2) / 9)).astype(np.int32)
    f["i1_rand_64"] = rng.integers(-2**28, 2**28, 64).astype(np.int32)
    f["i1_partial_13"] = rng.integers(-5, 5, 13).astype(np.int32)
    f["i1_ramp_100"] = (np.arange(100) * 1000 - 40000).astype(np.int32)
    return f


def main_i32():
    out = {}
    for name, fld in int_fields().items():
        out[f"{name}/in"] = fld
        rates = RATES_SMALL if fld.ndim == 3 else RATES_2D if fld.ndim == 2 else RATES_1D
        for r in rates:
            stream, dec = run_zfp(fld, r)
            out[f"{name}/r{r}/stream"] = stream
            out[f"{name}/r{r}/dec"] = dec
    np.savez_compressed(os.path.join(HERE, "zfp_golden_i32.npz"), **out)
    print("wrote", len(out), "int32 arrays")


def wide_fields():
    """float64 and int64 fields of 1, 2 and 3 dimensions."""
    rng = np.random.default_rng(4242)
    f = {}
    f["d3_rand_8x8x8"] = rng.standard_normal((8, 8, 8))
    f["d3_partial_7x5x6"] = rng.standard_normal((7, 5, 6)) * 1e3
    z = rng.standard_normal((8, 8, 8))
    z[0:4, 0:4, 0:4] = 0.0
    z[4:8, 4:8, 4:8] = -7.5
    z[0:4, 4:8, 0:4] = -0.0
    f["d3_zero_const_blocks"] = z
    g = np.arange(12, dtype=np.float64)
    zz, yy, xx = np.meshgrid(g, g, g, indexing="ij")
    f["d3_smooth_12"] = np.exp(-((xx - 5) ** 2 + (yy - 6) ** 2 + (zz - 4) ** 2) / 30)
    w = rng.standard_normal((4, 8, 8)) * 2.0 ** rng.integers(-300, 300, size=(4, 8, 8))
    f["d3_wide_range"] = w
    f["d3_big_small"] = rng.standard_normal((4, 4, 8)) * np.array([1e250, 1e-250] * 4)
    f["d3_nx2_ny2_8x2x2"] = rng.standard_normal((8, 2, 2))
    f["d3_single"] = np.array([[[3.25]]])
    f["d2_rand_8x12"] = rng.standard_normal((8, 12))
    f["d2_partial_7x9"] = rng.standard_normal((7, 9)) * 1e-5
    f["d2_smooth_20x20"] = np.exp(-((g[None, :] - 5) ** 2 + (g[:, None] - 6) ** 2) / 40)
    f["d1_rand_64"] = rng.standard_normal(64)
    o = rng.standard_normal(41)
    o[8:16] = 0.0
    f["d1_partial_zero_41"] = o
    f["d1_smooth_100"] = np.sin(np.arange(100) / 9.0)
    f["l3_rand_8x8x8"] = rng.integers(-2**40, 2**40, (8, 8, 8))
    f["l3_partial_7x5x6"] = rng.integers(-1000, 1000, (7, 5, 6))
    f["l3_wide_4x4x8"] = rng.integers(-2**61, 2**61, (4, 4, 8))
    zi = rng.integers(-500, 500, (8, 8, 8))
    zi[0:4, 0:4, 0:4] = 0
    zi[4:8, 4:8, 4:8] = 123456789012
    f["l3_zero_const_blocks"] = zi
    f["l3_smooth_12"] = (1e15 * np.exp(-((xx - 5) ** 2 + (yy - 6) ** 2 + (zz - 4) ** 2) / 30)).astype(np.int64)
    f["l2_rand_8x12"] = rng.integers(-2**50, 2**50, (8, 12))
    f["l2_partial_7x9"] = rng.integers(-99, 99, (7, 9))
    f["l1_rand_64"] = rng.integers(-2**60, 2**60, 64)
    f["l1_partial_13"] = rng.integers(-5, 5, 13)
    return {k: np.ascontiguousarray(v.astype(np.int64 if k[0] == "l" else np.float64)) for k, v in f.items()}


RATES_64 = {3: [1, 2.5, 4, 8, 9.75, 16, 32, 48, 64], 2: [2, 4, 8, 12.5, 16, 32, 64], 1: [4, 8, 12, 16, 24, 32, 64]}


def main_w64():
    out = {}
    for name, fld in wide_fields().items():
        out[f"{name}/in"] = fld
        for r in RATES_64[fld.ndim]:
            stream, dec = run_zfp(fld, r)
            out[f"{name}/r{r}/stream"] = stream
            out[f"{name}/r{r}/dec"] = dec
    np.savez_compressed(os.path.join(HERE, "zfp_golden_64.npz"), **out)
    print("wrote", len(out), "64-bit arrays")


def small_fields():
    rng = np.random.default_rng(1234)
    f = {}
    f["rand_8x8x8"] = rng.standard_normal((8, 8, 8)).astype(np.float32)
    f["one_block"] = rng.standard_normal((4, 4, 4)).astype(np.float32) * 100
    f["partial_7x5x6"] = rng.standard_normal((7, 5, 6)).astype(np.float32)
    f["rows_8x4x12"] = np.maximum(rng.standard_normal((8, 4, 12)), 0).astype(np.float32)
    f["prelu_16x8x8"] = rng.standard_normal((16, 8, 8)).astype(np.float32)
    f["prelu_16x8x8"] = np.where(f["prelu_16x8x8"] > 0, f["prelu_16x8x8"],
                                 0.25 * f["prelu_16x8x8"]).astype(np.float32)
    f["nx2_ny2_8x2x2"] = rng.standard_normal((8, 2, 2)).astype(np.float32)
    f["odd_4x3x9"] = rng.standard_normal((4, 3, 9)).astype(np.float32)
    f["single_1x1x1"] = np.array([[[3.25]]], dtype=np.float32)
    f["line_5x1x3"] = rng.standard_normal((5, 1, 3)).astype(np.float32)
    z = rng.standard_normal((8, 8, 8)).astype(np.float32)
    z[0:4, 0:4, 0:4] = 0.0            # an all-zero block
    z[4:8, 4:8, 4:8] = 7.5            # a constant block
    z[0:4, 4:8, 0:4] = -0.0           # negative zeros only
    f["zero_const_blocks"] = z
    g = np.arange(12, dtype=np.float32)
    zz, yy, xx = np.meshgrid(g, g, g, indexing="ij")
    f["smooth_12"] = np.exp(-((xx - 5) ** 2 + (yy - 6) ** 2 + (zz - 4) ** 2) / 30).astype(np.float32)
    w = rng.standard_normal((4, 8, 8)).astype(np.float32)
    w *= np.float32(2.0) ** rng.integers(-40, 40, size=w.shape).astype(np.float32)
    f["wide_range"] = w.astype(np.float32)
    f["big_small"] = (rng.standard_normal((4, 4, 8)) * np.array([1e30, 1e-30] * 4)).astype(np.float32)
    s = np.zeros((4, 4, 4), dtype=np.float32)
    s[1, 2, 3] = -1.0
    f["single_spike"] = s
    f["softmax_like"] = (rng.random((4, 8, 16)) ** 8 / 16).astype(np.float32)
    return f


def low_dim_fields():
    rng = np.random.default_rng(4321)
    f = {}
    f["2d_rand_8x12"] = rng.standard_normal((8, 12)).astype(np.float32)
    f["2d_partial_7x9"] = rng.standard_normal((7, 9)).astype(np.float32) * 50
    f["2d_relu_16x16"] = np.maximum(rng.standard_normal((16, 16)), 0).astype(np.float32)
    f["2d_row_1x5"] = rng.standard_normal((1, 5)).astype(np.float32)
    z = rng.standard_normal((8, 8)).astype(np.float32)
    z[0:4, 0:4] = 0.0
    z[4:8, 4:8] = -2.25
    f["2d_zero_const"] = z
    g = np.arange(20, dtype=np.float32)
    f["2d_smooth_20x20"] = np.exp(-((g[None, :] - 9) ** 2 + (g[:, None] - 11) ** 2) / 40).astype(np.float32)
    f["1d_rand_64"] = rng.standard_normal(64).astype(np.float32)
    f["1d_partial_13"] = (rng.standard_normal(13) * 1e-3).astype(np.float32)
    f["1d_single"] = np.array([-7.5], dtype=np.float32)
    o = rng.standard_normal(40).astype(np.float32)
    o[8:16] = 0.0
    f["1d_with_zero_blocks"] = o
    f["1d_smooth_100"] = np.sin(np.arange(100, dtype=np.float32) / 9).astype(np.float32)
    return f


RATES_2D = [2, 4, 8, 12.5, 16, 32]      # maxbits = 16 * rate
RATES_1D = [4, 8, 12, 16, 24, 32]       # maxbits = 4 * rate
RATES_SMALL = [1, 2.5, 4, 4.5, 8, 9.75, 16, 20, 32]
RATES_BIG = [4, 8, 16]


def sha(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    out = {}
    for name, fld in small_fields().items():
        out[f"{name}/in"] = fld
        for r in RATES_SMALL:
            stream, dec = run_zfp(fld, r)
            out[f"{name}/r{r}/stream"] = stream
            out[f"{name}/r{r}/dec"] = dec
    np.savez_compressed(os.path.join(HERE, "zfp_golden.npz"), **out)

    low = {}
    for name, fld in low_dim_fields().items():
        low[f"{name}/in"] = fld
        for r in (RATES_2D if fld.ndim == 2 else RATES_1D):
            stream, dec = run_zfp(fld, r)
            low[f"{name}/r{r}/stream"] = stream
            low[f"{name}/r{r}/dec"] = dec
    np.savez_compressed(os.path.join(HERE, "zfp_golden_12d.npz"), **low)

    dig = {}
    big = {"config1_prelu_4096x32x32": config1_field()}
    for nm, fld in config3_fields(batch=16).items():
        big[f"config3_b16_{nm}"] = fld
    for name, fld in big.items():
        e = {"shape": list(fld.shape), "input_sha256": sha(fld), "rates": {}}
        for r in RATES_BIG:
            stream, dec = run_zfp(fld, r)
            e["rates"][str(r)] = {
                "stream_bytes": int(stream.size),
                "stream_sha256": sha(stream),
                "decoded_sha256": sha(dec),
                "max_abs_err": float(np.max(np.abs(dec.astype(np.float64) - fld))),
            }
        dig[name] = e
    with open(os.path.join(HERE, "zfp_digests.json"), "w") as fh:
        json.dump(dig, fh, indent=1, sort_keys=True)
    print("wrote", len(out), "arrays and", len(dig), "digest entries")


if __name__ == "__main__":
    if "--i32" in sys.argv:
        main_i32()
    elif "--w64" in sys.argv:
        main_w64()
    else:
        main()
        main_i32()
        main_w64()
