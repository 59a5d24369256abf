"""Host build of the PRODUCT's per-block codec (cswap_amd/csrc/zfp_block.h, the
code every GPU lane runs) against the zfp 0.5.5 golden vectors.  Not a GPU test:
it catches logic errors in the block codec before any kernel is launched."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT, golden_cases

SO = os.path.join(ROOT, "tests", "libhost_block_codec.so")
SRC = os.path.join(ROOT, "tests", "host_block_codec.cpp")
HDR = os.path.join(ROOT, "cswap_amd", "csrc", "zfp_block.h")


@pytest.fixture(scope="module")
def host():
    if (not os.path.exists(SO) or os.path.getmtime(SO) < max(os.path.getmtime(SRC), os.path.getmtime(HDR))):
        subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-pthread", "-o", SO, SRC])
    L = C.CDLL(SO)
    L.host_zfp_encode3.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    L.host_zfp_decode3.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    L.host_zfp_decode3_fenced.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p,
                                          C.c_uint32]
    L.host_zfp_decode3_fenced.restype = C.c_uint
    L.host_zfp_encode3_slots.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    L.host_zfp_encode3_slots.restype = C.c_uint
    L.host_transpose32.argtypes = [C.c_void_p]
    L.host_zfp_encode_low.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    L.host_zfp_decode_low.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    return L


def test_multiply_shift_division_matches_integer_division(host):
    """Block coordinates come from floor(b / d) computed as (b * mul) >> shift;
    exact for every b < 2^31, checked at the edges of each quotient step."""
    host.host_div31.restype = C.c_uint32
    host.host_div31.argtypes = [C.c_uint32, C.c_uint32]
    rng = np.random.default_rng(7)
    divisors = [1, 2, 3, 5, 7, 8, 9, 127, 128, 129, 1000, 65535, 65536, 65537, 2**24 + 1, 2**31 - 1, 2**31,
                2**32 - 1] + [int(v) for v in rng.integers(1, 2**31, 40)]
    for d in divisors:
        bs = {0, 1, d - 1, d, d + 1, 2**31 - 1, 2**31 - 2}
        top = (2**31 - 1) // d
        for q in {1, 2, top // 2, top - 1, top} | {int(v) for v in rng.integers(0, top + 1, 20)}:
            bs |= {q * d - 1, q * d, q * d + d - 1}
        bs |= {int(v) for v in rng.integers(0, 2**31, 50)}
        for b in bs:
            if 0 <= b < 2**31:
                assert host.host_div31(b, d) == b // d, (b, d)


def test_scale_factors_equal_ldexp(host):
    """The decoder's 2^(emax-30) for every 8-bit header exponent against ldexp
    (the reference's LDEXP, shared.h:184-205)."""
    import math

    host.host_decode_scale.restype = C.c_float
    host.host_decode_scale.argtypes = [C.c_uint32]
    for e8 in range(256):
        want = np.float32(math.ldexp(1.0, e8 - 127 - 30))
        assert np.float32(host.host_decode_scale(e8)).view(np.uint32) == want.view(np.uint32), e8


def test_transpose32_is_a_bit_matrix_transpose(host):
    a = np.random.default_rng(0).integers(0, 2**32, 32, dtype=np.uint32)
    b = a.copy()
    host.host_transpose32(b.ctypes.data)
    A = np.unpackbits(a.view(np.uint8).reshape(32, 4), axis=1, bitorder="little")
    B = np.unpackbits(b.view(np.uint8).reshape(32, 4), axis=1, bitorder="little")
    assert np.array_equal(B, A.T)


def test_block_codec_matches_golden_vectors(host, golden):
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden):
        nz, ny, nx = f.shape
        blocks = -(-nx // 4) * -(-ny // 4) * -(-nz // 4)
        words = (blocks * maxbits + 63) // 64
        s = np.zeros(words + 2, dtype=np.uint64)
        host.host_zfp_encode3(f.ctypes.data, nx, ny, nz, maxbits, s.ctypes.data)
        sb = s[:words].view(np.uint8)
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any()
        if maxbits % 64 == 0:  # the encoder variant the device uses for whole-word rates
            s2 = np.zeros(words, dtype=np.uint64)
            top = host.host_zfp_encode3_slots(f.ctypes.data, nx, ny, nz, maxbits, s2.ctypes.data)
            assert np.array_equal(s2.view(np.uint8)[:k], stream[:k]), (name, rate, "slots")
            assert top < maxbits // 32 + 4, (name, rate, "wrote past the 128 bits of slack")
        g = np.zeros((words + 2) * 8, dtype=np.uint8)
        g[:k] = stream[:k]
        o = np.zeros_like(f)
        host.host_zfp_decode3(g.ctypes.data, nx, ny, nz, maxbits, o.ctypes.data)
        assert np.array_equal(o.view(np.uint32), dec.view(np.uint32)), (name, rate)
        if maxbits % 64 == 0:  # the variant the device uses for whole-word rates
            o2 = np.zeros_like(f)
            top = host.host_zfp_decode3_fenced(g.ctypes.data, nx, ny, nz, maxbits, o2.ctypes.data, n)
            assert np.array_equal(o2.view(np.uint32), dec.view(np.uint32)), (name, rate, "fenced")
            assert top < maxbits // 32 + 4, (name, rate, top)
        n += 1
    assert n >= 100


def test_low_dimensional_block_codecs_match_golden_vectors(host, golden_12d):
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_12d):
        nx = f.shape[-1]
        ny = f.shape[0] if f.ndim == 2 else 0
        blocks = -(-nx // 4) * (-(-ny // 4) if ny else 1)
        words = (blocks * maxbits + 63) // 64
        s = np.zeros(words + 2, dtype=np.uint64)
        host.host_zfp_encode_low(f.ctypes.data, nx, ny, maxbits, s.ctypes.data)
        sb = s[:words].view(np.uint8)
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any()
        g = np.zeros((words + 2) * 8, dtype=np.uint8)
        g[:k] = stream[:k]
        o = np.zeros_like(f)
        host.host_zfp_decode_low(g.ctypes.data, nx, ny, maxbits, o.ctypes.data)
        assert np.array_equal(o.view(np.uint32), dec.view(np.uint32)), (name, rate)
        n += 1
    assert n >= 60


def test_int32_block_codec_matches_golden_vectors(host, golden_i32):
    """The int32 front ends of the header the GPU lanes run (no exponent header, no
    cast) against the zfp 0.5.5 vectors for 1-D, 2-D and 3-D fields."""
    A = [C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    host.host_zfp_encode_i32.argtypes = A
    host.host_zfp_decode_i32.argtypes = A
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_i32):
        shp = (1,) * (3 - f.ndim) + f.shape
        nz, ny, nx = shp
        blocks = int(np.prod([-(-d // 4) for d in f.shape]))
        words = (blocks * maxbits + 63) // 64
        s = np.zeros(words + 2, dtype=np.uint64)
        host.host_zfp_encode_i32(f.ctypes.data, f.ndim, nx, ny, nz, maxbits, s.ctypes.data)
        sb = s[:words].view(np.uint8)
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any()
        g = np.zeros((words + 2) * 8, dtype=np.uint8)
        g[:k] = stream[:k]
        o = np.zeros_like(f)
        host.host_zfp_decode_i32(g.ctypes.data, f.ndim, nx, ny, nz, maxbits, o.ctypes.data)
        assert np.array_equal(o, dec), (name, rate)
        n += 1
    assert n == 99


def test_64_bit_block_codec_matches_golden_vectors(host, golden_64):
    """The float64 / int64 front ends of the header the GPU lanes run (64 planes as
    two passes over 32-bit words, 12-bit header for doubles) against the zfp 0.5.5
    vectors for 1-D, 2-D and 3-D fields."""
    A = [C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    host.host_zfp_encode_w64.argtypes = A
    host.host_zfp_decode_w64.argtypes = A
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_64):
        is_int = int(f.dtype == np.int64)
        shp = (1,) * (3 - f.ndim) + f.shape
        nz, ny, nx = shp
        blocks = int(np.prod([-(-d // 4) for d in f.shape]))
        words = (blocks * maxbits + 63) // 64
        s = np.zeros(words + 2, dtype=np.uint64)
        host.host_zfp_encode_w64(f.ctypes.data, is_int, f.ndim, nx, ny, nz, maxbits, s.ctypes.data)
        sb = s[:words].view(np.uint8)
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any()
        g = np.zeros((words + 2) * 8, dtype=np.uint8)
        g[:k] = stream[:k]
        o = np.zeros_like(f)
        host.host_zfp_decode_w64(g.ctypes.data, is_int, f.ndim, nx, ny, nz, maxbits, o.ctypes.data)
        assert np.array_equal(o.view(np.uint64), dec.view(np.uint64)), (name, rate)
        n += 1
    assert n == 187


def test_64_bit_block_codec_agrees_with_checker_on_tiny_and_huge_doubles(host):
    """Blocks near the bottom of the double range: the scale 2^(62-emax) overflows
    below 2^-961 (the cast saturates) and fewer than 64 planes are coded below
    2^-1018; the reference leaves these undefined, the two implementations here
    agree on them.  Also infinities of the scale's other end (values near 1e308)."""
    import oracle

    A = [C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    host.host_zfp_encode_w64.argtypes = A
    host.host_zfp_decode_w64.argtypes = A
    rng = np.random.default_rng(9)
    for scale in (1e-300, 1e-306, 3e-308, 5e-320, 1e300, 1.5e308):
        with np.errstate(over="ignore"):
            f = np.ascontiguousarray(rng.standard_normal((4, 8, 4)) * scale)
        if scale > 1e307:
            f = np.clip(f, -1.7e308, 1.7e308)
        for maxbits in (512, 1030, 4096):
            words = 2 * maxbits // 64 + 1
            s = np.zeros(words + 2, dtype=np.uint64)
            host.host_zfp_encode_w64(f.ctypes.data, 0, 3, 4, 8, 4, maxbits, s.ctypes.data)
            want = oracle.zfp_encode_64(f, maxbits)
            assert np.array_equal(s[: want.size], want), (scale, maxbits)
            o = np.zeros_like(f)
            host.host_zfp_decode_w64(s.ctypes.data, 0, 3, 4, 8, 4, maxbits, o.ctypes.data)
            d = oracle.zfp_decode_64(want, f.shape, maxbits, np.float64)
            assert np.array_equal(o.view(np.uint64), d.view(np.uint64)), (scale, maxbits)


def test_unguarded_encoder_stays_inside_its_slack(host):
    """The encoder variant without end-of-block guards lets a block that runs out
    of budget finish its bit plane.  On noise, where a plane that starts with few
    significant coefficients finds many at once, what it writes past the block's
    end must stay within the 128 bits of slack, and the kept bits must equal the
    guarded encoder's."""
    rng = np.random.default_rng(11)
    for maxbits in (64, 128, 192, 256, 512):
        for scale in (1.0, 1e-3, 1e4):
            f = (rng.standard_normal((8, 16, 64)) * scale).astype(np.float32)
            f[rng.random(f.shape) < 0.1] *= 1e3          # a few outliers: leading planes with long runs
            nz, ny, nx = f.shape
            words = (nx // 4) * (ny // 4) * (nz // 4) * maxbits // 64
            a = np.zeros(words + 2, dtype=np.uint64)
            host.host_zfp_encode3(f.ctypes.data, nx, ny, nz, maxbits, a.ctypes.data)
            b = np.zeros(words, dtype=np.uint64)
            top = host.host_zfp_encode3_slots(f.ctypes.data, nx, ny, nz, maxbits, b.ctypes.data)
            assert np.array_equal(a[:words], b), (maxbits, scale)
            assert top < maxbits // 32 + 4, (maxbits, scale, top)


def test_fenced_decoder_ignores_what_lies_behind_its_fence(host):
    """The device gives every lane a slot of the block's bits and 64 one bits; what
    the decoder reads beyond those (the window it looks through is wider than what
    it uses) belongs to the next lane.  On noise and on fields with outliers, at
    every whole-word rate: the result does not depend on those bits, and no read
    goes further than 128 bits past the block."""
    rng = np.random.default_rng(12)
    for maxbits in (64, 128, 192, 256, 512, 1024, 2048):
        for scale in (1.0, 1e-3, 1e4):
            f = (rng.standard_normal((8, 16, 64)) * scale).astype(np.float32)
            f[rng.random(f.shape) < 0.1] *= 1e3
            f[:, :4, :8] = 0.0                             # empty blocks: nothing but the fence is looked at
            nz, ny, nx = f.shape
            words = (nx // 4) * (ny // 4) * (nz // 4) * maxbits // 64
            a = np.zeros(words + 2, dtype=np.uint64)
            host.host_zfp_encode3(f.ctypes.data, nx, ny, nz, maxbits, a.ctypes.data)
            plain = np.zeros_like(f)
            host.host_zfp_decode3(a.ctypes.data, nx, ny, nz, maxbits, plain.ctypes.data)
            for junk in (0, 1, 0xffffffff, 12345):
                o = np.zeros_like(f)
                top = host.host_zfp_decode3_fenced(a.ctypes.data, nx, ny, nz, maxbits, o.ctypes.data, junk)
                assert np.array_equal(o.view(np.uint32), plain.view(np.uint32)), (maxbits, scale, junk)
                assert top < maxbits // 32 + 4, (maxbits, scale, top)


# ---- the encoder's pair form: a block shared by two wavefronts (here: two host threads)
def _pair(host):
    host.host_zfp_encode3_pair.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    host.host_zfp_encode3_pair.restype = C.c_uint
    host.host_skip_plane_agrees.argtypes = [C.c_uint64, C.c_uint, C.c_uint, C.c_uint]
    host.host_skip_plane_agrees.restype = C.c_int
    host.host_zfp_decode3_pair.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint, C.c_void_p]
    host.host_zfp_decode3_pair.restype = C.c_int
    return host


@pytest.mark.timeout(300)
def test_skipping_a_plane_in_closed_form_leaves_the_coder_where_coding_it_does(host):
    """BlockEncoder::skip_plane against BlockEncoder::plane (the coder of
    encode.cuh:331-344) on single planes: every count of known coefficients, planes
    that are empty, full, sparse, dense, that end in the last coefficient."""
    L = _pair(host)
    rng = np.random.default_rng(11)
    planes = [0, 1, 2**63, 2**64 - 1, 2**63 | 1, 2**62, 0x5555555555555555, 0xAAAAAAAAAAAAAAAA, 2**32, 2**31]
    for dens in (0.02, 0.1, 0.5, 0.9):
        for _ in range(60):
            bits = rng.random(64) < dens
            planes.append(int(np.packbits(bits, bitorder="little").view(np.uint64)[0]))
    for k in range(64):
        planes += [1 << k, (1 << k) - 1 if k else 0, ((1 << 64) - 1) ^ ((1 << k) - 1)]
    bad = []
    for x in planes:
        for n in list(range(0, 65, 3)) + [1, 2, 62, 63, 64]:
            for pos in (9, 200, 511):
                if not L.host_skip_plane_agrees(x, n, pos, 2048):
                    bad.append((hex(x), n, pos))
    assert not bad, bad[:10]


@pytest.mark.timeout(600)
def test_pair_form_of_the_encoder_matches_golden_vectors_and_the_block_encoder(host, golden):
    """The pair form (two halves of a workgroup per block; here two threads with the
    kernel's reuse of its shared words) gives the streams of the golden vectors and of
    encode_block on random fields, at every whole-word rate incl. the ones that code the
    low 16 planes, and stays within the slot's 128 bits of slack."""
    L = _pair(host)
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden):
        nz, ny, nx = f.shape
        if nx % 4 or ny % 4 or nz % 4 or maxbits % 64:
            continue
        words = (nx // 4) * (ny // 4) * (nz // 4) * maxbits // 64
        s = np.zeros(words, dtype=np.uint64)
        top = L.host_zfp_encode3_pair(f.ctypes.data, nx, ny, nz, maxbits, s.ctypes.data)
        assert top != 0xFFFFFFFF
        assert np.array_equal(s.view(np.uint8), stream[:words * 8]), (name, rate)
        assert top < maxbits // 32 + 4, (name, rate, "wrote past the 128 bits of slack")
        n += 1
    assert n >= 20, n
    rng = np.random.default_rng(5)
    kinds = {
        "noise": lambda shape: rng.standard_normal(shape),
        "smooth": lambda shape: np.cumsum(np.cumsum(rng.standard_normal(shape), axis=2), axis=1) * 1e-3,
        "sparse": lambda shape: rng.standard_normal(shape) * (rng.random(shape) < 0.05),
        "wide": lambda shape: rng.standard_normal(shape) * np.exp(8 * rng.standard_normal(shape)),
        "const": lambda shape: np.full(shape, 1.5),
        "zero": lambda shape: np.zeros(shape),
        "tiny": lambda shape: rng.standard_normal(shape) * 1e-30,
    }
    for kind, make in kinds.items():
        for shape in ((4, 4, 4), (8, 12, 16), (12, 8, 20)):
            f = np.ascontiguousarray(make(shape), dtype=np.float32)
            nz, ny, nx = shape
            for maxbits in (64, 128, 256, 512, 1024, 2048, 4096):
                words = (nx // 4) * (ny // 4) * (nz // 4) * maxbits // 64
                want = np.zeros(words + 2, dtype=np.uint64)
                host.host_zfp_encode3(f.ctypes.data, nx, ny, nz, maxbits, want.ctypes.data)
                s = np.zeros(words, dtype=np.uint64)
                top = L.host_zfp_encode3_pair(f.ctypes.data, nx, ny, nz, maxbits, s.ctypes.data)
                assert np.array_equal(s, want[:words]), (kind, shape, maxbits)
                assert top < maxbits // 32 + 4, (kind, shape, maxbits, top)


@pytest.mark.timeout(600)
def test_pair_form_of_the_decoder_matches_golden_vectors_and_the_block_decoder(host, golden):
    """The decoder's pair form (half 0 decodes the bit planes, both halves share what follows; here
    two threads with the kernel's reuse of its shared words) gives the decoded values of the golden
    vectors and of decode_block on the streams of random fields, at every whole-word rate."""
    L = _pair(host)
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden):
        nz, ny, nx = f.shape
        if nx % 4 or ny % 4 or nz % 4 or maxbits % 64:
            continue
        words = (nx // 4) * (ny // 4) * (nz // 4) * maxbits // 64
        g = np.zeros(words * 8, dtype=np.uint8)
        g[:] = stream[:words * 8]
        o = np.full(f.shape, -7.0, dtype=np.float32)
        assert L.host_zfp_decode3_pair(g.ctypes.data, nx, ny, nz, maxbits, o.ctypes.data) == 0
        assert np.array_equal(o.view(np.uint32), dec.view(np.uint32)), (name, rate)
        n += 1
    assert n >= 20, n
    rng = np.random.default_rng(6)
    kinds = {
        "noise": lambda shape: rng.standard_normal(shape),
        "smooth": lambda shape: np.cumsum(np.cumsum(rng.standard_normal(shape), axis=2), axis=1) * 1e-3,
        "sparse": lambda shape: rng.standard_normal(shape) * (rng.random(shape) < 0.05),
        "wide": lambda shape: rng.standard_normal(shape) * np.exp(8 * rng.standard_normal(shape)),
        "const": lambda shape: np.full(shape, 1.5),
        "zero": lambda shape: np.zeros(shape),
    }
    for kind, make in kinds.items():
        for shape in ((4, 4, 4), (8, 12, 16)):
            f = np.ascontiguousarray(make(shape), dtype=np.float32)
            nz, ny, nx = shape
            for maxbits in (64, 128, 256, 512, 1024, 2048, 4096):
                words = (nx // 4) * (ny // 4) * (nz // 4) * maxbits // 64
                s = np.zeros(words + 2, dtype=np.uint64)
                host.host_zfp_encode3(f.ctypes.data, nx, ny, nz, maxbits, s.ctypes.data)
                want = np.zeros_like(f)
                host.host_zfp_decode3(s.ctypes.data, nx, ny, nz, maxbits, want.ctypes.data)
                o = np.full(f.shape, -7.0, dtype=np.float32)
                assert L.host_zfp_decode3_pair(s.ctypes.data, nx, ny, nz, maxbits, o.ctypes.data) == 0
                assert np.array_equal(o.view(np.uint32), want.view(np.uint32)), (kind, shape, maxbits)
