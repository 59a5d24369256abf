"""Pins the CPU checker's ZFP restatement (oracle/cswap_oracle.c) against
 (a) streams/decodes made by the stock zfp 0.5.5 serial codec (tests/golden),
 (b) what the mathematics fixes: lifting matrices, negabinary closed form,
     permutation ordering, header layout, block independence, brute force.
None of these retypes the oracle's own formulas."""
import hashlib
import math

import numpy as np
import pytest

import oracle
from conftest import MID_SIZE_CASES, golden_cases, libzfp, libzfp_round_trip, mid_size_field
from cswap_amd.workloads import config1_field, config3_fields


def test_golden_streams_and_decodes(golden):
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden):
        s = oracle.zfp_encode3(f, maxbits).view(np.uint8)
        k = min(s.size, stream.size)
        assert np.array_equal(s[:k], stream[:k]), (name, rate)
        assert not s[k:].any() and not stream[k:].any(), (name, rate)
        # decode the GOLDEN stream, not our own
        pad = np.zeros((-stream.size) % 8, dtype=np.uint8)
        d = oracle.zfp_decode3(np.concatenate([stream, pad]).view(np.uint64), f.shape, maxbits)
        assert np.array_equal(d.view(np.uint32), dec.view(np.uint32)), (name, rate)
        n += 1
    assert n >= 100


@pytest.mark.parametrize("rate", [4, 8, 16])
def test_config1_digests(digests, rate):
    f = config1_field()
    e = digests["config1_prelu_4096x32x32"]
    assert hashlib.sha256(f.tobytes()).hexdigest() == e["input_sha256"]
    s = oracle.zfp_encode3(f, 64 * rate)
    assert s.nbytes == e["rates"][str(rate)]["stream_bytes"]
    assert hashlib.sha256(s.tobytes()).hexdigest() == e["rates"][str(rate)]["stream_sha256"]
    d = oracle.zfp_decode3(s, f.shape, 64 * rate)
    assert hashlib.sha256(d.tobytes()).hexdigest() == e["rates"][str(rate)]["decoded_sha256"]
    assert float(np.max(np.abs(d.astype(np.float64) - f))) == pytest.approx(
        e["rates"][str(rate)]["max_abs_err"], rel=1e-12)


def test_config3_digests(digests):
    for name, f in config3_fields(batch=16).items():
        e = digests[f"config3_b16_{name}"]
        assert hashlib.sha256(f.tobytes()).hexdigest() == e["input_sha256"]
        for rate in (4, 8, 16):
            s = oracle.zfp_encode3(f, 64 * rate)
            r = e["rates"][str(rate)]
            sb = s.view(np.uint8)
            assert sb.size == r["stream_bytes"]
            assert hashlib.sha256(sb.tobytes()).hexdigest() == r["stream_sha256"], (name, rate)
            d = oracle.zfp_decode3(s, f.shape, 64 * rate)
            assert hashlib.sha256(d.tobytes()).hexdigest() == r["decoded_sha256"], (name, rate)


def test_stream_bytes_closed_form():
    for (nx, ny, nz) in [(32, 32, 4096), (2, 2, 65536), (7, 5, 6), (1, 1, 1), (3072, 512, 32)]:
        for maxbits in (256, 512, 1024, 288):
            blocks = math.ceil(nx / 4) * math.ceil(ny / 4) * math.ceil(nz / 4)
            assert oracle.zfp_stream_bytes(nx, ny, nz, maxbits) == (blocks * maxbits // 64) * 8


# ---- lifting: the matrices the reference documents (encode.cuh:84-88, shared.h:233-239)
FWD = np.array([[4, 4, 4, 4], [5, 1, -1, -5], [-4, 4, 4, -4], [-2, 6, -6, 2]], dtype=np.int64)
INV = np.array([[4, 6, -4, -1], [4, 2, 4, 5], [4, -2, 4, -5], [4, -6, -4, 1]], dtype=np.int64)


def test_fwd_lift_is_exact_matrix_on_multiples_of_16():
    rng = np.random.default_rng(0)
    for _ in range(2000):
        v = rng.integers(-2**20, 2**20, size=4) * 16
        assert np.array_equal(oracle.fwd_lift(v), FWD @ v // 16)


def test_inv_lift_is_exact_matrix_on_multiples_of_4():
    rng = np.random.default_rng(1)
    for _ in range(2000):
        v = rng.integers(-2**20, 2**20, size=4) * 4
        assert np.array_equal(oracle.inv_lift(v), INV @ v // 4)


def test_lift_near_inverse_and_wraparound():
    rng = np.random.default_rng(2)
    for _ in range(5000):
        v = rng.integers(-2**29, 2**29, size=4)
        r = oracle.inv_lift(oracle.fwd_lift(v))
        assert np.max(np.abs(r.astype(np.int64) - v)) <= 2
    # multiples of 4 in, forward matrix exact -> round trip exact
    for _ in range(2000):
        v = rng.integers(-2**24, 2**24, size=4) * 16
        assert np.array_equal(oracle.inv_lift(oracle.fwd_lift(v)), v)
    # wrap-around: must agree with Python big-int arithmetic reduced mod 2^32

    def wrap(a):
        return ((int(a) + 2**31) % 2**32) - 2**31

    def py_fwd(x, y, z, w):
        x = wrap(x + w); x >>= 1; w = wrap(w - x)
        z = wrap(z + y); z >>= 1; y = wrap(y - z)
        x = wrap(x + z); x >>= 1; z = wrap(z - x)
        w = wrap(w + y); w >>= 1; y = wrap(y - w)
        w = wrap(w + (y >> 1)); y = wrap(y - (w >> 1))
        return [x, y, z, w]

    for _ in range(2000):
        v = rng.integers(-2**31, 2**31, size=4)
        assert list(oracle.fwd_lift(v)) == py_fwd(*v)


def test_xform3_axis_order():
    # a field that varies only along one axis must decorrelate into that axis'
    # coefficients only: f(x,y,z)=16*g(x) -> non-zeros only at (i,0,0)
    g = np.array([1, 5, -3, 8]) * 1024
    for axis in range(3):
        shp = [1, 1, 1]
        shp[2 - axis] = 4
        b = np.broadcast_to(g.reshape(shp), (4, 4, 4)).astype(np.int32)  # [z][y][x]
        t = oracle.fwd_xform3(b.reshape(64)).reshape(4, 4, 4)
        line = np.moveaxis(t, 2 - axis, 0)[:, 0, 0]
        assert np.array_equal(line, FWD @ g // 16)
        mask = np.ones((4, 4, 4), bool)
        idx = [0, 0, 0]
        idx[2 - axis] = slice(None)
        mask[tuple(idx)] = False
        assert not t[mask].any()


def test_negabinary_closed_form_and_bijection():
    rng = np.random.default_rng(3)
    xs = list(rng.integers(-2**31, 2**31, size=3000)) + [0, 1, -1, 2**31 - 1, -2**31]
    for x in xs:
        u = oracle.lib().orc_int2uint(int(x))
        # negabinary: sum of bit_i * (-2)^i == x  (mod 2^32)
        val = sum(((u >> i) & 1) * (-2) ** i for i in range(32))
        assert (val - int(x)) % 2**32 == 0
        assert oracle.lib().orc_uint2int(u) == int(x)


def test_perm3_is_sequency_sorted_permutation():
    p = oracle.perm3()
    assert sorted(p) == list(range(64))
    keys = [((i & 3) + ((i >> 2) & 3) + (i >> 4), (i & 3) ** 2 + ((i >> 2) & 3) ** 2 + (i >> 4) ** 2)
            for i in p]
    assert keys == sorted(keys)


def test_emax_matches_frexp():
    rng = np.random.default_rng(4)
    for _ in range(500):
        b = (rng.standard_normal(64) * 2.0 ** rng.integers(-30, 30)).astype(np.float32)
        assert oracle.block_emax(b) == math.frexp(float(np.max(np.abs(b))))[1]
    assert oracle.block_emax(np.zeros(64, np.float32)) == -127
    one = np.zeros(64, np.float32); one[5] = 1.0
    assert oracle.block_emax(one) == 1


def test_cast_truncates_toward_zero():
    b = np.array([0.75, -0.75, 0.999999, -0.999999] * 16, dtype=np.float32)
    i = oracle.fwd_cast(b, 0)  # scale 2^30
    assert list(i[:4]) == [int(0.75 * 2**30), -int(0.75 * 2**30),
                           int(float(np.float32(0.999999)) * 2**30),
                           -int(float(np.float32(0.999999)) * 2**30)]


def test_header_and_empty_block():
    z = oracle.zfp_encode_block(np.zeros(64, np.float32), 512)
    assert not z.any()
    one = np.zeros(64, np.float32); one[0] = 1.0          # emax = 1 -> e = 128
    w = oracle.zfp_encode_block(one, 512)
    assert int(w[0]) & 0x1ff == 2 * 128 + 1
    tiny = np.full(64, 2.0 ** -100, np.float32)            # emax = -99 -> e = 28
    assert int(oracle.zfp_encode_block(tiny, 512)[0]) & 0x1ff == 2 * 28 + 1


def test_blocks_are_independent_of_position():
    rng = np.random.default_rng(5)
    f = rng.standard_normal((4, 4, 16)).astype(np.float32)  # 4 blocks along x
    s = oracle.zfp_encode3(f, 512).reshape(4, 8)
    perm = [2, 0, 3, 1]
    f2 = np.concatenate([f[:, :, 4 * p:4 * p + 4] for p in perm], axis=2)
    s2 = oracle.zfp_encode3(np.ascontiguousarray(f2), 512).reshape(4, 8)
    assert np.array_equal(s2, s[perm])


def test_budget_is_prefix_cut():
    """A smaller bit budget yields exactly a prefix of a larger budget's block."""
    rng = np.random.default_rng(6)
    for _ in range(50):
        b = rng.standard_normal(64).astype(np.float32)
        big = oracle.zfp_encode_block(b, 2048)
        bits_big = np.unpackbits(big.view(np.uint8), bitorder="little")
        for mb in (64, 100, 256, 300, 512, 777):
            small = oracle.zfp_encode_block(b, mb)
            bits = np.unpackbits(small.view(np.uint8), bitorder="little")
            assert np.array_equal(bits[:mb], bits_big[:mb])
            assert not bits[mb:].any()


def test_full_precision_roundtrip_is_near_lossless():
    """With an (effectively) unlimited budget every bit plane is coded, so the
    decoder must reproduce the integer coefficients: error <= a few ulps of the
    block-floating-point grid 2^(emax-30)."""
    rng = np.random.default_rng(7)
    for _ in range(50):
        b = rng.standard_normal(64).astype(np.float32)
        w = oracle.zfp_encode_block(b, 4096)
        d = oracle.zfp_decode_block(w, 4096)
        emax = oracle.block_emax(b)
        assert np.max(np.abs(d.astype(np.float64) - b)) <= 64 * 2.0 ** (emax - 30)


def test_ref_host_bitstream_order_and_max_size():
    """Where the reference's own host C built (oracle/_ref), its bit stream must
    agree with the checker's bit order, and its stream-size bookkeeping with the
    closed form."""
    import ctypes as C

    ref = oracle.ref_host_lib()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference sources absent)")
    ref.stream_open.restype = C.c_void_p
    ref.stream_open.argtypes = [C.c_void_p, C.c_size_t]
    ref.stream_write_bits.restype = C.c_uint64
    ref.stream_write_bits.argtypes = [C.c_void_p, C.c_uint64, C.c_uint]
    ref.stream_flush.argtypes = [C.c_void_p]
    ref.stream_close.argtypes = [C.c_void_p]
    buf = np.zeros(8, dtype=np.uint64)
    bs = ref.stream_open(buf.ctypes.data, buf.nbytes)
    # a block header followed by odd-sized pieces
    pieces = [(2 * 130 + 1, 9), (0x5, 3), (0xdeadbeefcafef00d, 64), (1, 1), (0x3ff, 10), (0x123456789, 37)]
    for v, n in pieces:
        ref.stream_write_bits(bs, v, n)
    ref.stream_flush(bs)
    ref.stream_close(bs)
    bits = []
    for v, n in pieces:
        bits += [(v >> i) & 1 for i in range(n)]
    want = np.zeros(8 * 64, dtype=np.uint8)
    want[: len(bits)] = bits
    assert np.array_equal(np.unpackbits(buf.view(np.uint8), bitorder="little"), want)
    # the first 9 bits are what the checker writes as a header for e = 130
    blk = np.zeros(64, np.float32); blk[0] = 5.0  # emax = 3 -> e = 130
    assert int(oracle.zfp_encode_block(blk, 512)[0]) & 0x1ff == int(buf[0]) & 0x1ff


def test_golden_streams_and_decodes_1d_2d(golden_12d):
    """The 2-D and 1-D restatements (4x4 and 4-value blocks) against zfp 0.5.5."""
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_12d):
        s = oracle.zfp_encode_nd(f, maxbits).view(np.uint8)
        k = min(s.size, stream.size)
        assert np.array_equal(s[:k], stream[:k]), (name, rate)
        assert not s[k:].any() and not stream[k:].any(), (name, rate)
        pad = np.zeros((-stream.size) % 8, dtype=np.uint8)
        d = oracle.zfp_decode_nd(np.concatenate([stream, pad]).view(np.uint64), f.shape, maxbits)
        assert np.array_equal(d.view(np.uint32), dec.view(np.uint32)), (name, rate)
        n += 1
    assert n >= 60


def test_perm2_is_sequency_sorted_permutation():
    p = np.zeros(16, dtype=np.uint8)
    oracle.lib().orc_perm2(p.ctypes.data)
    assert sorted(p) == list(range(16))
    keys = [((i & 3) + (i >> 2), (i & 3) ** 2 + (i >> 2) ** 2) for i in p]
    assert keys == sorted(keys)


def test_int32_fields_match_golden_vectors(golden_i32):
    """zfp_type_int32 (cuZFP.cu:412-416,513-517): no exponent header, no cast, the
    whole block budget goes to the coder.  Streams and decoded values of the zfp
    0.5.5 command-line codec (-t i32) for 1-D, 2-D and 3-D fields, partial blocks,
    all-zero and constant blocks, values up to 2^30, rates from 1 to 32."""
    import oracle

    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_i32):
        assert f.dtype == np.int32
        s = oracle.zfp_encode_i32(f, maxbits)
        sb = s.view(np.uint8)
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any(), (name, rate)
        d = oracle.zfp_decode_i32(stream[: (stream.size // 8) * 8].view(np.uint64) if stream.size % 8 == 0
                                  else np.frombuffer(stream.tobytes() + bytes(8 - stream.size % 8), dtype=np.uint64),
                                  f.shape, maxbits)
        assert np.array_equal(d, dec), (name, rate)
        n += 1
    assert n == 99


def _words(stream):
    if stream.size % 8 == 0:
        return stream.view(np.uint64)
    return np.frombuffer(stream.tobytes() + bytes(8 - stream.size % 8), dtype=np.uint64)


def test_64_bit_fields_match_golden_vectors(golden_64):
    """zfp_type_double and zfp_type_int64 (cuZFP.cu:401-423,479-504): 64 bit planes,
    for doubles a 12-bit header and the scale 2^(62-emax).  Streams and decoded
    values of the zfp 0.5.5 command-line codec (-d, -t i64) for 1-D, 2-D and 3-D
    fields: partial, all-zero, negative-zero and constant blocks, magnitudes from
    1e-250 to 1e250 inside one field, integers up to 2^61, rates 1 to 64."""
    import oracle

    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_64):
        assert f.dtype == (np.int64 if name[0] == "l" else np.float64)
        sb = oracle.zfp_encode_64(f, maxbits).view(np.uint8)
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any(), (name, rate)
        d = oracle.zfp_decode_64(_words(stream), f.shape, maxbits, f.dtype)
        assert np.array_equal(d.view(np.uint64), dec.view(np.uint64)), (name, rate)
        n += 1
    assert n == 187


def test_64_bit_high_rate_is_nearly_lossless():
    import oracle

    rng = np.random.default_rng(6)
    f = rng.integers(-2**58, 2**58, (8, 8, 8))
    d = oracle.zfp_decode_64(oracle.zfp_encode_64(f, 64 * 72), f.shape, 64 * 72, np.int64)
    assert np.abs(d - f).max() <= 32
    x = rng.standard_normal((4, 8, 12))
    y = oracle.zfp_decode_64(oracle.zfp_encode_64(x, 64 * 64), x.shape, 64 * 64, np.float64)
    assert np.abs(y - x).max() < 1e-15 * 64
    z = np.zeros((4, 4, 4))
    assert not oracle.zfp_encode_64(z, 512).any()
    # the reference's decoder leaves an empty block untouched; the field level pre-zeroes it
    assert not oracle.zfp_decode_64(np.zeros(8, dtype=np.uint64), z.shape, 512, np.float64).any()


def test_int32_high_rate_is_nearly_lossless():
    """With 32 bits per value the coder runs through every plane; what is left is
    the rounding of the lifting transform: at most a few units per component."""
    import oracle

    rng = np.random.default_rng(5)
    f = rng.integers(-2**28, 2**28, (8, 8, 8)).astype(np.int32)
    d = oracle.zfp_decode_i32(oracle.zfp_encode_i32(f, 64 * 40), f.shape, 64 * 40)
    assert np.abs(d.astype(np.int64) - f).max() <= 32       # three lifting passes, each rounding twice
    z = np.zeros((4, 4, 4), dtype=np.int32)
    s = oracle.zfp_encode_i32(z, 512)
    assert not s.any()                       # zeros code as zero bits: every plane is a negative group test
    assert not oracle.zfp_decode_i32(s, z.shape, 512).any()


@pytest.mark.parametrize("kind", ["f32", "i32", "f64", "i64"])
@pytest.mark.parametrize("shape,rate", MID_SIZE_CASES)
def test_checker_equals_the_zfp_library_on_mid_size_fields(kind, shape, rate):
    """The checker against the stock zfp 0.5.5 library (where this machine has
    it) on fields of a few hundred thousand values of every scalar type and
    dimensionality: stream bytes and decoded values."""
    import oracle

    Z = libzfp()
    if Z is None:
        pytest.skip("no zfp 0.5.5 library on this machine")
    f = mid_size_field(kind, shape, rate)
    maxbits, stream, dec = libzfp_round_trip(Z, f, rate)
    if kind == "f32":
        s = oracle.zfp_encode_nd(f, maxbits)
        d = oracle.zfp_decode_nd(s, f.shape, maxbits)
    elif kind == "i32":
        s = oracle.zfp_encode_i32(f, maxbits)
        d = oracle.zfp_decode_i32(s, f.shape, maxbits)
    else:
        s = oracle.zfp_encode_64(f, maxbits)
        d = oracle.zfp_decode_64(s, f.shape, maxbits, f.dtype)
    sb = s.view(np.uint8)
    k = min(sb.size, stream.size)
    assert np.array_equal(sb[:k], stream[:k]), (kind, shape, maxbits)
    assert not sb[k:].any() and not stream[k:].any()
    assert np.array_equal(d.view(np.uint8), dec.view(np.uint8)), (kind, shape, maxbits)
