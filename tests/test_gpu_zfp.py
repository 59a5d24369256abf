"""GPU parity of the ZFP fixed-rate codec: the HIP path (through the C ABI) must
be bit-exact against the committed zfp 0.5.5 golden vectors and against the CPU
checker on the same seeded inputs."""
import hashlib
import os

import numpy as np
import pytest

from conftest import MID_SIZE_CASES, golden_cases, libzfp as _libzfp, libzfp_round_trip, mid_size_field

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


SIZE_MAX = 2 ** 64 - 1
FORMS = {"as shipped": None, "one lane per block": (0, 0), "pair form wherever the shape allows": (SIZE_MAX, SIZE_MAX)}


@pytest.fixture(params=list(FORMS))
def zfp_form(request):
    """Which form of the 3-D fp32 kernels runs: the shipped size thresholds, the form with
    one lane per block for every field, or the pair form (two wavefronts per 64 blocks)
    for every field whose shape allows it."""
    import ctypes as C

    from cswap_amd._lib import lib

    want = FORMS[request.param]
    if want is None:
        yield request.param
        return
    before = (C.c_size_t * 2)()
    lib().cswap_zfp_set_pair_bytes(want[0], want[1], before)
    yield request.param
    lib().cswap_zfp_set_pair_bytes(before[0], before[1], None)


def gpu_encode(torch, f, maxbits):
    from cswap_amd import api

    t = torch.from_numpy(np.ascontiguousarray(f)).cuda()
    s = api.cuda_compress(t, maxbits)
    torch.cuda.synchronize()
    return s


def test_golden_vectors(torch_cuda, golden, zfp_form):
    torch = torch_cuda
    from cswap_amd import api

    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden):
        print("case", name, rate, flush=True)
        s = gpu_encode(torch, f, maxbits)
        sb = s.cpu().numpy()
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any(), (name, rate)
        # decode the golden stream
        gs = np.zeros(sb.size, dtype=np.uint8)
        gs[:k] = stream[:k]
        d = api.cuda_decompress(torch.from_numpy(gs).cuda(), f.shape, maxbits)
        torch.cuda.synchronize()
        assert np.array_equal(d.cpu().numpy().view(np.uint32), dec.view(np.uint32)), (name, rate)
        n += 1
    assert n >= 100


@pytest.mark.parametrize("rate", [4, 8, 16])
def test_config1_bit_exact(torch_cuda, digests, rate, zfp_form):
    torch = torch_cuda
    import oracle
    from cswap_amd import api
    from cswap_amd.workloads import config1_field

    f = config1_field()
    e = digests["config1_prelu_4096x32x32"]["rates"][str(rate)]
    s = gpu_encode(torch, f, 64 * rate)
    sb = s.cpu().numpy()
    assert sb.size == e["stream_bytes"]
    assert hashlib.sha256(sb.tobytes()).hexdigest() == e["stream_sha256"]
    assert np.array_equal(sb.view(np.uint64), oracle.zfp_encode3(f, 64 * rate))
    d = api.cuda_decompress(s, f.shape, 64 * rate)
    torch.cuda.synchronize()
    dn = d.cpu().numpy()
    assert hashlib.sha256(dn.tobytes()).hexdigest() == e["decoded_sha256"]


@pytest.mark.parametrize("rate", [4, 8, 16])
def test_config3_stack_vs_checker(torch_cuda, rate, zfp_form):
    torch = torch_cuda
    import oracle
    from cswap_amd import api
    from cswap_amd.workloads import config3_fields

    for name, f in config3_fields(batch=128).items():
        print("case", name, rate, f.shape, flush=True)
        s = gpu_encode(torch, f, 64 * rate)
        want = oracle.zfp_encode3(f, 64 * rate, omp=True)
        assert np.array_equal(s.cpu().numpy().view(np.uint64), want), name
        d = api.cuda_decompress(s, f.shape, 64 * rate)
        torch.cuda.synchronize()
        wd = oracle.zfp_decode3(want, f.shape, 64 * rate, omp=True)
        assert np.array_equal(d.cpu().numpy().view(np.uint32), wd.view(np.uint32)), name


@pytest.mark.parametrize("shape", [(5, 7, 9), (1, 1, 1), (3, 4, 130), (9, 2, 2), (2, 257, 3), (64, 8, 12)])
@pytest.mark.parametrize("maxbits", [64, 100, 288, 512, 1000, 2048])
def test_ragged_shapes_and_odd_rates(torch_cuda, shape, maxbits):
    torch = torch_cuda
    import oracle
    from cswap_amd import api

    rng = np.random.default_rng(sum(shape) * 4099 + maxbits)
    f = (rng.standard_normal(shape) * 10.0 ** rng.integers(-3, 4)).astype(np.float32)
    s = gpu_encode(torch, f, maxbits)
    want = oracle.zfp_encode3(f, maxbits)
    assert np.array_equal(s.cpu().numpy().view(np.uint64), want)
    d = api.cuda_decompress(s, f.shape, maxbits)
    torch.cuda.synchronize()
    assert np.array_equal(d.cpu().numpy().view(np.uint32),
                          oracle.zfp_decode3(want, f.shape, maxbits).view(np.uint32))


def test_strided_field(torch_cuda):
    """Non-default strides (zfp/cuZFP.cu:372-375): a field embedded in a larger
    allocation must code exactly like its contiguous copy."""
    torch = torch_cuda
    import oracle
    from cswap_amd._lib import check, lib

    rng = np.random.default_rng(11)
    big = rng.standard_normal((10, 12, 20)).astype(np.float32)
    sub = np.ascontiguousarray(big[1:9, 2:10, 3:19])           # (8, 8, 16)
    tb = torch.from_numpy(big).cuda()
    nz, ny, nx = sub.shape
    cap = lib().cswap_zfp_stream_capacity(nx, ny, nz, 512)
    s = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    base = tb.data_ptr() + 4 * (1 * 12 * 20 + 2 * 20 + 3)
    check(lib().cswap_zfp_compress_f32(base, nx, ny, nz, 1, 20, 240, 512, s.data_ptr(), None), "compress")
    torch.cuda.synchronize()
    want = oracle.zfp_encode3(sub, 512)
    assert np.array_equal(s.cpu().numpy().view(np.uint64), want)
    out = torch.full((10, 12, 20), -7.0, dtype=torch.float32, device="cuda")
    check(lib().cswap_zfp_decompress_f32(s.data_ptr(), nx, ny, nz, 1, 20, 240, 512,
                                         out.data_ptr() + 4 * (1 * 12 * 20 + 2 * 20 + 3), None), "decompress")
    torch.cuda.synchronize()
    o = out.cpu().numpy()
    assert np.array_equal(o[1:9, 2:10, 3:19].view(np.uint32), oracle.zfp_decode3(want, sub.shape, 512).view(np.uint32))
    o[1:9, 2:10, 3:19] = -7.0
    assert np.all(o == -7.0)   # nothing outside the field was touched


@pytest.mark.parametrize("case", ["padded_rows_and_planes", "one_block_per_slab", "slab_crossing", "planes_before_rows",
                                  "big_offsets"])
def test_aligned_strided_fields(torch_cuda, case, zfp_form):
    """Fields embedded in larger allocations with 16-byte aligned rows: these take
    the 16-byte row path with a wave-uniform base and 32-bit lane offsets (a
    wavefront's 64 blocks may span many slabs of four planes), except when the
    strides do not nest (planes closer together than rows), which must fall back
    to the element path.  Either way the stream equals that of the contiguous copy
    and nothing outside the field is written."""
    torch = torch_cuda
    import oracle
    from cswap_amd._lib import check, lib

    rng = np.random.default_rng(sum(map(ord, case)))
    if case == "padded_rows_and_planes":
        alloc, sl = (14, 12, 24), (slice(1, 13), slice(4, 12), slice(4, 20))       # (12, 8, 16) inside
    elif case == "one_block_per_slab":
        alloc, sl = (400, 4, 8), (slice(0, 400), slice(0, 4), slice(4, 8))         # nx = ny = 4: 64 blocks = 64 slabs
    elif case == "slab_crossing":
        alloc, sl = (24, 20, 28), (slice(0, 24), slice(0, 20), slice(0, 28))       # 35 blocks per slab, contiguous
    elif case == "big_offsets":
        alloc, sl = (40, 260, 1028), (slice(4, 36), slice(0, 256), slice(4, 1028))  # 40 MB allocation
    else:
        alloc, sl = None, None
    if case == "planes_before_rows":
        # memory order (y, z, x): sy = 8*16, sz = 16  -> planes are closer together than rows
        big = rng.standard_normal((8, 8, 16)).astype(np.float32)                   # [y][z][x]
        sub = np.ascontiguousarray(big.transpose(1, 0, 2))                         # field [z][y][x]
        nz, ny, nx = sub.shape
        sx, sy, sz, off = 1, 8 * 16, 16, 0
    else:
        big = rng.standard_normal(alloc).astype(np.float32)
        sub = np.ascontiguousarray(big[sl])
        nz, ny, nx = sub.shape
        sx, sy, sz = 1, alloc[2], alloc[1] * alloc[2]
        off = sl[0].start * sz + sl[1].start * sy + sl[2].start
    tb = torch.from_numpy(big).cuda()
    assert (tb.data_ptr() + 4 * off) % 16 == 0
    cap = lib().cswap_zfp_stream_capacity(nx, ny, nz, 512)
    s = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    check(lib().cswap_zfp_compress_f32(tb.data_ptr() + 4 * off, nx, ny, nz, sx, sy, sz, 512, s.data_ptr(), None),
          "compress")
    torch.cuda.synchronize()
    want = oracle.zfp_encode3(sub, 512, omp=True)
    assert np.array_equal(s.cpu().numpy().view(np.uint64), want)
    out = torch.full(big.shape, -7.0, dtype=torch.float32, device="cuda")
    check(lib().cswap_zfp_decompress_f32(s.data_ptr(), nx, ny, nz, sx, sy, sz, 512, out.data_ptr() + 4 * off, None),
          "decompress")
    torch.cuda.synchronize()
    o = out.cpu().numpy()
    dec = oracle.zfp_decode3(want, sub.shape, 512, omp=True)
    if case == "planes_before_rows":
        assert np.array_equal(o.transpose(1, 0, 2).view(np.uint32), dec.view(np.uint32))
    else:
        assert np.array_equal(o[sl].view(np.uint32), dec.view(np.uint32))
        o[sl] = -7.0
        assert np.all(o == -7.0)   # nothing outside the field was touched


def test_large_tensor_properties(torch_cuda):
    """At full size (402 MB softmax-shaped tensor) the checker is too slow, so
    use properties that hold at any size: (a) a sampled slab equals the checker,
    (b) the reconstruction error is bounded relative to the field maximum, (c) all-zero slabs give all-zero stream words."""
    torch = torch_cuda
    import oracle
    from cswap_amd import api

    g = torch.Generator(device="cuda"); g.manual_seed(0)
    x = torch.softmax(torch.randn((32, 12, 512, 512), generator=g, device="cuda"), dim=-1).contiguous()
    x[5].zero_()
    s = api.cuda_compress(x, 512)
    d = api.cuda_decompress(s, x.shape, 512)
    torch.cuda.synchronize()
    assert s.numel() == x.numel()          # rate 8: one stream byte per value
    # (a) slab 7 of the batch: 12*512 z-planes -> a contiguous range of blocks
    slab = x[7].cpu().numpy().reshape(-1, 512, 512)
    words_per_slab = s.numel() // 8 // 32
    sw = s.view(torch.int64)[7 * words_per_slab:8 * words_per_slab].cpu().numpy().view(np.uint64)
    assert np.array_equal(sw, oracle.zfp_encode3(slab, 512, omp=True))
    dw = d[7].cpu().numpy().reshape(-1, 512, 512)
    assert np.array_equal(dw.view(np.uint32), oracle.zfp_decode3(sw, slab.shape, 512, omp=True).view(np.uint32))
    # (c) zero slab -> zero words, decodes to +0.0
    assert not s.view(torch.int64)[5 * words_per_slab:6 * words_per_slab].any().item()
    assert not d[5].view(torch.int32).any().item()
    # (b) rate 8 keeps ~3 significant bits of the block maximum: the error stays
    # well below the largest value of the field
    assert float((d - x).abs().max()) < 0.125 * float(x.max())


def nd_args(shape):
    """(dims, nx, ny, nz) of a C-contiguous field of 1, 2 or 3 dimensions."""
    ext = list(reversed(shape)) + [0, 0]
    return len(shape), ext[0], ext[1], ext[2]


def gpu_codec_nd(torch, f, maxbits, stream_bytes=None):
    from cswap_amd._lib import check, lib

    L = lib()
    dims, nx, ny, nz = nd_args(f.shape)
    cap = L.cswap_zfp_stream_capacity_nd(dims, nx, ny, nz, maxbits)
    t = torch.from_numpy(np.ascontiguousarray(f)).cuda()
    s = torch.empty(cap, dtype=torch.uint8, device="cuda")
    check(L.cswap_zfp_compress_f32_nd(t.data_ptr(), dims, nx, ny, nz, 0, 0, 0, maxbits, s.data_ptr(), None), "enc")
    if stream_bytes is not None:          # decode a given stream instead of our own
        g = np.zeros(cap, dtype=np.uint8)
        k = min(cap, stream_bytes.size)
        g[:k] = stream_bytes[:k]
        src = torch.from_numpy(g).cuda()
    else:
        src = s
    out = torch.full(f.shape, -3.0, dtype=torch.float32, device="cuda")
    check(L.cswap_zfp_decompress_f32_nd(src.data_ptr(), dims, nx, ny, nz, 0, 0, 0, maxbits, out.data_ptr(), None),
          "dec")
    torch.cuda.synchronize()
    return s.cpu().numpy(), out.cpu().numpy()


def test_golden_vectors_1d_2d(torch_cuda, golden_12d):
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_12d):
        print("case", name, rate, flush=True)
        sb, d = gpu_codec_nd(torch_cuda, f, maxbits, stream_bytes=stream)
        k = min(sb.size, stream.size)
        assert np.array_equal(sb[:k], stream[:k]), (name, rate)
        assert not sb[k:].any() and not stream[k:].any(), (name, rate)
        assert np.array_equal(d.view(np.uint32), dec.view(np.uint32)), (name, rate)
        n += 1
    assert n >= 60


@pytest.mark.parametrize("shape,maxbits", [((1000, 333), 128), ((257, 1030), 200), ((4096, 768), 64),
                                            ((100003,), 32), ((1 << 20,), 48), ((777,), 16)])
def test_larger_1d_2d_fields_vs_checker(torch_cuda, shape, maxbits):
    import oracle

    rng = np.random.default_rng(sum(shape) + maxbits)
    f = np.maximum(rng.standard_normal(shape), -0.2).astype(np.float32)
    sb, d = gpu_codec_nd(torch_cuda, f, maxbits)
    want = oracle.zfp_encode_nd(f, maxbits)
    assert np.array_equal(sb.view(np.uint64), want)
    assert np.array_equal(d.view(np.uint32), oracle.zfp_decode_nd(want, f.shape, maxbits).view(np.uint32))


def _gpu_i32(torch, f, maxbits):
    from cswap_amd._lib import check, lib

    L = lib()
    shp = (1,) * (3 - f.ndim) + f.shape
    nz, ny, nx = shp
    t = torch.from_numpy(f).cuda()
    cap = L.cswap_zfp_stream_capacity_nd(f.ndim, nx, ny, nz, maxbits)
    s = torch.zeros(cap + 16, dtype=torch.uint8, device="cuda")
    check(L.cswap_zfp_compress_i32_nd(t.data_ptr(), f.ndim, nx, ny, nz, 0, 0, 0, maxbits, s.data_ptr(), None), "c")
    o = torch.full(f.shape, -123456, dtype=torch.int32, device="cuda")
    check(L.cswap_zfp_decompress_i32_nd(s.data_ptr(), f.ndim, nx, ny, nz, 0, 0, 0, maxbits, o.data_ptr(), None), "d")
    torch.cuda.synchronize()
    return s[:cap].cpu().numpy(), o.cpu().numpy()


def test_int32_golden_vectors(torch_cuda, golden_i32):
    """zfp_type_int32 fields of 1, 2 and 3 dimensions (cuZFP.cu:412-416,513-517)
    against the zfp 0.5.5 vectors: stream bytes and decoded values."""
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_i32):
        s, o = _gpu_i32(torch_cuda, f, maxbits)
        k = min(s.size, stream.size)
        assert np.array_equal(s[:k], stream[:k]), (name, rate)
        assert not s[k:].any() and not stream[k:].any(), (name, rate)
        assert np.array_equal(o, dec), (name, rate)
        n += 1
    assert n == 99


@pytest.mark.parametrize("shape,maxbits", [((40, 36, 132), 512), ((33, 7, 9), 288), ((300, 260), 128), ((5000,), 40),
                                           ((64, 64, 64), 1024),
                                           ((32, 1024, 1024), 1024)])   # 128 MiB: loaded with the nontemporal hint
def test_int32_fields_vs_checker(torch_cuda, shape, maxbits):
    import oracle

    rng = np.random.default_rng(sum(shape) + maxbits)
    f = (rng.standard_normal(shape) * 10.0 ** rng.integers(2, 8)).astype(np.int32)
    s, o = _gpu_i32(torch_cuda, f, maxbits)
    want = oracle.zfp_encode_i32(f, maxbits)
    assert np.array_equal(s.view(np.uint64), want)
    assert np.array_equal(o, oracle.zfp_decode_i32(want, f.shape, maxbits))


def test_cuda_compress_dispatches_on_the_scalar_type(torch_cuda):
    """cuda_compress / cuda_decompress look at field->type (cuZFP.cu:388-423): all
    four scalar types are coded; an unknown type reports failure (size 0 / stream
    pointer not advanced)."""
    torch = torch_cuda
    import ctypes as C

    import oracle
    from cswap_amd import api
    from cswap_amd._lib import ZfpBitstream, ZfpField, ZfpStream, lib

    L = lib()
    rng = np.random.default_rng(3)
    fields = {1: rng.integers(-2**20, 2**20, (8, 12, 16)).astype(np.int32),
              2: rng.integers(-2**50, 2**50, (8, 12, 16)),
              3: rng.standard_normal((8, 12, 16)).astype(np.float32),
              4: rng.standard_normal((8, 12, 16)) * 1e10}
    for ztype, f in fields.items():
        t = torch.from_numpy(f).cuda()
        if ztype == 1:
            want = oracle.zfp_encode_i32(f, 512)
            dec = oracle.zfp_decode_i32(want, f.shape, 512)
        elif ztype == 3:
            want = oracle.zfp_encode3(f, 512)
            dec = oracle.zfp_decode3(want, f.shape, 512)
        else:
            want = oracle.zfp_encode_64(f, 512)
            dec = oracle.zfp_decode_64(want, f.shape, 512, f.dtype)
        # torch-facing wrapper
        s = api.cuda_compress(t, 512)
        assert np.array_equal(s.cpu().numpy().view(np.uint64)[: want.size], want), ztype
        d = api.cuda_decompress(s, f.shape, 512, dtype=t.dtype)
        torch.cuda.synchronize()
        assert np.array_equal(d.cpu().numpy().view(np.uint8), dec.view(np.uint8)), ztype
        # the reference-named entry points with zfp_field.type = ztype
        cap = L.cswap_zfp_stream_capacity(16, 12, 8, 512)
        sbuf = torch.zeros(cap, dtype=torch.uint8, device="cuda")
        bs = ZfpBitstream(0, 0, sbuf.data_ptr(), sbuf.data_ptr(), sbuf.data_ptr() + cap)
        zs = ZfpStream(1, 512, 64, -1074, C.pointer(bs), 0, 0, 0)
        fld = ZfpField(ztype, 16, 12, 8, 0, 0, 0, 0, 0, t.data_ptr())
        assert L.cuda_compress(C.byref(zs), C.byref(fld)) == cap
        assert np.array_equal(sbuf.cpu().numpy().view(np.uint64), want), ztype
        back = torch.zeros_like(t)
        bs.ptr = bs.begin
        fld_out = ZfpField(ztype, 16, 12, 8, 0, 0, 0, 0, 0, back.data_ptr())
        L.cuda_decompress(C.byref(zs), C.byref(fld_out))
        assert bs.ptr == bs.begin + cap
        assert np.array_equal(back.cpu().numpy().view(np.uint8), dec.view(np.uint8)), ztype
        # a host-resident field of the same type goes through the staged path
        hs = np.zeros(cap // 8, dtype=np.uint64)
        hb = ZfpBitstream(0, 0, hs.ctypes.data, hs.ctypes.data, hs.ctypes.data + cap)
        hz = ZfpStream(1, 512, 64, -1074, C.pointer(hb), 0, 0, 0)
        hf = ZfpField(ztype, 16, 12, 8, 0, 0, 0, 0, 0, f.ctypes.data)
        assert L.cuda_compress(C.byref(hz), C.byref(hf)) == cap
        assert np.array_equal(hs, want), ztype
    with pytest.raises((RuntimeError, TypeError, ValueError)):
        api.cuda_compress(torch.zeros(4, 4, 4, dtype=torch.float16, device="cuda"), 512)
    bs.ptr = bs.begin
    bad = ZfpField(0, 16, 12, 8, 0, 0, 0, 0, 0, t.data_ptr())
    assert L.cuda_compress(C.byref(zs), C.byref(bad)) == 0


def _gpu_w64(torch, f, maxbits, strides=None):
    from cswap_amd._lib import check, lib

    L = lib()
    kind = "i64" if f.dtype == np.int64 else "f64"
    shp = (1,) * (3 - f.ndim) + f.shape
    nz, ny, nx = shp
    t = torch.from_numpy(f).cuda()
    cap = L.cswap_zfp_stream_capacity_nd(f.ndim, nx, ny, nz, maxbits)
    s = torch.zeros(cap + 16, dtype=torch.uint8, device="cuda")
    check(getattr(L, f"cswap_zfp_compress_{kind}_nd")(t.data_ptr(), f.ndim, nx, ny, nz, 0, 0, 0, maxbits,
                                                        s.data_ptr(), None), "c")
    o = torch.full(f.shape, -123456, dtype=t.dtype, device="cuda")
    check(getattr(L, f"cswap_zfp_decompress_{kind}_nd")(s.data_ptr(), f.ndim, nx, ny, nz, 0, 0, 0, maxbits,
                                                          o.data_ptr(), None), "d")
    torch.cuda.synchronize()
    return s[:cap].cpu().numpy(), o.cpu().numpy()


def test_64_bit_golden_vectors(torch_cuda, golden_64):
    """zfp_type_double and zfp_type_int64 fields of 1, 2 and 3 dimensions
    (cuZFP.cu:401-423,479-504) against the zfp 0.5.5 vectors: stream bytes and
    decoded values, rates 1 to 64 bits per value."""
    n = 0
    for name, rate, maxbits, f, stream, dec in golden_cases(golden_64):
        s, o = _gpu_w64(torch_cuda, f, maxbits)
        k = min(s.size, stream.size)
        assert np.array_equal(s[:k], stream[:k]), (name, rate)
        assert not s[k:].any() and not stream[k:].any(), (name, rate)
        assert np.array_equal(o.view(np.uint64), dec.view(np.uint64)), (name, rate)
        n += 1
    assert n == 187


@pytest.mark.parametrize("dtype", ["f64", "i64"])
@pytest.mark.parametrize("shape,maxbits", [((40, 36, 132), 512), ((33, 7, 9), 1030), ((300, 260), 256), ((5000,), 72),
                                           ((64, 64, 64), 2048), ((16, 64, 64), 4096)])
def test_64_bit_fields_vs_checker(torch_cuda, dtype, shape, maxbits):
    import oracle

    rng = np.random.default_rng(sum(shape) + maxbits)
    if dtype == "f64":
        f = rng.standard_normal(shape) * 10.0 ** rng.integers(-30, 30, size=shape[:1] + (1,) * (len(shape) - 1))
    else:
        f = (rng.standard_normal(shape) * 10.0 ** rng.integers(2, 17)).astype(np.int64)
    f = np.ascontiguousarray(f)
    s, o = _gpu_w64(torch_cuda, f, maxbits)
    want = oracle.zfp_encode_64(f, maxbits)
    assert np.array_equal(s.view(np.uint64), want)
    assert np.array_equal(o.view(np.uint64), oracle.zfp_decode_64(want, f.shape, maxbits, f.dtype).view(np.uint64))


def test_64_bit_strided_and_edge_doubles(torch_cuda):
    """A sub-volume of a larger double tensor through element strides (general
    path), and blocks at the bottom of the double range where the scale overflows
    and fewer than 64 planes are coded: same bits as the checker."""
    torch = torch_cuda
    import oracle
    from cswap_amd._lib import check, lib

    L = lib()
    rng = np.random.default_rng(77)
    big = rng.standard_normal((12, 20, 30))
    sub = np.ascontiguousarray(big[1:9, 2:13, 3:22])          # 8 x 11 x 19, partial blocks, odd offsets
    t = torch.from_numpy(big).cuda()
    nz, ny, nx = sub.shape
    cap = L.cswap_zfp_stream_capacity(nx, ny, nz, 1024)
    s = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    base = t.data_ptr() + 8 * (1 * 600 + 2 * 30 + 3)
    check(L.cswap_zfp_compress_f64_nd(base, 3, nx, ny, nz, 1, 30, 600, 1024, s.data_ptr(), None), "c")
    want = oracle.zfp_encode_64(sub, 1024)
    assert np.array_equal(s.cpu().numpy().view(np.uint64), want)
    o = torch.zeros_like(t)
    check(L.cswap_zfp_decompress_f64_nd(s.data_ptr(), 3, nx, ny, nz, 1, 30, 600, 1024,
                                        o.data_ptr() + 8 * (1 * 600 + 2 * 30 + 3), None), "d")
    torch.cuda.synchronize()
    got = o.cpu().numpy()
    assert np.array_equal(got[1:9, 2:13, 3:22].view(np.uint64),
                          oracle.zfp_decode_64(want, sub.shape, 1024, np.float64).view(np.uint64))
    mask = np.ones_like(got, dtype=bool)
    mask[1:9, 2:13, 3:22] = False
    assert not got[mask].any()                                # nothing outside the sub-volume was written

    for scale in (1e-300, 1e-306, 3e-308, 5e-320, 1e300):
        f = np.ascontiguousarray(rng.standard_normal((4, 8, 8)) * scale)
        for maxbits in (512, 4096):
            sb, ob = _gpu_w64(torch, f, maxbits)
            w = oracle.zfp_encode_64(f, maxbits)
            assert np.array_equal(sb.view(np.uint64), w), (scale, maxbits)
            assert np.array_equal(ob.view(np.uint64),
                                  oracle.zfp_decode_64(w, f.shape, maxbits, np.float64).view(np.uint64)), (scale, maxbits)


def test_random_shapes_rates_types_and_strides_vs_checker(torch_cuda):
    """240 seeded cases: dimensionality 1-3, extents 1-37 (partial blocks on any
    axis), block budgets from 16 to 4096 bits that are and are not whole words, all
    four scalar types, and the field embedded with element strides in a larger
    array.  Stream words and decoded values equal the checker's; nothing outside
    the field is written."""
    torch = torch_cuda
    import oracle
    from cswap_amd._lib import check, lib

    L = lib()
    rng = np.random.default_rng(20240)
    kinds = {"f32": (np.float32, torch.float32), "i32": (np.int32, torch.int32),
             "f64": (np.float64, torch.float64), "i64": (np.int64, torch.int64)}
    for case in range(240):
        kind = ("f32", "i32", "f64", "i64")[case % 4]
        npdt, tdt = kinds[kind]
        dims = int(rng.integers(1, 4))
        shape = tuple(int(v) for v in rng.integers(1, 38, size=dims))            # (nz, ny, nx)[-dims:]
        pad = tuple(int(v) for v in rng.integers(0, 4, size=dims))               # extra elements per axis
        off = tuple(int(rng.integers(0, p + 1)) for p in pad)
        big_shape = tuple(s + p for s, p in zip(shape, pad))
        if kind[0] == "f":
            big = rng.standard_normal(big_shape) * 10.0 ** int(rng.integers(-6, 7))
            if rng.random() < 0.3:
                big[rng.random(big_shape) < 0.5] = 0.0
        else:
            big = rng.integers(-2 ** int(rng.integers(4, 30 if kind == "i32" else 61)),
                               2 ** int(rng.integers(4, 30 if kind == "i32" else 61)) + 1, size=big_shape)
        big = np.ascontiguousarray(big.astype(npdt))
        sl = tuple(slice(o, o + s) for o, s in zip(off, shape))
        sub = np.ascontiguousarray(big[sl])
        maxbits = int(rng.choice([16, 40, 64, 100, 128, 200, 256, 500, 512, 1000, 1024, 2048, 4000, 4096]))
        if kind == "f64":
            maxbits = max(maxbits, 24)                                               # room for the 12-bit header
        st = [int(v) for v in np.array(big.strides) // big.itemsize]              # element strides, slowest first
        nzyx = (1,) * (3 - dims) + shape
        sz, sy, sx = ([0] * (3 - dims) + st)
        nz, ny, nx = nzyx
        t = torch.from_numpy(big).cuda()
        base = t.data_ptr() + big.itemsize * sum(o * s for o, s in zip(off, st))
        cap = L.cswap_zfp_stream_capacity_nd(dims, nx, ny, nz, maxbits)
        s = torch.zeros(cap, dtype=torch.uint8, device="cuda")
        tag = (case, kind, shape, pad, off, maxbits)
        check(getattr(L, f"cswap_zfp_compress_{kind}_nd")(base, dims, nx, ny, nz, sx, sy, sz, maxbits,
                                                            s.data_ptr(), None), "compress")
        if kind == "f32":
            want = oracle.zfp_encode_nd(sub, maxbits)
            dec = oracle.zfp_decode_nd(want, sub.shape, maxbits)
        elif kind == "i32":
            want = oracle.zfp_encode_i32(sub, maxbits)
            dec = oracle.zfp_decode_i32(want, sub.shape, maxbits)
        else:
            want = oracle.zfp_encode_64(sub, maxbits)
            dec = oracle.zfp_decode_64(want, sub.shape, maxbits, npdt)
        got = s.cpu().numpy().view(np.uint64)
        assert np.array_equal(got, want[: got.size]), tag
        o = torch.zeros(big_shape, dtype=tdt, device="cuda")
        obase = o.data_ptr() + big.itemsize * sum(oo * ss for oo, ss in zip(off, st))
        check(getattr(L, f"cswap_zfp_decompress_{kind}_nd")(s.data_ptr(), dims, nx, ny, nz, sx, sy, sz, maxbits,
                                                              obase, None), "decompress")
        torch.cuda.synchronize()
        back = o.cpu().numpy()
        assert np.array_equal(back[sl].view(np.uint8), dec.view(np.uint8)), tag
        outside = np.ones(big_shape, dtype=bool)
        outside[sl] = False
        assert not back[outside].any(), tag


def test_full_size_tensor_equals_the_zfp_library(torch_cuda):
    """The benchmark's own 402 MB tensor (softmax(N(0,1)) [32,12,512,512], field
    512 x 512 x 384, rate 8) against the stock zfp 0.5.5 serial codec running on
    this machine's CPU: all 100,663,296 stream bytes and all decoded values."""
    torch = torch_cuda
    from cswap_amd import api

    L = _libzfp()
    if L is None:
        pytest.skip("no zfp 0.5.5 library on this machine")
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    x = torch.softmax(torch.randn((32, 12, 512, 512), generator=g, device="cuda"), dim=-1).contiguous()
    s = api.cuda_compress(x, 512)
    d = api.cuda_decompress(s, x.shape, 512)
    torch.cuda.synchronize()
    xs = x.cpu().numpy().reshape(384, 512, 512)
    nbytes = s.numel()
    assert nbytes == xs.size                                   # 8 bits per value
    buf = np.zeros(nbytes + 64, dtype=np.uint8)
    bs = L.stream_open(buf.ctypes.data, buf.size)
    zs = L.zfp_stream_open(bs)
    assert L.zfp_stream_set_rate(zs, 8.0, 3, 3, 0) == 8.0       # zfp_type_float = 3
    fld = L.zfp_field_3d(xs.ctypes.data, 3, 512, 512, 384)
    L.zfp_stream_rewind(zs)
    print("zfp library: compressing 402 MB on one core", flush=True)
    assert L.zfp_compress(zs, fld) == nbytes
    got = s.cpu().numpy()
    assert np.array_equal(got, buf[:nbytes])
    out = np.empty_like(xs)
    fo = L.zfp_field_3d(out.ctypes.data, 3, 512, 512, 384)
    L.zfp_stream_rewind(zs)
    print("zfp library: decompressing", flush=True)
    assert L.zfp_decompress(zs, fo) == nbytes
    assert np.array_equal(d.cpu().numpy().reshape(out.shape).view(np.uint32), out.view(np.uint32))
    for f in (fld, fo):
        L.zfp_field_free(f)
    L.zfp_stream_close(zs)
    L.stream_close(bs)


@pytest.mark.parametrize("kind", ["f32", "i32", "f64", "i64"])
@pytest.mark.parametrize("shape,rate", MID_SIZE_CASES)
def test_mid_size_fields_equal_the_zfp_library(torch_cuda, kind, shape, rate):
    """Fields of a few hundred thousand values of every scalar type and
    dimensionality against the stock zfp 0.5.5 library on this machine's CPU."""
    torch = torch_cuda
    from cswap_amd._lib import check, lib

    Z = _libzfp()
    if Z is None:
        pytest.skip("no zfp 0.5.5 library on this machine")
    f = mid_size_field(kind, shape, rate)
    maxbits, stream, dec = libzfp_round_trip(Z, f, rate)
    dims = f.ndim
    nz, ny, nx = (1,) * (3 - dims) + f.shape
    L = lib()
    t = torch.from_numpy(f).cuda()
    cap = L.cswap_zfp_stream_capacity_nd(dims, nx, ny, nz, maxbits)
    s = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    check(getattr(L, f"cswap_zfp_compress_{kind}_nd")(t.data_ptr(), dims, nx, ny, nz, 0, 0, 0, maxbits,
                                                        s.data_ptr(), None), "compress")
    got = s.cpu().numpy()
    k = min(stream.size, cap)
    assert np.array_equal(got[:k], stream[:k]), (kind, shape, maxbits)
    assert not got[k:].any() and not stream[k:].any()
    o = torch.zeros_like(t)
    check(getattr(L, f"cswap_zfp_decompress_{kind}_nd")(s.data_ptr(), dims, nx, ny, nz, 0, 0, 0, maxbits,
                                                          o.data_ptr(), None), "decompress")
    torch.cuda.synchronize()
    assert np.array_equal(o.cpu().numpy().view(np.uint8), dec.view(np.uint8)), (kind, shape, maxbits)


def test_pair_form_equals_the_form_with_one_lane_per_block(torch_cuda):
    """The pair form of the kernels (two wavefronts share 64 blocks) against the form with one
    lane per block, which the tests above pin to the golden vectors and the checker: the same
    stream bytes and the same decoded bits, on fields whose last workgroup is not full, at every
    rate the pair form takes (and two it must leave to the other form), on noise, smooth, sparse,
    constant and all-zero data; and against the checker itself on one field per rate."""
    torch = torch_cuda
    import ctypes as C

    import oracle
    from cswap_amd import api
    from cswap_amd._lib import lib

    L = lib()
    before = (C.c_size_t * 2)()
    L.cswap_zfp_set_pair_bytes(0, 0, before)
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    try:
        for shape in ((4, 4, 4), (4, 8, 12), (20, 36, 28), (3, 64, 32, 32), (1, 12, 260, 516), (9, 4, 512, 512)):
            for kind in ("noise", "smooth", "sparse", "const", "zero"):
                x = torch.randn(shape, generator=g, device="cuda")
                if kind == "smooth":
                    x = torch.cumsum(torch.cumsum(x, -1), -2) * 1e-3
                elif kind == "sparse":
                    x = x * (torch.rand(shape, generator=g, device="cuda") < 0.03)
                elif kind == "const":
                    x = torch.full(shape, 0.3, device="cuda")
                elif kind == "zero":
                    x = torch.zeros(shape, device="cuda")
                for maxbits in (192, 256, 512, 520, 768, 1024, 2048, 4096):
                    print("case", shape, kind, maxbits, flush=True)
                    L.cswap_zfp_set_pair_bytes(0, 0, None)
                    a = api.cuda_compress(x, maxbits)
                    da = api.cuda_decompress(a, x.shape, maxbits)
                    L.cswap_zfp_set_pair_bytes(SIZE_MAX, SIZE_MAX, None)
                    b = api.cuda_compress(x, maxbits)
                    db = api.cuda_decompress(a, x.shape, maxbits)
                    torch.cuda.synchronize()
                    assert torch.equal(a, b), (shape, kind, maxbits)
                    assert torch.equal(da.view(torch.int32), db.view(torch.int32)), (shape, kind, maxbits)
        L.cswap_zfp_set_pair_bytes(SIZE_MAX, SIZE_MAX, None)
        f = np.random.default_rng(3).standard_normal((24, 20, 36)).astype(np.float32)
        f[5:9] *= 1e-3
        for maxbits in (256, 512, 1024, 2048):
            s = gpu_encode(torch, f, maxbits)
            want = oracle.zfp_encode3(f, maxbits)
            assert np.array_equal(s.cpu().numpy().view(np.uint64), want), maxbits
            d = api.cuda_decompress(s, f.shape, maxbits)
            torch.cuda.synchronize()
            assert np.array_equal(d.cpu().numpy().view(np.uint32), oracle.zfp_decode3(want, f.shape, maxbits).view(np.uint32))
    finally:
        L.cswap_zfp_set_pair_bytes(before[0], before[1], None)
