"""Fields and tensors at the top of what the entry points accept: more than 2^32
elements (ZFP), 2^31 - 1 elements (ZVC, whose sizes are ints as in
CSWAP+/zfp/compression.cuh:5-8), more than 4 GiB through the swap engine.  The
CPU checker cannot code tens of gigabytes, but ZFP blocks are coded one by one
and ZVC chunks likewise, so slabs cut where an element index, a byte offset or
a stream offset passes 2^30, 2^31 and 2^32 are compared with the checker run
on that slab alone."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

NX = NY = 1024
NZ = 4100                                    # 4100 * 2^20 elements: 2^32 is passed at z = 4096
CUTS = (0, 1020, 2044, 3068, 4092)           # slabs of eight planes from these z


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


def _free(torch):
    import gc

    gc.collect()
    torch.cuda.empty_cache()


def _pieces_agree(torch, x, s, d, maxbits, planes, layer):
    """Every block of the large field: runs of ``planes`` planes (a multiple of
    four, small enough that no offset inside one passes 2^32 elements) coded as
    fields of their own give the same stream bytes and the same values."""
    from cswap_amd import api

    for z0 in range(0, x.shape[0], planes):
        piece = x[z0:z0 + planes]
        sp = api.cuda_compress(piece, maxbits)
        dp = api.cuda_decompress(sp, piece.shape, maxbits, dtype=x.dtype)
        torch.cuda.synchronize()
        nbytes = (piece.shape[0] // 4) * layer
        assert torch.equal(sp[:nbytes], s[(z0 // 4) * layer:(z0 // 4) * layer + nbytes]), z0
        assert torch.equal(dp.view(torch.uint8), d[z0:z0 + planes].view(torch.uint8)), z0
        del sp, dp


def test_zfp_f32_field_beyond_2_32_elements(torch_cuda):
    torch = torch_cuda
    import oracle
    from cswap_amd import api

    g = torch.Generator(device="cuda"); g.manual_seed(3)
    x = torch.randn((NZ, NY, NX), generator=g, device="cuda")
    x[2046:2050].mul_(1e-30)                 # planes of tiny values and a layer of zeros in checked slabs
    x[4096:4100].zero_()
    print("encode", x.numel(), flush=True)
    s = api.cuda_compress(x, 512)
    torch.cuda.synchronize()
    assert s.numel() >= x.numel()            # rate 8: one stream byte per value
    print("decode", flush=True)
    d = api.cuda_decompress(s, x.shape, 512)
    torch.cuda.synchronize()
    layer = (NX // 4) * (NY // 4) * 64       # stream bytes of one layer of blocks (four planes)
    for z in CUTS:
        print("slab", z, flush=True)
        slab = x[z:z + 8].cpu().numpy()
        got = s[(z // 4) * layer:(z // 4 + 2) * layer].cpu().numpy().view(np.uint64)
        want = oracle.zfp_encode3(slab, 512, omp=True)
        assert np.array_equal(got, want[:got.size]), z
        back = d[z:z + 8].cpu().numpy()
        assert np.array_equal(back.view(np.uint32), oracle.zfp_decode3(got, slab.shape, 512, omp=True).view(np.uint32)), z
    assert not d[4096:4100].view(torch.int32).any().item()     # a layer of empty blocks decodes to +0.0
    _pieces_agree(torch, x, s, d, 512, 820, layer)
    del x, s, d
    _free(torch)


def test_zfp_f32_general_path_beyond_2_32_elements(torch_cuda):
    """The same extents seen through a base pointer that is only 4-byte aligned
    and rows of 1023 values in a pitch of 1024: the per-element path with its
    64-bit element offsets, partial blocks along x."""
    torch = torch_cuda
    import oracle
    from cswap_amd._lib import check, lib

    L = lib()
    g = torch.Generator(device="cuda"); g.manual_seed(4)
    x = torch.randn((NZ, NY, NX), generator=g, device="cuda")
    nx = NX - 1
    cap = L.cswap_zfp_stream_capacity(nx, NY, NZ, 512)
    s = torch.empty(cap, dtype=torch.uint8, device="cuda")
    print("encode", flush=True)
    check(L.cswap_zfp_compress_f32(x.data_ptr() + 4, nx, NY, NZ, 1, NX, NX * NY, 512, s.data_ptr(), None), "enc")
    torch.cuda.synchronize()
    out = torch.full((NZ, NY, NX), -7.0, device="cuda")
    print("decode", flush=True)
    check(L.cswap_zfp_decompress_f32(s.data_ptr(), nx, NY, NZ, 1, NX, NX * NY, 512, out.data_ptr() + 4, None), "dec")
    torch.cuda.synchronize()
    layer = ((nx + 3) // 4) * (NY // 4) * 64
    flat_x, flat_o = x.view(-1), out.view(-1)
    for z in CUTS:
        print("slab", z, flush=True)
        lo, hi = z * NX * NY + 1, (z + 8) * NX * NY + 1
        if hi > flat_x.numel():              # the last row of the last slab ends with the allocation
            hi = flat_x.numel()
        raw = torch.zeros(8 * NX * NY, device="cuda")
        raw[:hi - lo] = flat_x[lo:hi]
        slab = np.ascontiguousarray(raw.view(8, NY, NX)[:, :, :nx].cpu().numpy())
        got = s[(z // 4) * layer:(z // 4 + 2) * layer].cpu().numpy().view(np.uint64)
        want = oracle.zfp_encode3(slab, 512, omp=True)
        assert np.array_equal(got, want[:got.size]), z
        rawo = torch.zeros(8 * NX * NY, device="cuda")
        rawo[:hi - lo] = flat_o[lo:hi]
        back = np.ascontiguousarray(rawo.view(8, NY, NX)[:, :, :nx].cpu().numpy())
        assert np.array_equal(back.view(np.uint32), oracle.zfp_decode3(got, slab.shape, 512, omp=True).view(np.uint32)), z
    # the pitch column and the first element were never written
    assert flat_o[0].item() == -7.0
    assert bool((out.view(-1)[1:].view(-1)[NX - 1::NX] == -7.0).all().item())
    del x, s, out, flat_x, flat_o
    _free(torch)


def test_zfp_f64_field_beyond_2_32_elements(torch_cuda):
    torch = torch_cuda
    import oracle
    from cswap_amd import api

    g = torch.Generator(device="cuda"); g.manual_seed(5)
    x = torch.empty((NZ, NY, NX), dtype=torch.float64, device="cuda")
    for z0 in range(0, NZ, 410):             # filled in pieces: randn of doubles makes a temporary as large as its result
        x[z0:z0 + 410] = torch.randn((410, NY, NX), generator=g, device="cuda", dtype=torch.float64)
    maxbits = 1024                           # 16 bits per value
    print("encode", x.numel(), flush=True)
    s = api.cuda_compress(x, maxbits)
    torch.cuda.synchronize()
    print("decode", flush=True)
    d = api.cuda_decompress(s, x.shape, maxbits, dtype=torch.float64)
    torch.cuda.synchronize()
    layer = (NX // 4) * (NY // 4) * (maxbits // 8)
    for z in (2044, 4092):                   # byte offsets of the field pass 2^34 and 2^35, of the stream 2^32 and 2^33
        print("slab", z, flush=True)
        slab = x[z:z + 8].cpu().numpy()
        got = s[(z // 4) * layer:(z // 4 + 2) * layer].cpu().numpy().view(np.uint64)
        want = oracle.zfp_encode_64(slab, maxbits)
        assert np.array_equal(got, want[:got.size]), z
        back = d[z:z + 8].cpu().numpy()
        assert np.array_equal(back.view(np.uint64), oracle.zfp_decode_64(got, slab.shape, maxbits, np.float64).view(np.uint64)), z
    _pieces_agree(torch, x, s, d, maxbits, 400, layer)
    del x, s, d
    _free(torch)


def test_zfp_i32_field_loaded_with_the_nontemporal_hint(torch_cuda):
    """An int32 field of 160 MiB: above the size from which the encoder loads its
    rows with the nontemporal hint (a separate instantiation per element kind).
    First, middle and last slab against the checker, every block against pieces."""
    torch = torch_cuda
    import oracle
    from cswap_amd import api

    nz, ny, nx = 640, 256, 256
    g = torch.Generator(device="cuda"); g.manual_seed(8)
    x = torch.randint(-(1 << 28), 1 << 28, (nz, ny, nx), generator=g, device="cuda", dtype=torch.int32)
    x[300:304].zero_()
    s = api.cuda_compress(x, 512)
    d = api.cuda_decompress(s, x.shape, 512, dtype=torch.int32)
    torch.cuda.synchronize()
    layer = (nx // 4) * (ny // 4) * 64
    for z in (0, 296, 632):
        slab = x[z:z + 8].cpu().numpy()
        got = s[(z // 4) * layer:(z // 4 + 2) * layer].cpu().numpy().view(np.uint64)
        want = oracle.zfp_encode_i32(slab, 512)
        assert np.array_equal(got, want[:got.size]), z
        back = d[z:z + 8].cpu().numpy()
        assert np.array_equal(back, oracle.zfp_decode_i32(got, slab.shape, 512)), z
    assert not d[300:304].any().item()
    _pieces_agree(torch, x, s, d, 512, 128, layer)       # pieces of 32 MiB: plain loads
    del x, s, d
    _free(torch)


def test_zfp_rejects_fields_beyond_its_block_index_range(torch_cuda):
    """2^31 blocks or more, or an extent above 2^31 - 1, are refused before any launch."""
    torch = torch_cuda
    from cswap_amd._lib import lib

    L = lib()
    t = torch.zeros(64, device="cuda")
    s = torch.zeros(64, dtype=torch.uint8, device="cuda")
    assert L.cswap_zfp_compress_f32(t.data_ptr(), 1 << 14, 1 << 14, 1 << 10, 0, 0, 0, 512, s.data_ptr(), None) < 0   # 2^32 blocks
    assert L.cswap_zfp_compress_f32(t.data_ptr(), 1 << 32, 4, 4, 0, 0, 0, 512, s.data_ptr(), None) < 0
    assert L.cswap_zfp_decompress_f32(s.data_ptr(), 1 << 14, 1 << 14, 1 << 10, 0, 0, 0, 512, t.data_ptr(), None) < 0
    torch.cuda.synchronize()
    assert not t.any().item() and not s.any().item()


@pytest.mark.parametrize("process", [512 * 32, 1 << 20])
def test_zvc_at_int_max_elements(torch_cuda, process):
    """n = 2^31 - 1 (odd, so the last chunk is ragged and the tensor's end is not
    16-byte aligned); 16384 chunks of 131072 elements take the three-kernel path,
    2^20 chunks of 2048 the layout the engine picks for large tensors."""
    torch = torch_cuda
    import oracle
    from cswap_amd import api

    n = (1 << 31) - 1
    g = torch.Generator(device="cuda"); g.manual_seed(6)
    t = torch.empty(n, device="cuda")
    step = 1 << 28
    for a in range(0, n, step):              # relu(randn) in pieces
        b = min(n, a + step)
        t[a:b] = torch.relu(torch.randn(b - a, generator=g, device="cuda"))
    t[-1] = 2.5
    print("compress", n, process, flush=True)
    values, mask, begin, nnz = api.zvc_compress(t, process)
    torch.cuda.synchronize()
    k = int(nnz.item())
    assert k == int(api.probe_nnz(t).item()) == sum(int((t[a:a + step] != 0).sum().item()) for a in range(0, n, step))
    E, W, K = oracle.zvc_geometry(n, process)
    b = begin.cpu().numpy().astype(np.int64)
    assert b[0] == 0 and np.all(np.diff(b[:K]) >= 0) and b[K - 1] <= k
    # chunks at the start, either side of element 2^30, and the ragged last one, against the checker
    for c in (0, (1 << 30) // E - 1, (1 << 30) // E, K - 2, K - 1):
        print("chunk", c, flush=True)
        lo, hi = c * E, min(n, (c + 1) * E)
        chunk = t[lo:hi].cpu().numpy()
        cnt = int(np.count_nonzero(chunk))
        nxt = int(b[c + 1]) if c + 1 < K else k
        assert nxt - int(b[c]) == cnt, c
        got_v = values[int(b[c]):int(b[c]) + cnt].cpu().numpy()
        assert np.array_equal(got_v.view(np.uint32), chunk[chunk != 0].view(np.uint32)), c
        got_m = mask[c * W:(c + 1) * W].cpu().numpy().view(np.uint8)
        want_m = np.packbits(chunk != 0, bitorder="little")
        assert np.array_equal(got_m[:want_m.size], want_m) and not got_m[want_m.size:].any(), c
    print("expand", flush=True)
    out = torch.full_like(t, 3.0)
    api.GPUdecompression(values, out, mask, begin, process)
    torch.cuda.synchronize()
    for a in range(0, n, step):
        assert torch.equal(out[a:a + step], t[a:a + step]), a
    del t, values, mask, begin, out
    _free(torch)


def test_swap_engine_tensor_beyond_4_gib(torch_cuda):
    """One 4.5 GiB tensor through the engine raw, as ZVC and as ZFP: pool offsets,
    copy sizes and ticket sizes above 2^32 bytes."""
    torch = torch_cuda
    from cswap_amd import api, swap

    shape = (1152, 1024, 1024)
    g = torch.Generator(device="cuda"); g.manual_seed(7)
    t = torch.relu(torch.randn(shape, generator=g, device="cuda"))
    eng = swap.SwapEngine(pinned_bytes=6 << 30, device_bytes=5 << 30)
    zfp_want = api.cuda_decompress(api.cuda_compress(t, 512), shape, 512)
    for policy, name in ((swap.NONE, "raw"), (swap.SPARSE, "zvc"), (swap.ZFP, "zfp")):
        print("policy", name, flush=True)
        ticket = eng.pre(t, policy)
        eng.post(ticket)
        info = eng.info(ticket)
        assert info.policy == policy
        if policy == swap.NONE:
            assert info.bytes_out == t.numel() * 4
        back = torch.full(shape, -1.0, device="cuda")
        eng.swap_in(ticket, back)
        torch.cuda.synchronize()
        eng.release(ticket)
        assert torch.equal(back, zfp_want if policy == swap.ZFP else t), name
        del back
    eng.close()
    del t, zfp_want
    _free(torch)
