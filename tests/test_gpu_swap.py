"""GPU tests of the swap engine (Execution::pre/post mirror + backward swap-in)
and of the reference-named entry points."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


@pytest.fixture(scope="module")
def engine(torch_cuda):
    from cswap_amd import swap

    e = swap.SwapEngine(pinned_bytes=512 << 20, device_bytes=512 << 20)
    yield e
    e.close()


def relu_tensor(torch, shape, zeros, seed):
    from cswap_amd.workloads import _ndtri

    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape, dtype=np.float32) - np.float32(_ndtri(zeros))
    return torch.from_numpy(np.maximum(x, 0).astype(np.float32)).cuda()


@pytest.mark.parametrize("policy_name", ["none", "sparse", "zfp"])
def test_round_trip_equals_codec_round_trip(torch_cuda, engine, policy_name):
    torch = torch_cuda
    import oracle
    from cswap_amd import swap

    pol = {"none": swap.NONE, "sparse": swap.SPARSE, "zfp": swap.ZFP}[policy_name]
    x = relu_tensor(torch, (16, 64, 32, 32), 0.6, 3)
    out = torch.full_like(x, -5.0)
    tk = engine.pre(x, pol)
    engine.post(tk)
    info = engine.info(tk)
    assert info.policy == pol and info.state == 2
    engine.swap_in(tk, out)
    torch.cuda.synchronize()
    engine.release(tk)
    xn = x.cpu().numpy()
    if pol == swap.ZFP:
        f = xn.reshape(-1, 32, 32)
        want = oracle.zfp_decode3(oracle.zfp_encode3(f, 512, omp=True), f.shape, 512, omp=True)
        assert np.array_equal(out.cpu().numpy().reshape(f.shape).view(np.uint32), want.view(np.uint32))
        assert info.bytes_out == xn.size
    else:
        assert torch.equal(out, x)
        if pol == swap.SPARSE:
            nnz = np.count_nonzero(xn)
            assert info.nnz == nnz
            assert info.bytes_out == 4 * nnz + xn.size // 8 + 4 * engine.process_for(xn.size)


def test_auto_policy_follows_selector(torch_cuda, engine):
    torch = torch_cuda
    from cswap_amd import swap

    cases = [(relu_tensor(torch, (32, 64, 32, 32), 0.7, 1), swap.SPARSE),
             (torch.randn((32, 64, 32, 32), device="cuda"), swap.ZFP),
             (relu_tensor(torch, (1, 4, 8, 8), 0.7, 2), swap.NONE)]
    for x, want in cases:
        tk = engine.pre(x)
        engine.post(tk)
        info = engine.info(tk)
        assert info.policy == want
        from cswap_amd.workloads import field_dims
        assert info.policy == swap.select_field(*field_dims(x.shape), info.nnz).policy
        out = torch.empty_like(x)
        engine.swap_in(tk, out)
        torch.cuda.synchronize()
        engine.release(tk)
        if want != swap.ZFP:
            assert torch.equal(out, x)
        else:
            assert float((out - x).abs().max()) < 0.5


def test_many_in_flight_and_overlap_ordering(torch_cuda, engine):
    """Several tensors out at once; compute keeps running on the compute stream
    between pre and post; results come back intact in any order."""
    torch = torch_cuda
    from cswap_amd import swap

    xs = [relu_tensor(torch, (8, 64, 32, 32), 0.5 + 0.05 * i, 10 + i) for i in range(6)]
    a = torch.randn(1024, 1024, device="cuda")
    tks = []
    for i, x in enumerate(xs):
        tks.append(engine.pre(x, [swap.SPARSE, swap.NONE, swap.AUTO][i % 3]))
        a = a @ a * 1e-3          # layer compute while the copy is in flight
    for tk in tks:
        engine.post(tk)
    keep = [x.clone() for x in xs]
    for x in xs:
        x.zero_()                 # device copies are gone
    for i in reversed(range(len(xs))):
        engine.swap_in(tks[i], xs[i])
    torch.cuda.synchronize()
    for tk in tks:
        engine.release(tk)
    for x, k in zip(xs, keep):
        assert torch.equal(x, k)


def test_copies_are_ordered_against_compute_by_events(torch_cuda, engine):
    """The outbound copy must not start before the compute stream has produced the
    tensor, and consumers on the compute stream must see the swapped-in data
    without any host synchronisation in between."""
    torch = torch_cuda
    from cswap_amd import swap

    a = torch.randn(4096, 4096, device="cuda")
    for pol in (swap.NONE, swap.SPARSE, swap.ZFP):
        x = torch.zeros(8, 64, 32, 32, device="cuda")
        b = a
        for _ in range(8):                       # tens of ms of queued compute ...
            b = (b @ a) * 1e-2
        x.fill_(7.0)                              # ... and only then the data to be swapped
        x[0, 0, 0, :8] = 0.0
        tk = engine.pre(x, pol)                   # returns while the matmuls are still running
        engine.post(tk)
        want = x.clone()
        x.fill_(-1.0)
        out = torch.empty_like(x)
        engine.swap_in(tk, out)
        total = out.sum()                         # consumer queued right behind the swap-in, no sync
        torch.cuda.synchronize()
        engine.release(tk)
        if pol == swap.ZFP:
            assert float((out - want).abs().max()) < 0.1
        else:
            assert torch.equal(out, want)
            assert float(total) == float(want.sum())


@pytest.mark.parametrize("policy_name", ["none", "sparse", "zfp", "auto"])
def test_prefetch_then_swap_in_equals_plain_swap_in(torch_cuda, engine, policy_name):
    """cswap_swap_prefetch moves the payload to device staging ahead of time; the
    swap-in that follows must give bit for bit what an on-demand swap-in gives,
    also when the prefetch is issued while the outbound copy is still in flight."""
    torch = torch_cuda
    from cswap_amd import swap

    pol = {"none": swap.NONE, "sparse": swap.SPARSE, "zfp": swap.ZFP, "auto": swap.AUTO}[policy_name]
    x = relu_tensor(torch, (8, 64, 32, 32), 0.7, 11)
    plain = torch.full_like(x, -5.0)
    tk = engine.pre(x, pol)
    engine.post(tk)
    engine.swap_in(tk, plain)
    torch.cuda.synchronize()
    engine.release(tk)

    for settle_first in (True, False):
        out = torch.full_like(x, -7.0)
        tk = engine.pre(x, pol)
        if settle_first:
            engine.post(tk)
        engine.prefetch(tk)
        assert engine.info(tk).state == 4
        engine.prefetch(tk)                      # idempotent
        busy = torch.randn(1024, 1024, device="cuda")
        for _ in range(4):                       # compute that the copy can hide under
            busy = busy @ busy * 1e-3
        engine.swap_in(tk, out)
        assert engine.info(tk).state == 3
        torch.cuda.synchronize()
        engine.release(tk)
        assert torch.equal(out.view(torch.int32), plain.view(torch.int32)), (policy_name, settle_first)


def test_prefetched_ticket_can_be_released_unused(torch_cuda, engine):
    torch = torch_cuda
    from cswap_amd import swap

    x = relu_tensor(torch, (4, 64, 32, 32), 0.5, 12)
    tk = engine.pre(x, swap.ZFP)
    engine.prefetch(tk)
    engine.release(tk)
    assert engine.info(tk).state == 0
    L = __import__("cswap_amd._lib", fromlist=["lib"]).lib()
    assert L.cswap_swap_prefetch(engine._h, tk) == -5       # released ticket
    assert L.cswap_swap_prefetch(engine._h, 10 ** 6) == -1  # no such ticket


def test_chunk_count_follows_size_rule_tuning_and_configuration(torch_cuda):
    """With process=0 the engine picks the ZVC chunk count per tensor: the size
    rule first, the measured winner once cswap_engine_tune has run for that size
    class; a configured chunk count overrides both.  Results stay bit-exact."""
    torch = torch_cuda
    from cswap_amd import swap
    from cswap_amd._lib import lib

    L = lib()
    eng = swap.SwapEngine(pinned_bytes=256 << 20, device_bytes=256 << 20)
    n = 3 * 1024 * 1024 + 17
    x = relu_tensor(torch, (n,), 0.6, 5)
    assert eng.process_for(n) == L.cswap_zvc_pick_process(n) == 2048
    best = eng.tune(n)
    assert best in (1024, 2048, 4096, 8192, 16384, 32768, 65536)
    assert eng.process_for(n) == best and eng.process_for(n // 8) == L.cswap_zvc_pick_process(n // 8)
    for e, want in ((eng, best), (swap.SwapEngine(pinned_bytes=64 << 20, device_bytes=64 << 20, process=16384), 16384)):
        out = torch.full_like(x, -1.0)
        tk = e.pre(x, swap.SPARSE)
        e.post(tk)
        info = e.info(tk)
        E = -(-n // want)
        assert info.bytes_out == 4 * int((x != 0).sum()) + 4 * want + 4 * want * (-(-E // 32))
        e.swap_in(tk, out)
        torch.cuda.synchronize()
        e.release(tk)
        assert torch.equal(out, x)
        if e is not eng:
            e.close()
    eng.close()


def test_selector_degrades_to_raw_swap_when_staging_is_full(torch_cuda):
    """A staging pool too small for either compressed form: an explicit ZFP or
    ZVC request is refused (no memory), the selector's request goes out raw and
    comes back bit-exact."""
    torch = torch_cuda
    from cswap_amd import swap
    from cswap_amd._lib import lib

    eng = swap.SwapEngine(pinned_bytes=128 << 20, device_bytes=1 << 20)
    x = torch.randn(64, 64, 2048, device="cuda")     # 32 MiB dense: the selector would take ZFP
    L = lib()
    tk = C.c_int(-1)
    for pol in (swap.ZFP, swap.SPARSE):
        assert L.cswap_swap_out(eng._h, x.data_ptr(), 64, 64, 2048, pol, None, C.byref(tk)) == -4
    t = eng.pre(x, swap.AUTO)
    eng.post(t)
    info = eng.info(t)
    assert info.policy == swap.NONE and info.bytes_out == x.numel() * 4
    out = torch.empty_like(x)
    eng.swap_in(t, out)
    torch.cuda.synchronize()
    eng.release(t)
    assert torch.equal(out, x)
    eng.close()


def test_state_machine_errors(torch_cuda, engine):
    torch = torch_cuda
    from cswap_amd._lib import lib

    x = torch.randn(4096 * 64, device="cuda")
    L = lib()
    assert L.cswap_swap_wait(engine._h, 12345) == -1
    assert L.cswap_swap_release(engine._h, 0) in (-5, 0)   # ticket 0 is free unless a test leaked it
    tk = engine.pre(x.view(64, 64, 64), 2)
    engine.post(tk)
    engine.swap_in(tk, x)
    assert L.cswap_swap_in(engine._h, tk, x.data_ptr(), None) == -5   # already in flight
    torch.cuda.synchronize()
    engine.release(tk)
    assert L.cswap_swap_release(engine._h, tk) == -5
    t2 = C.c_int(-1)
    assert L.cswap_swap_out(engine._h, x.data_ptr(), 64, 64, 64, 99, None, C.byref(t2)) == -1
    huge = C.c_int(-1)
    assert L.cswap_swap_out(engine._h, x.data_ptr(), 1 << 14, 1 << 14, 8, 2, None, C.byref(huge)) == -4


def test_calibration_gives_sane_costs(torch_cuda):
    from cswap_amd import swap

    eng = swap.SwapEngine(pinned_bytes=256 << 20, device_bytes=64 << 20)
    c = eng.calibrate()
    eng.close()
    assert 1 < c.probe_latency_us < 1000 and c.probe_gbs > 100
    assert 5 < c.bw_d2h_gbs < 200 and 5 < c.bw_h2d_gbs < 200
    assert c.zfp_compress_gbs > 50 and c.zfp_decompress_gbs > 50
    assert 3.0 < c.zfp_latency_us < 60.0          # one wavefront's serial work, measured on a 1024-block field
    assert c.zvc_compress_gbs > 50 and c.zvc_expand_gbs > 50


def test_reference_named_entry_points(torch_cuda):
    """cuda_compress / cuda_decompress with the reference's struct layout and
    device pointers (CSWAP+/simple.c:26-74 with device memory), compress /
    decompress / setRatio (CSWAP+/Execution.h:63,113) and the four ZVC launchers."""
    torch = torch_cuda
    import oracle
    from cswap_amd._lib import ZfpBitstream, ZfpField, ZfpStream, lib

    L = lib()
    rng = np.random.default_rng(5)
    f = rng.standard_normal((12, 8, 16)).astype(np.float32)
    t = torch.from_numpy(f).cuda()
    cap = L.cswap_zfp_stream_capacity(16, 8, 12, 1024)
    sbuf = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    bs = ZfpBitstream(0, 0, sbuf.data_ptr(), sbuf.data_ptr(), sbuf.data_ptr() + cap)
    zs = ZfpStream(1, 1024, 64, -1074, C.pointer(bs), 0, 0, 0)     # zfp_stream_open defaults: maxbits 1024
    fld = ZfpField(3, 16, 8, 12, 0, 0, 0, 0, 0, t.data_ptr())
    n = L.cuda_compress(C.byref(zs), C.byref(fld))
    assert n == cap == bs.ptr - bs.begin
    want = oracle.zfp_encode3(f, 1024)
    assert np.array_equal(sbuf.cpu().numpy().view(np.uint64), want)
    t.zero_()
    bs.ptr = bs.begin
    L.cuda_decompress(C.byref(zs), C.byref(fld))
    assert bs.ptr - bs.begin == cap
    assert np.array_equal(t.cpu().numpy().view(np.uint32), oracle.zfp_decode3(want, f.shape, 1024).view(np.uint32))
    # host pointers are staged like the reference does
    hs = np.zeros(cap, dtype=np.uint8)
    bs2 = ZfpBitstream(0, 0, hs.ctypes.data, hs.ctypes.data, hs.ctypes.data + cap)
    zs2 = ZfpStream(1, 1024, 64, -1074, C.pointer(bs2), 0, 0, 0)
    fh = f.copy()
    fld2 = ZfpField(3, 16, 8, 12, 0, 0, 0, 0, 0, fh.ctypes.data)
    assert L.cuda_compress(C.byref(zs2), C.byref(fld2)) == cap
    assert np.array_equal(hs.view(np.uint64), want)
    fh[:] = 0
    L.cuda_decompress(C.byref(zs2), C.byref(fld2))
    assert np.array_equal(fh.view(np.uint32), oracle.zfp_decode3(want, f.shape, 1024).view(np.uint32))
    # a 2-D field (nz = 0) goes through the 4x4-block codec (cuZFP.cu:105-151 picks by dimensionality)
    f2 = rng.standard_normal((20, 36)).astype(np.float32)
    t2 = torch.from_numpy(f2).cuda()
    cap2 = L.cswap_zfp_stream_capacity_nd(2, 36, 20, 0, 128)
    s2 = torch.zeros(cap2, dtype=torch.uint8, device="cuda")
    bs3 = ZfpBitstream(0, 0, s2.data_ptr(), s2.data_ptr(), s2.data_ptr() + cap2)
    zs3 = ZfpStream(1, 128, 64, -1074, C.pointer(bs3), 0, 0, 0)
    fld4 = ZfpField(3, 36, 20, 0, 0, 0, 0, 0, 0, t2.data_ptr())
    assert L.cuda_compress(C.byref(zs3), C.byref(fld4)) == cap2
    want2 = oracle.zfp_encode_nd(f2, 128)
    assert np.array_equal(s2.cpu().numpy().view(np.uint64), want2)
    t2.zero_()
    L.cuda_decompress(C.byref(zs3), C.byref(fld4))
    assert np.array_equal(t2.cpu().numpy().view(np.uint32), oracle.zfp_decode_nd(want2, f2.shape, 128).view(np.uint32))
    # a type value outside zfp_type -> failure value 0, nothing launched
    fld3 = ZfpField(7, 16, 8, 12, 0, 0, 0, 0, 0, t.data_ptr())
    assert L.cuda_compress(C.byref(zs), C.byref(fld3)) == 0

    # compress / decompress / setRatio on a flat activation (viewed as 32x32 rows)
    x = torch.randn(64 * 1024, device="cuda")
    L.setRatio(128)
    nbytes = C.c_size_t(0)
    buf = L.compress(x.data_ptr(), x.numel(), C.byref(nbytes))
    assert buf and nbytes.value == x.numel()
    y = torch.empty_like(x)
    assert L.decompress(buf, x.numel(), y.data_ptr()) == 0
    xf = x.cpu().numpy().reshape(-1, 32, 32)
    wantx = oracle.zfp_decode3(oracle.zfp_encode3(xf, 512), xf.shape, 512)
    assert np.array_equal(y.cpu().numpy().reshape(xf.shape).view(np.uint32), wantx.view(np.uint32))
    hip = C.CDLL("libamdhip64.so")                           # the default allocator is hipMalloc / hipFree
    hip.hipFree.argtypes = [C.c_void_p]
    assert hip.hipFree(buf) == 0

    # ZVC launchers in the reference's order
    r = torch.relu(torch.randn(16384 * 96, device="cuda"))
    nE = r.numel()
    idx = torch.zeros(16384, dtype=torch.int32, device="cuda")
    num = torch.zeros(1, dtype=torch.int32, device="cuda")
    L.PreGPUcompression(nE, 16384, r.data_ptr(), idx.data_ptr(), 512, 32, None)
    L.PreAcc(idx.data_ptr(), 16384, num.data_ptr(), 1, 1, None)
    k = int(num.item())
    vals = torch.empty(k, dtype=torch.float32, device="cuda")
    mask = torch.empty(3 * 16384, dtype=torch.int32, device="cuda")
    L.GPUcompression(nE, 16384, r.data_ptr(), vals.data_ptr(), idx.data_ptr(), mask.data_ptr(), 512, 32, None)
    dest = torch.full_like(r, 9.0)
    L.GPUdecompression(vals.data_ptr(), dest.data_ptr(), nE, 16384, mask.data_ptr(), idx.data_ptr(), 512, 32)
    torch.cuda.synchronize()
    assert torch.equal(dest, r) and k == int((r != 0).sum().item())


def test_simple_c_harness(torch_cuda):
    """What the reference's only executable check does (CSWAP+/simple.c:107-159): a
    2560x512x50 float field with values (r1 + x+y+z) / (x+y+z + r2) * (-1)^(i+j+k),
    r1 in 0..19, r2 in 0..2, x,y,z in [0,2), handed to cuda_compress as HOST memory
    with a freshly opened zfp_stream (maxbits = 1024, CSWAP+/zfp/zfp.h:23), zeroed,
    cuda_decompress-ed, and compared element by element.  simple.c draws r1, r2 from
    an unseeded rand() in an unspecified evaluation order, so the same value law is
    generated here from a seeded generator; simple.c asserts nothing, this test
    additionally requires bit-equality with the CPU checker."""
    torch = torch_cuda
    import oracle
    from cswap_amd._lib import ZfpBitstream, ZfpField, ZfpStream, lib

    L = lib()
    nx, ny, nz = 2560, 512, 50
    rng = np.random.default_rng(2024)
    i = (2.0 * np.arange(nx) / nx)[None, None, :]
    j = (2.0 * np.arange(ny) / ny)[None, :, None]
    k = (2.0 * np.arange(nz) / nz)[:, None, None]
    base = i + j + k
    r1 = rng.integers(0, 20, size=(nz, ny, nx))
    r2 = rng.integers(0, 3, size=(nz, ny, nx))
    sign = 1.0 - 2.0 * ((np.arange(nx)[None, None, :] + np.arange(ny)[None, :, None]
                         + np.arange(nz)[:, None, None]) % 2)
    with np.errstate(divide="ignore", invalid="ignore"):
        a = ((r1 + base) / (base + r2) * sign)
    a[~np.isfinite(a)] = 0.0                       # the single 0/0 at the origin when r2 == 0
    a = np.ascontiguousarray(a, dtype=np.float32)
    ori = a.copy()

    maxbits = 1024
    cap = L.cswap_zfp_stream_capacity(nx, ny, nz, maxbits)
    buf = np.zeros(cap, dtype=np.uint8)            # host buffer, as simple.c's malloc
    bs = ZfpBitstream(0, 0, buf.ctypes.data, buf.ctypes.data, buf.ctypes.data + cap)
    zs = ZfpStream(1, maxbits, 64, -1074, C.pointer(bs), 0, 0, 0)
    fld = ZfpField(3, nx, ny, nz, 0, 0, 0, 0, 0, a.ctypes.data)
    zfpsize = L.cuda_compress(C.byref(zs), C.byref(fld))
    assert zfpsize == cap == (nx // 4) * (ny // 4) * 13 * 128   # 16 bits/value over nz padded from 50 to 52
    a[:] = 0
    L.cuda_decompress(C.byref(zs), C.byref(fld))
    cnt = int(np.count_nonzero(a != ori))          # simple.c's "error cnt" (lossy: most values differ)
    rel = float(np.mean(np.abs((ori.ravel()[:1000] - a.ravel()[:1000]) / ori.ravel()[:1000])))
    print(f"simple.c harness: zfpsize {zfpsize / 2**20:.1f} MB, error cnt {cnt}, accuracy loss {rel:.3e}")
    assert rel < 0.05                               # rate 16 on a field with sign flips and 1/x spikes
    want = oracle.zfp_encode3(ori, maxbits, omp=True)
    assert np.array_equal(buf.view(np.uint64), want)
    assert np.array_equal(a.view(np.uint32), oracle.zfp_decode3(want, ori.shape, maxbits, omp=True).view(np.uint32))


def test_reference_harness_binary_runs_against_this_library(torch_cuda):
    """oracle/_ref/simple_harness is the reference's own command-line harness
    (CSWAP+/simple.c with CSWAP+/zfp/zfp.c), compiled unmodified and linked
    against libcswap_hip.so in place of the reference's CUDA library: host arrays
    of 2560 x 512 x 50 floats through zfp_stream_set_accuracy + cuda_compress +
    cuda_decompress.  The binary is built where the reference tree is present
    and travels with the tree; without it there is nothing to run."""
    import os
    import re
    import subprocess

    from conftest import ROOT

    exe = os.path.join(ROOT, "oracle", "_ref", "simple_harness")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/simple_harness was not built (no reference tree at build time)")
    out = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    print(out.stdout, out.stderr, flush=True)
    assert out.returncode == 0
    n = 2560 * 512 * 50
    assert "All tensor size =  250 MB" in out.stdout
    size_mb = float(re.search(r"zfpsize : ([0-9.]+) MB", out.stdout).group(1))
    # the harness asks for accuracy mode; the reference's CUDA path only reads maxbits from the stream
    # (cuZFP.cu:105-151), so the size is blocks x maxbits
    assert 0 < size_mb < 4.0 * n / 2**20 * 1.1
    cnt = int(re.search(r"error cnt:(\d+)", out.stdout).group(1))
    assert 0 <= cnt <= n
    loss = float(re.search(r"Final accuray loss is -> ([0-9.eE+-]+)", out.stdout).group(1))
    assert loss < 0.05


def test_random_ticket_traffic_with_small_pools(torch_cuda):
    """600 random engine operations (swap-out under every policy, wait, prefetch,
    swap-in, release, in any legal order) on pools small enough to fill up and
    fragment: a refused request (no memory) leaves the engine usable, every tensor
    that comes back is bit-identical to what its policy promises, and in the end
    both pools are whole again."""
    torch = torch_cuda
    from cswap_amd import api, swap
    from cswap_amd._lib import CswapError

    eng = swap.SwapEngine(pinned_bytes=6 << 20, device_bytes=3 << 20, max_tickets=24)
    rng = np.random.default_rng(4711)
    shapes = [(64, 64, 16), (32, 32, 64), (8, 8, 2048), (4, 4, 1000), (128, 64, 32), (2, 2, 4096), (64, 64, 128)]
    pool = []
    for i, shp in enumerate(shapes):
        x = relu_tensor(torch, shp, [0.3, 0.6, 0.9][i % 3], 100 + i)
        if i % 2:
            x = x + 0.25 * torch.randn_like(x) * (x != 0)
        s = api.cuda_compress(x, 512)
        zfp = api.cuda_decompress(s, x.shape, 512)
        pool.append((x, zfp))
    torch.cuda.synchronize()
    live = {}          # ticket -> (tensor index, state)
    refused = done = 0
    for step in range(600):
        op = rng.choice(["out", "out", "wait", "prefetch", "in", "release"])
        if op == "out" or not live:
            i = int(rng.integers(len(pool)))
            pol = int(rng.choice([swap.NONE, swap.SPARSE, swap.ZFP, swap.AUTO]))
            try:
                tk = eng.pre(pool[i][0], pol)
            except CswapError as err:
                assert err.code == -4, (step, err)
                refused += 1
                if live:                                   # make room: retire the oldest ticket
                    old = next(iter(live))
                    eng.release(old)
                    del live[old]
                continue
            assert tk not in live
            live[tk] = i
            continue
        tk = int(rng.choice(list(live)))
        i = live[tk]
        if op == "wait":
            st = eng.info(tk).state
            if st in (1, 2):
                eng.post(tk)
        elif op == "prefetch":
            if eng.info(tk).state in (1, 2, 4):
                try:
                    eng.prefetch(tk)
                except CswapError as err:
                    assert err.code == -4, (step, err)
                    refused += 1
        elif op == "in":
            if eng.info(tk).state in (1, 2, 4):
                out = torch.full_like(pool[i][0], -7.0)
                try:
                    eng.swap_in(tk, out)
                except CswapError as err:
                    assert err.code == -4, (step, err)
                    refused += 1
                    continue
                torch.cuda.synchronize()
                pol = eng.info(tk).policy
                want = pool[i][1] if pol == swap.ZFP else pool[i][0]
                assert torch.equal(out.view(torch.int32), want.view(torch.int32)), (step, tk, i, pol)
                eng.release(tk)
                del live[tk]
                done += 1
        else:
            eng.release(tk)
            del live[tk]
    for tk in list(live):
        eng.release(tk)
    assert done > 50 and refused > 0, (done, refused)
    # both pools are whole again: one allocation of (almost) the full size fits
    big = torch.zeros(64, 64, (6 << 20) // 4 // 4096 - 1, device="cuda")       # 6 MiB less 16 KiB
    tk = eng.pre(big, swap.NONE)
    eng.post(tk)
    eng.release(tk)
    eng.close()


def test_compat_allocator_field_hint_and_copy_stream(torch_cuda):
    """The knobs around the reference-named compress()/decompress(): a caller's
    allocator receives the stream buffer request (the reference allocates through
    c10, Execution.h:113-114), the field hint changes how a flat tensor is cut into
    blocks, the engine's copy stream can be handed to torch, and the last HIP error
    of a clean sequence is hipSuccess."""
    torch = torch_cuda
    import oracle
    from cswap_amd import api, swap
    from cswap_amd._lib import lib

    L = lib()
    calls = {"alloc": [], "free": []}
    keep = {}
    ALLOC = C.CFUNCTYPE(C.c_void_p, C.c_size_t)
    FREE = C.CFUNCTYPE(None, C.c_void_p)

    def my_alloc(nbytes):
        t = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        keep[t.data_ptr()] = t
        calls["alloc"].append(nbytes)
        return t.data_ptr()

    def my_free(p):
        calls["free"].append(p)
        keep.pop(p, None)

    a, f = ALLOC(my_alloc), FREE(my_free)
    x = torch.randn(64 * 64 * 32, device="cuda")
    L.setRatio(128)
    try:
        L.cswap_set_allocator(C.cast(a, C.c_void_p), C.cast(f, C.c_void_p))
        L.cswap_compat_set_field(64, 64)
        nbytes = C.c_size_t(0)
        buf = L.compress(x.data_ptr(), x.numel(), C.byref(nbytes))
        assert buf in keep and calls["alloc"] == [nbytes.value] and nbytes.value == x.numel()
        want = oracle.zfp_encode3(x.cpu().numpy().reshape(32, 64, 64), 512)
        got = keep[buf].cpu().numpy().view(np.uint64)
        assert np.array_equal(got, want)                      # blocks cut from the (64, 64, 32) field, not 32 x 32 rows
        y = torch.empty_like(x)
        assert L.decompress(buf, x.numel(), y.data_ptr()) == 0
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy().view(np.uint32),
                              oracle.zfp_decode3(want, (32, 64, 64), 512).reshape(-1).view(np.uint32))
    finally:
        L.cswap_compat_set_field(0, 0)
        L.cswap_set_allocator(None, None)
    # default layout again: 32 x 32 rows
    nbytes = C.c_size_t(0)
    buf2 = L.compress(x.data_ptr(), x.numel(), C.byref(nbytes))
    assert buf2 and calls["alloc"] == [x.numel()]             # the default allocator served this one
    s2 = api.cuda_compress(x.view(-1, 32, 32), 512)
    torch.cuda.synchronize()
    view = torch.empty(nbytes.value, dtype=torch.uint8, device="cuda")
    hip = C.CDLL("libamdhip64.so")                           # the default allocator is hipMalloc / hipFree
    assert hip.hipMemcpy(C.c_void_p(view.data_ptr()), C.c_void_p(buf2), C.c_size_t(nbytes.value), 3) == 0
    assert torch.equal(view, s2[: nbytes.value])
    assert hip.hipFree(C.c_void_p(buf2)) == 0
    assert L.cswap_last_hip_error() == 0

    eng = swap.SwapEngine(pinned_bytes=16 << 20, device_bytes=16 << 20)
    h = L.cswap_engine_copy_stream(eng._h)
    assert h
    ext = torch.cuda.ExternalStream(h)
    tk = eng.pre(x.view(64, 64, 32), swap.NONE)
    ext.synchronize()                                         # the copy went onto that stream
    assert eng.info(tk).state in (1, 2)
    eng.post(tk)
    eng.release(tk)
    eng.close()


def test_two_threads_share_one_engine(torch_cuda):
    """Engine calls are serialised by a mutex (the probe's pinned nnz slot and its
    event are shared): two host threads, each on its own compute stream, swap
    different tensors in and out through one engine and get their own data back."""
    torch = torch_cuda
    import threading

    from cswap_amd import api, swap

    eng = swap.SwapEngine(pinned_bytes=64 << 20, device_bytes=32 << 20)
    errors = []

    def worker(k):
        try:
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                xs = [relu_tensor(torch, (64, 64, 8 + 8 * j), 0.3 + 0.3 * ((j + k) % 3), 50 * k + j) for j in range(4)]
                zf = [api.cuda_decompress(api.cuda_compress(x, 512), x.shape, 512) for x in xs]
                st.synchronize()
                for it in range(60):
                    j = (it + k) % 4
                    pol = (swap.NONE, swap.SPARSE, swap.ZFP, swap.AUTO)[(it + 2 * k) % 4]
                    tk = eng.pre(xs[j], pol)
                    if it % 3 == 0:
                        eng.post(tk)
                    if it % 2:
                        eng.prefetch(tk)
                    out = torch.full_like(xs[j], -3.0)
                    eng.swap_in(tk, out)
                    st.synchronize()
                    want = zf[j] if eng.info(tk).policy == swap.ZFP else xs[j]
                    if not torch.equal(out.view(torch.int32), want.view(torch.int32)):
                        errors.append((k, it, j, pol))
                    eng.release(tk)
        except Exception as exc:  # noqa: BLE001
            errors.append((k, repr(exc)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert not errors, errors[:5]
    eng.close()


@pytest.mark.parametrize("device_pool_mib", [320, 200])
def test_large_zvc_request_takes_the_single_pass(torch_cuda, device_pool_mib):
    """An explicit ZVC request for a 256 MiB tensor is compressed in one pass over the
    tensor into a staging block of the worst-case size, cut back once the count is
    known; without room for the worst case (the 200 MiB pool) the probe path runs
    instead.  Same payload, same round trip either way."""
    torch = torch_cuda
    from cswap_amd import swap
    from cswap_amd._lib import lib

    n = 64 << 20
    g = torch.Generator(device="cuda"); g.manual_seed(21)
    x = torch.relu(torch.randn(n, generator=g, device="cuda")).reshape(64, 64, 128, 128)
    nnz = int((x != 0).sum().item())
    eng = swap.SwapEngine(pinned_bytes=256 << 20, device_bytes=device_pool_mib << 20)
    try:
        process = eng.process_for(n)
        assert lib().cswap_zvc_takes_single_pass(n, process) == 1
        for rep in range(2):
            print("pool", device_pool_mib, "rep", rep, flush=True)
            tk = eng.pre(x, swap.SPARSE)
            eng.post(tk)
            info = eng.info(tk)
            assert info.policy == swap.SPARSE and info.nnz == nnz
            assert info.bytes_out == 4 * nnz + n // 8 + 4 * process
            out = torch.full_like(x, -1.0)
            eng.swap_in(tk, out)
            torch.cuda.synchronize()
            eng.release(tk)
            assert torch.equal(out, x)
    finally:
        eng.close()


def test_engine_falls_back_when_the_single_pass_gives_up(torch_cuda):
    """The single pass reports a wait that ran out through a negative count (forced here
    from the host, as in test_gpu_zvc.py: every kernel still exits normally); the
    engine then compresses the tensor with the probe path and the swap is as good."""
    torch = torch_cuda
    from cswap_amd import swap
    from cswap_amd._lib import lib

    L = lib()
    n = 48 << 20                                       # 192 MiB
    g = torch.Generator(device="cuda"); g.manual_seed(22)
    x = torch.relu(torch.randn(n, generator=g, device="cuda")).reshape(48, 64, 128, 128)
    nnz = int((x != 0).sum().item())
    eng = swap.SwapEngine(pinned_bytes=256 << 20, device_bytes=320 << 20)
    try:
        assert L.cswap_zvc_takes_single_pass(n, eng.process_for(n)) == 1
        L.cswap_zvc_debug_set_lookback(4, 1)
        try:
            print("forced give-up inside the engine", flush=True)
            tk = eng.pre(x, swap.SPARSE)
        finally:
            L.cswap_zvc_debug_set_lookback(0, 0)
        eng.post(tk)
        info = eng.info(tk)
        assert info.policy == swap.SPARSE and info.nnz == nnz
        out = torch.full_like(x, -1.0)
        eng.swap_in(tk, out)
        torch.cuda.synchronize()
        eng.release(tk)
        assert torch.equal(out, x)
    finally:
        eng.close()


@pytest.mark.parametrize("policy_name", ["sparse", "zfp"])
def test_swap_in_while_the_outbound_copy_is_in_flight_reads_the_staging_block(torch_cuda, policy_name):
    """A compressed tensor that is asked back before its outbound copy has finished is
    decompressed straight from its staging block (no wait for the copy, nothing on the
    link); the result is what a swap through the host gives, the ticket can be released
    at once, and the pools are whole again afterwards."""
    torch = torch_cuda
    from cswap_amd import swap

    pol = {"sparse": swap.SPARSE, "zfp": swap.ZFP}[policy_name]
    eng = swap.SwapEngine(pinned_bytes=64 << 20, device_bytes=24 << 20)
    try:
        x = relu_tensor(torch, (16, 64, 32, 32), 0.6, 21)               # 4 MiB
        plain = torch.full_like(x, -5.0)
        tk = eng.pre(x, pol); eng.post(tk); eng.swap_in(tk, plain)
        torch.cuda.synchronize(); eng.release(tk)
        for rep in range(6):
            outs = []
            for k in range(3):                                           # several in flight at once
                tk = eng.pre(x, pol)
                out = torch.full_like(x, -7.0)
                if k == 1:
                    eng.prefetch(tk)                                     # found on the device: stays there
                    assert eng.info(tk).state == 4
                eng.swap_in(tk, out)
                assert eng.info(tk).state == 3
                if k == 2:
                    eng.post(tk)                                         # a late wait for the outbound copy is still answered
                eng.release(tk)                                          # at once; memory comes back when the work is done
                assert eng.info(tk).state == 0
                outs.append(out)
            torch.cuda.synchronize()
            for out in outs:
                assert torch.equal(out.view(torch.int32), plain.view(torch.int32)), (policy_name, rep)
        big = torch.zeros(64, 64, (24 << 20) // 4 // 4096 - 8, device="cuda")
        tk = eng.pre(big, swap.ZFP)                                      # a quarter of the staging pool; and the host pool
        eng.post(tk); eng.release(tk)
        tk = eng.pre(torch.zeros(64, 64, (60 << 20) // 4 // 4096, device="cuda"), swap.NONE)   # 60 of 64 MiB pinned
        eng.post(tk); eng.release(tk)
    finally:
        eng.close()


def test_a_full_staging_pool_makes_requests_wait_not_fail(torch_cuda):
    """Swap-outs issued back to back, without waiting for any copy, into a staging pool
    that holds two payloads: each request that finds the pool full waits for the oldest
    copy in flight instead of failing or going out raw, and everything comes back intact."""
    torch = torch_cuda
    from cswap_amd import api, swap

    x = relu_tensor(torch, (32, 64, 32, 32), 0.5, 22)                    # 8 MiB, 2 MiB at 8 bits per value
    eng = swap.SwapEngine(pinned_bytes=64 << 20, device_bytes=(4 << 20) + (256 << 10))
    try:
        want = api.cuda_decompress(api.cuda_compress(x, 512), x.shape, 512)
        tks = [eng.pre(x, swap.ZFP if k % 2 else swap.AUTO) for k in range(8)]
        for tk in tks:
            info = eng.info(tk)
            assert info.policy in (swap.ZFP, swap.SPARSE), info.policy   # none degraded to a raw swap
        for tk in tks:
            out = torch.full_like(x, -1.0)
            eng.swap_in(tk, out)
            torch.cuda.synchronize()
            exact = eng.info(tk).policy == swap.SPARSE
            assert torch.equal(out.view(torch.int32), (x if exact else want).view(torch.int32))
            eng.release(tk)
    finally:
        eng.close()


def test_selector_with_the_compaction_as_its_probe(torch_cuda):
    """CSWAP_POLICY_AUTO_SPARSE: the selector for a tensor its caller expects to be sparse.  The
    single-kernel compaction runs first and yields the count; a sparse tensor ends up as ZVC with
    one host round trip and the payload the three kernels make; a dense one is handed on to the
    selector's choice (ZFP here) and still comes back as that codec would give it; plain AUTO on a
    tensor small enough for the one-kernel form takes the same route.  Sizes on both sides of the
    pipeline kernel's threshold."""
    torch = torch_cuda
    import oracle
    from cswap_amd import swap
    from cswap_amd._lib import lib

    eng = swap.SwapEngine(pinned_bytes=384 << 20, device_bytes=640 << 20)
    try:
        for shape, zeros in (((32, 64, 32, 32), 0.7), ((64, 64, 64, 64), 0.6), ((128, 64, 64, 64), 0.5)):
            x = relu_tensor(torch, shape, zeros, 31)
            n = x.numel()
            nnz = int((x != 0).sum().item())
            form = lib().cswap_zvc_takes_single_pass(n, eng.process_for(n))
            assert form in (1, 2)
            for pol in (swap.AUTO_SPARSE, swap.AUTO, swap.SPARSE):
                print("sparse", shape, pol, "form", form, flush=True)
                before = eng.probe_count()
                tk = eng.pre(x, pol)
                assert eng.probe_count() == before + 1          # one host round trip, whichever way
                info = eng.info(tk)
                assert info.policy == swap.SPARSE and info.nnz == nnz
                assert info.bytes_out == 4 * nnz + n // 8 + 4 * eng.process_for(n)
                out = torch.full_like(x, -1.0)
                eng.swap_in(tk, out)
                torch.cuda.synchronize()
                eng.release(tk)
                assert torch.equal(out, x)
        g = torch.Generator(device="cuda"); g.manual_seed(5)
        for shape in ((32, 64, 32, 32), (128, 64, 64, 64)):
            x = torch.randn(shape, generator=g, device="cuda")
            for pol in (swap.AUTO_SPARSE, swap.AUTO):
                print("dense", shape, pol, flush=True)
                tk = eng.pre(x, pol)
                info = eng.info(tk)
                assert info.policy == swap.ZFP and info.nnz == int((x != 0).sum().item())
                out = torch.full_like(x, -1.0)
                eng.swap_in(tk, out)
                torch.cuda.synchronize()
                eng.release(tk)
                f = x.cpu().numpy().reshape(-1, shape[-2], shape[-1])
                want = oracle.zfp_decode3(oracle.zfp_encode3(f, 512, omp=True), f.shape, 512, omp=True)
                assert np.array_equal(out.cpu().numpy().reshape(f.shape).view(np.uint32), want.view(np.uint32))
    finally:
        eng.close()


@pytest.mark.parametrize("policy_name", ["none", "sparse", "zfp", "auto"])
def test_phase_times_of_a_ticket_come_from_the_engine(torch_cuda, policy_name):
    """An engine created with timing brackets every phase of a ticket with events on the stream
    it runs on (the reference's profiler slots, Execution.h:109-126,285-295): after a swap-out,
    a wait, a swap-in and a synchronize the four figures are there, the copies take the time
    the link needs for the payload, and together they fit inside the wall clock around the
    calls.  Before a phase has finished its figure is -1; an engine without timing refuses."""
    torch = torch_cuda
    import time

    from cswap_amd import swap
    from cswap_amd._lib import CswapError

    pol = {"none": swap.NONE, "sparse": swap.SPARSE, "zfp": swap.ZFP, "auto": swap.AUTO}[policy_name]
    x = relu_tensor(torch, (64, 64, 64, 64), 0.6, 9)          # 64 MiB
    out = torch.empty_like(x)
    eng = swap.SwapEngine(pinned_bytes=256 << 20, device_bytes=256 << 20, timing=True)
    try:
        for rep in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            tk = eng.pre(x, pol)
            first = eng.timing(tk)
            eng.post(tk)
            mid = eng.timing(tk)
            eng.swap_in(tk, out)
            torch.cuda.synchronize()
            wall_us = (time.perf_counter() - t0) * 1e6
            t = eng.timing(tk)
            info = eng.info(tk)
            eng.release(tk)
            print(policy_name, rep, "compress %.1f copy out %.1f copy in %.1f decompress %.1f us; wall %.1f us; %d bytes"
                  % (t.compress_us, t.copy_out_us, t.copy_in_us, t.decompress_us, wall_us, info.bytes_out), flush=True)
            assert first.copy_in_us == -1 and first.decompress_us == -1
            assert mid.compress_us >= 0 and mid.copy_out_us > 0 and mid.copy_in_us == -1
            assert t.compress_us == mid.compress_us and t.copy_out_us == mid.copy_out_us
            assert t.copy_in_us > 0 and t.decompress_us >= 0
            if info.policy != swap.NONE:
                assert t.compress_us > 1 and t.decompress_us > 1
            # a link of 20 to 100 GB/s
            for c in (t.copy_out_us, t.copy_in_us):
                assert info.bytes_out / 100e3 <= c <= info.bytes_out / 20e3 + 50, (c, info.bytes_out)
            assert t.compress_us + t.copy_out_us + t.copy_in_us + t.decompress_us <= wall_us
        assert torch.equal(out, x) or pol in (swap.ZFP,)
    finally:
        eng.close()
    plain = swap.SwapEngine(pinned_bytes=64 << 20, device_bytes=64 << 20)
    try:
        tk = plain.pre(x[:4], swap.NONE)
        with pytest.raises(CswapError):
            plain.timing(tk)
        plain.post(tk)
        plain.release(tk)
    finally:
        plain.close()


def test_pipeline_kernel_of_the_compaction_runs_beside_payload_copies(torch_cuda):
    """The pipeline form of the single-pass compaction needs every one of its workgroups
    resident at once, and on this GPU the engine's transfers are themselves kernels on the copy
    streams.  A 256 MiB raw swap-out keeps the outbound copy stream busy for milliseconds; an
    explicit ZVC request for a 192 MiB tensor issued right behind it must still finish its
    single pass (a count of -1 would send the engine to the three kernels, which would show as
    a second probe) with the payload the three kernels make, and in about the time it takes
    alone."""
    torch = torch_cuda
    import time

    from cswap_amd import swap
    from cswap_amd._lib import lib

    g = torch.Generator(device="cuda"); g.manual_seed(77)
    big = torch.randn(64 << 20, generator=g, device="cuda").reshape(64, 64, 128, 128)        # 256 MiB, goes out raw
    n = 48 << 20
    x = torch.relu(torch.randn(n, generator=g, device="cuda")).reshape(48, 64, 128, 128)     # 192 MiB
    nnz = int((x != 0).sum().item())
    eng = swap.SwapEngine(pinned_bytes=640 << 20, device_bytes=320 << 20, timing=True)
    try:
        assert lib().cswap_zvc_takes_single_pass(n, eng.process_for(n)) == 1
        alone = []
        for _ in range(3):
            tk = eng.pre(x, swap.SPARSE)
            eng.post(tk)
            alone.append(eng.timing(tk).compress_us)
            eng.release(tk)
        beside = []
        for rep in range(3):
            print("rep", rep, flush=True)
            torch.cuda.synchronize()
            tb = eng.pre(big, swap.NONE)                     # its copy is now running on the copy stream
            before = eng.probe_count()
            tk = eng.pre(x, swap.SPARSE)
            assert eng.probe_count() == before + 1, "the single pass gave up and the three kernels ran"
            info = eng.info(tk)
            assert info.policy == swap.SPARSE and info.nnz == nnz
            out = torch.full_like(x, -1.0)
            eng.swap_in(tk, out)                             # from its staging block: its own copy waits behind the big one
            torch.cuda.synchronize()
            assert torch.equal(out, x)
            eng.post(tb)
            eng.post(tk)
            beside.append(eng.timing(tk).compress_us)
            eng.release(tk)
            eng.release(tb)
        print("single pass + count round trip, 192 MiB: alone %s us, beside a 256 MiB copy %s us"
              % (["%.0f" % v for v in alone], ["%.0f" % v for v in beside]), flush=True)
        assert min(beside) < 3 * min(alone) + 200
    finally:
        eng.close()
