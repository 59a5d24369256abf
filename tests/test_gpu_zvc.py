"""GPU parity of zero-value compaction: bit-exact mask, packed values, chunk
offsets and reconstruction against the CPU checker and numpy."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
P = 512 * 32


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


@pytest.fixture(scope="module", autouse=True)
def single_pass_at_any_size():
    """cswap_zvc_compress_fused runs its single pass only from 64 MiB on (the three
    kernels finish sooner below); the tests here want it on small shapes too."""
    from cswap_amd._lib import lib

    before = lib().cswap_zvc_set_single_pass_bytes(0)
    yield
    lib().cswap_zvc_set_single_pass_bytes(before)


@pytest.fixture(params=["pipeline", "small"])
def fused_form(request):
    """The two single-kernel forms behind cswap_zvc_compress_fused: the pipeline kernel, forced
    on at any size (what the module-wide fixture sets), and the one-kernel form that the size
    rule picks for tensors of up to 32 MiB (the pipeline kernel takes over at 64 MiB)."""
    from cswap_amd._lib import lib

    before = lib().cswap_zvc_set_single_pass_bytes(0 if request.param == "pipeline" else 64 << 20)
    yield request.param
    lib().cswap_zvc_set_single_pass_bytes(before)


def test_size_rule_of_the_single_pass():
    from cswap_amd._lib import lib

    L = lib()
    assert L.cswap_zvc_takes_single_pass(P * 64, P) == 1          # forced on for this module
    forced = L.cswap_zvc_set_single_pass_bytes(64 << 20)
    assert forced == 0
    mine = forced
    try:
        assert L.cswap_zvc_takes_single_pass(P * 512, P) == 2      # 32 MiB: the one-kernel form for small tensors
        assert L.cswap_zvc_takes_single_pass(P * 512 + 32 * P, P) == 0   # 34 MiB: too large for it, three kernels
        assert L.cswap_zvc_takes_single_pass(P * 64 + 5, P) == 0   # chunk length 65: three kernels
        assert L.cswap_zvc_takes_single_pass(P * 1024, P) == 1     # 64 MiB: the pipeline kernel
        assert L.cswap_zvc_takes_single_pass(P * 4096 + 5, P) == 0  # chunk length 4097: not whole half rows
        assert L.cswap_zvc_takes_single_pass(1 << 30, 1024) == 0   # more tiles than the workspace has words for
    finally:
        L.cswap_zvc_set_single_pass_bytes(mine)


@pytest.fixture(params=["by_size", "staged"])
def compact_form(request):
    """Both forms of cswap_zvc_compact and of the 16-byte-store expansion: the one the
    size rule picks (no LDS staging at these sizes) and the LDS-staged one, forced for
    inputs of any size."""
    from cswap_amd._lib import lib

    if request.param == "by_size":
        yield request.param
        return
    before = lib().cswap_zvc_set_staged_compact_bytes(0)
    try:
        yield request.param
    finally:
        lib().cswap_zvc_set_staged_compact_bytes(before)


def run_gpu(torch, x, process=P, fused=False):
    from cswap_amd import api

    t = torch.from_numpy(x).cuda()
    values, mask, begin, nnz = api.zvc_compress(t, process, fused=fused)
    out = torch.full_like(t, -1.0)                      # NOT pre-zeroed on purpose
    api.GPUdecompression(values, out, mask, begin, process)
    probe = api.probe_nnz(t)
    torch.cuda.synchronize()
    k = int(nnz.item())
    return (values[:k].cpu().numpy(), mask.cpu().numpy().view(np.uint32), begin.cpu().numpy(), k,
            out.cpu().numpy(), int(probe.item()))


def check_against_oracle(x, got, process=P):
    import oracle

    vals, mask, begin, nnz = oracle.zvc_compress(x, process)
    gv, gm, gb, gk, gout, gprobe = got
    assert gk == nnz == gprobe == np.count_nonzero(x)
    assert np.array_equal(gv.view(np.uint32), vals.view(np.uint32))
    assert np.array_equal(gm, mask)
    E, W, K = oracle.zvc_geometry(x.size, process)
    assert np.array_equal(gb[:K], begin[:K])
    want = np.where(x != 0, x, np.float32(0))
    assert np.array_equal(gout.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("pct", [30, 50, 70, 90])
def test_config2_sparsity_sweep(torch_cuda, compact_form, pct):
    from cswap_amd.workloads import config2_tensor

    x = config2_tensor(pct).reshape(-1)
    got = run_gpu(torch_cuda, x)
    check_against_oracle(x, got)
    assert np.array_equal(got[1].view(np.uint8), np.packbits(x != 0, bitorder="little"))


@pytest.mark.parametrize("n", [1, 31, 33, 64, 1000, P - 1, P, P + 1, 1_000_003, P * 62 + 17, P * 64, P * 96 + 5])
def test_ragged_sizes(torch_cuda, compact_form, n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * (rng.random(n) < 0.4)).astype(np.float32)
    print("n", n, flush=True)
    check_against_oracle(x, run_gpu(torch_cuda, x))


@pytest.mark.parametrize("process", [1, 7, 64, 4096])
def test_other_chunk_counts(torch_cuda, compact_form, process):
    rng = np.random.default_rng(process)
    x = np.maximum(rng.standard_normal(300_001), 0).astype(np.float32)
    check_against_oracle(x, run_gpu(torch_cuda, x, process), process)


@pytest.mark.parametrize("n,process", [(P * 8 - 3, P), (P * 260 - 1, P), (P * 512 - 2, P), (P * 2052 - 7, P),
                                        (P * 4096 - 254, P), (28, 7), (5000, 1), (299_992, 7), (64 * 2048, 64)])
def test_expand_four_per_lane(torch_cuda, compact_form, n, process):
    """Chunk lengths that are multiples of four take the 16-byte-store expansion
    (both of its forms: values fetched straight from global memory, and staged in
    LDS as for tensors beyond the cache size, which `compact_form` forces);
    the sizes end the last chunk inside a quad, inside a row and inside a refill
    group.  The same data is then expanded into a destination that is only
    4-byte aligned, which takes the per-element kernel: both must agree."""
    import oracle
    from cswap_amd import api

    torch = torch_cuda
    E, W, K = oracle.zvc_geometry(n, process)
    assert E % 4 == 0
    rng = np.random.default_rng(n + process)
    x = (rng.standard_normal(n) * (rng.random(n) < rng.uniform(0.1, 0.9))).astype(np.float32)
    print("n", n, "process", process, "E", E, flush=True)
    got = run_gpu(torch, x, process)
    check_against_oracle(x, got, process)
    t = torch.from_numpy(x).cuda()
    values, mask, begin, nnz = api.zvc_compress(t, process)
    buf = torch.full((n + 1,), -1.0, device="cuda")
    api.GPUdecompression(values, buf[1:], mask, begin, process)
    torch.cuda.synchronize()
    assert float(buf[0]) == -1.0
    assert np.array_equal(buf[1:].cpu().numpy().view(np.uint32), got[4].view(np.uint32))


@pytest.mark.parametrize("pct", [30, 50, 70, 90])
def test_fused_single_pass_config2(torch_cuda, fused_form, pct):
    from cswap_amd._lib import lib
    from cswap_amd.workloads import config2_tensor

    x = config2_tensor(pct).reshape(-1)
    assert lib().cswap_zvc_takes_single_pass(x.size, P) == (1 if fused_form == "pipeline" else 2)
    check_against_oracle(x, run_gpu(torch_cuda, x, fused=True))


@pytest.mark.parametrize("n,process", [(1, P), (33, P), (1000, P), (P - 1, P), (P + 1, P), (1_000_003, P),
                                        (P * 62 + 17, P), (P * 96 + 5, P), (P * 2048, P), (P * 4100 + 3, P),
                                        (300_001, 7), (64 * 9000 + 1, 64), (5000, 1)])
def test_fused_single_pass_ragged(torch_cuda, fused_form, n, process):
    """Every register-tile size of the fused kernel (8..128 values per lane), the
    fallback for chunks above 8192 elements, partial last chunks, idle chunks."""
    rng = np.random.default_rng(n % 1000 + process)
    x = (rng.standard_normal(n, dtype=np.float32) * (rng.random(n, dtype=np.float32) < 0.35)).astype(np.float32)
    print("n", n, "process", process, flush=True)
    check_against_oracle(x, run_gpu(torch_cuda, x, process, fused=True), process)


@pytest.mark.parametrize("n,process", [
    (P * 32, P),                 # one chunk per half row, 128 tiles: fewer tiles than compute units
    (P * 32 - 3205, P),          # the same with a hundred idle chunks and a partial row at the end
    (P * 32 * 3 - 45, P),        # chunks of 96 elements: they start on rows and on half rows
    (P * 512 - 1, P),            # 8 Mi elements, the last row one short
    (P * 4128 - 5000, P),        # 4128-element chunks: more than one round of the grid
    (P * 2048 - 10_000, P),      # several idle chunks
    (1024 * 16384, 1024),        # one chunk = one tile
    (999 * 160 - 37, 999),       # an odd number of mask words in all
    (64 * 2048 - 13, 64), (992, 1), (32, 1), (4096, 8)])
def test_single_pass_pipeline_kernel(torch_cuda, fused_form, n, process):
    """Shapes the single-kernel forms of the compression accept (chunk length a
    multiple of 32, at most 16384): grids smaller and larger than the number of tiles,
    partial rows, chunks that start in the middle of a row, idle chunks."""
    import oracle
    from cswap_amd._lib import lib

    E, W, K = oracle.zvc_geometry(n, process)
    assert E % 32 == 0 and E <= 16384
    takes = lib().cswap_zvc_takes_single_pass(n, process)
    rows = (W * process + 1) // 2                 # 64-element rows of the mask layout; the small form holds 256 x 16 x 32
    assert takes == (1 if fused_form == "pipeline" or 4 * n >= 64 << 20 else (2 if rows <= 131072 else 0))
    rng = np.random.default_rng(n % 977 + process)
    zeros = rng.uniform(0.2, 0.9)
    x = (rng.standard_normal(n, dtype=np.float32) * (rng.random(n, dtype=np.float32) > zeros)).astype(np.float32)
    print("n", n, "process", process, "E", E, flush=True)
    check_against_oracle(x, run_gpu(torch_cuda, x, process, fused=True), process)


def test_fused_repeated_calls_share_a_workspace(torch_cuda, fused_form):
    """A workspace is prepared once; every call that succeeds leaves it ready for the
    next: back-to-back calls on one stream with the same workspace, for tensors of
    different sizes, give the right result, and afterwards every word of it but the
    first is zero again."""
    torch = torch_cuda
    from cswap_amd import api
    from cswap_amd._lib import check, lib

    L = lib()
    ws = api.zvc_workspace(P)
    g = torch.Generator(device="cuda"); g.manual_seed(3)
    outs = []
    for rep, n in enumerate((P * 512, P * 64, P * 512)):
        t = torch.relu(torch.randn(n, generator=g, device="cuda"))
        values = torch.empty(n, device="cuda"); mask = torch.empty(n // 32, dtype=torch.int32, device="cuda")
        begin = torch.zeros(P, dtype=torch.int32, device="cuda"); nnz = torch.zeros(1, dtype=torch.int32, device="cuda")
        check(L.cswap_zvc_compress_fused(t.data_ptr(), n, P, ws.data_ptr(), begin.data_ptr(), nnz.data_ptr(),
                                         values.data_ptr(), mask.data_ptr(), None), "fused")
        torch.cuda.synchronize()
        k = int(nnz.item())
        assert k == int((t != 0).sum().item())
        assert torch.equal(values[:k], t[t != 0])
        assert int(ws.view(torch.int32)[1].item()) == 0      # no bounded wait ran out
        words = ws.view(torch.int32)
        assert int(words[3 if fused_form == "pipeline" else 4].item()) == rep + 1     # runs that have finished
        if fused_form == "pipeline":                         # every status word consumed and cleared
            assert int(words[5:].count_nonzero().item()) == 0 and int(words[2].item()) == 0
        else:                                                # all but this run's counts, which the next run clears
            tail = words[16:].clone()
            mine = tail.numel() - 512 + 256 * (rep & 1)
            assert int(tail[mine:mine + 256].count_nonzero().item()) == 256
            tail[mine:mine + 256] = 0
            assert int(tail.count_nonzero().item()) == 0


def test_fused_refuses_a_workspace_that_was_not_prepared(torch_cuda, fused_form):
    """A workspace that never went through cswap_zvc_workspace_clear is reported as a
    failure (nnz == -1), whatever it holds: zeros, or words that look like results
    (which the kernel then keeps from sending any write outside the outputs)."""
    torch = torch_cuda
    from cswap_amd._lib import check, lib

    L = lib()
    n = P * 256
    t = torch.relu(torch.randn(n, device="cuda"))
    values = torch.empty(n, device="cuda"); mask = torch.empty(n // 32, dtype=torch.int32, device="cuda")
    begin = torch.zeros(P, dtype=torch.int32, device="cuda")
    for fill in (0, -1):
        ws = torch.full((L.cswap_zvc_workspace_bytes(P) // 4,), fill, dtype=torch.int32, device="cuda")
        nnz = torch.zeros(1, dtype=torch.int32, device="cuda")
        check(L.cswap_zvc_compress_fused(t.data_ptr(), n, P, ws.data_ptr(), begin.data_ptr(), nnz.data_ptr(),
                                         values.data_ptr(), mask.data_ptr(), None), "fused")
        torch.cuda.synchronize()
        assert int(nnz.item()) == -1, fill


def test_fused_reports_a_wait_that_ran_out(torch_cuda, fused_form):
    """The single-pass kernel's waits for the counts of other workgroups are bounded.
    Forced from the host: the count of the first tile is never published and the bound
    is a few re-reads, so whoever waits for it gives up at once, every kernel still
    exits normally, and the caller sees nnz == -1 instead of made-up offsets.  The
    workspace stays refused until it is cleared; after that, with the defaults back,
    a call is correct again."""
    torch = torch_cuda
    from cswap_amd import api
    from cswap_amd._lib import check, lib

    L = lib()
    n = P * 256
    x = np.maximum(np.random.default_rng(5).standard_normal(n), 0).astype(np.float32)
    t = torch.from_numpy(x).cuda()
    ws = api.zvc_workspace(P)
    values = torch.empty(n, device="cuda"); mask = torch.empty(n // 32, dtype=torch.int32, device="cuda")
    begin = torch.zeros(P, dtype=torch.int32, device="cuda"); nnz = torch.zeros(1, dtype=torch.int32, device="cuda")
    L.cswap_zvc_debug_set_lookback(4, 1)
    try:
        print("forced give-up", flush=True)
        check(L.cswap_zvc_compress_fused(t.data_ptr(), n, P, ws.data_ptr(), begin.data_ptr(), nnz.data_ptr(),
                                         values.data_ptr(), mask.data_ptr(), None), "fused")
        torch.cuda.synchronize()
    finally:
        L.cswap_zvc_debug_set_lookback(0, 0)
    assert int(nnz.item()) == -1
    assert int(ws.view(torch.int32)[1].item()) == 1
    nnz.zero_()
    check(L.cswap_zvc_compress_fused(t.data_ptr(), n, P, ws.data_ptr(), begin.data_ptr(), nnz.data_ptr(),
                                     values.data_ptr(), mask.data_ptr(), None), "fused")
    torch.cuda.synchronize()
    assert int(nnz.item()) == -1                              # still refused: the failure sticks
    check(L.cswap_zvc_workspace_clear(ws.data_ptr(), P, None), "clear")
    check(L.cswap_zvc_compress_fused(t.data_ptr(), n, P, ws.data_ptr(), begin.data_ptr(), nnz.data_ptr(),
                                     values.data_ptr(), mask.data_ptr(), None), "fused")
    torch.cuda.synchronize()
    k = int(nnz.item())
    assert k == np.count_nonzero(x)
    assert np.array_equal(values[:k].cpu().numpy(), x[x != 0])
    check_against_oracle(x, run_gpu(torch, x, fused=True))


def test_special_values_and_extremes(torch_cuda, compact_form):
    n = P * 64
    x = np.zeros(n, dtype=np.float32)
    x[[3, 10, 11, 12, 13, 70]] = [-0.0, np.nan, np.inf, -np.inf, 1e-45, -2.5]
    got = run_gpu(torch_cuda, x)
    assert got[3] == 5
    assert np.array_equal(got[0].view(np.uint32), x[[10, 11, 12, 13, 70]].view(np.uint32))
    want = x.copy(); want[3] = 0.0
    assert np.array_equal(got[4].view(np.uint32), want.view(np.uint32))
    check_against_oracle(np.zeros(n, np.float32), run_gpu(torch_cuda, np.zeros(n, np.float32)))
    check_against_oracle(np.arange(1, n + 1, dtype=np.float32),
                         run_gpu(torch_cuda, np.arange(1, n + 1, dtype=np.float32)))


def test_special_values_and_extremes_single_kernel(torch_cuda, fused_form):
    """The same through both single-kernel forms: -0.0 is a zero, NaN, the infinities and the
    smallest subnormal are not; an all-zero tensor, a tensor without zeros, and tensors of one
    half row and of one workgroup's share."""
    from cswap_amd._lib import lib

    n = P * 64
    x = np.zeros(n, dtype=np.float32)
    x[[3, 10, 11, 12, 13, 70, n - 1]] = [-0.0, np.nan, np.inf, -np.inf, 1e-45, -2.5, 7.0]
    assert lib().cswap_zvc_takes_single_pass(n, P) == (1 if fused_form == "pipeline" else 2)
    got = run_gpu(torch_cuda, x, fused=True)
    assert got[3] == 6
    assert np.array_equal(got[0].view(np.uint32), x[[10, 11, 12, 13, 70, n - 1]].view(np.uint32))
    want = x.copy(); want[3] = 0.0
    assert np.array_equal(got[4].view(np.uint32), want.view(np.uint32))
    for y in (np.zeros(n, np.float32), np.arange(1, n + 1, dtype=np.float32),
              np.ones(32, np.float32), np.zeros(32, np.float32)):
        process = P if y.size == n else 1
        assert lib().cswap_zvc_takes_single_pass(y.size, process) != 0
        check_against_oracle(y, run_gpu(torch_cuda, y, process, fused=True), process)
    rng = np.random.default_rng(17)
    y = (rng.standard_normal(16 * 32 * 64 + 96, dtype=np.float32) * (rng.random(16 * 32 * 64 + 96) < 0.5)).astype(np.float32)
    check_against_oracle(y, run_gpu(torch_cuda, y, y.size // 32, fused=True), y.size // 32)   # chunks of one half row


def test_reference_call_sequence(torch_cuda):
    """The four launchers in the order CSWAP+/Execution.h:88-95 calls them, with a
    host read of nnz in between, produce what the one-call path produces."""
    torch = torch_cuda
    from cswap_amd import api
    from cswap_amd.workloads import config2_tensor

    x = config2_tensor(70, shape=(32, 256, 16, 16)).reshape(-1)
    t = torch.from_numpy(x).cuda()
    n = t.numel()
    E, W, K = api.zvc_geometry(n)
    index_begin = torch.zeros(P, dtype=torch.int32, device="cuda")
    num = torch.zeros(1, dtype=torch.int32, device="cuda")
    api.PreGPUcompression(t, index_begin)
    api.PreAcc(index_begin, K, num)
    nnz = int(num.item())
    values = torch.empty(nnz, dtype=torch.float32, device="cuda")
    mask = torch.empty(W * P, dtype=torch.int32, device="cuda")
    api.GPUcompression(t, values, index_begin, mask)
    dest = torch.empty_like(t)
    api.GPUdecompression(values, dest, mask, index_begin)
    torch.cuda.synchronize()
    assert torch.equal(dest, t)
    assert nnz == np.count_nonzero(x)
    assert np.array_equal(values.cpu().numpy(), x[x != 0])


def test_full_size_round_trip(torch_cuda):
    """256 MiB tensor: properties instead of the checker -- round trip, nnz,
    monotone chunk offsets, mask popcount == nnz."""
    torch = torch_cuda
    from cswap_amd import api

    g = torch.Generator(device="cuda"); g.manual_seed(1)
    t = torch.relu(torch.randn(64 * 1024 * 1024, generator=g, device="cuda"))
    v2, m2, b2, n2 = api.zvc_compress(t, fused=True)
    values, mask, begin, nnz = api.zvc_compress(t)
    torch.cuda.synchronize()
    k2 = int(n2.item())
    assert k2 == int(nnz.item()) and torch.equal(m2, mask) and torch.equal(b2, begin)
    assert torch.equal(v2[:k2], values[:k2])
    out = torch.full_like(t, 3.0)
    api.GPUdecompression(values, out, mask, begin)
    torch.cuda.synchronize()
    assert torch.equal(out, t)
    k = int(nnz.item())
    assert k == int((t != 0).sum().item()) == int(api.probe_nnz(t).item())
    b = begin.cpu().numpy()
    assert b[0] == 0 and np.all(np.diff(b) >= 0) and b[-1] <= k
    m = mask.cpu().numpy().view(np.uint8)
    assert int(np.unpackbits(m).sum()) == k
    assert torch.equal(values[:k], t[t != 0])


def test_random_sizes_chunk_counts_and_sparsities(torch_cuda, compact_form):
    """120 seeded cases: n from 1 to 400 000, chunk counts from 1 to 65 536 (more
    chunks than elements included), zero fractions from 0 to 1 with special values
    mixed in, plain and single-pass compaction, and a destination that is not
    16-byte aligned (the one-element-per-lane expansion)."""
    torch = torch_cuda
    from cswap_amd import api

    rng = np.random.default_rng(99)
    specials = np.array([-0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38], dtype=np.float32)
    for case in range(120):
        n = int(rng.choice([rng.integers(1, 100), rng.integers(100, 5000), rng.integers(5000, 400_000)]))
        process = int(rng.choice([1, 3, 7, 64, 1000, 1024, 4096, 16384, 65536]))
        zeros = float(rng.choice([0.0, 0.05, 0.5, 0.9, 0.999, 1.0]))
        x = rng.standard_normal(n).astype(np.float32)
        x[rng.random(n) < zeros] = 0.0
        k = rng.integers(0, 8)
        if k and n > 8:
            x[rng.integers(0, n, size=k)] = rng.choice(specials, size=k)
        fused = bool(case % 2)
        tag = (case, n, process, zeros, fused)
        print(tag, flush=True)
        got = run_gpu(torch, x, process, fused=fused)
        check_against_oracle(x, got, process)
        # unaligned destination
        t = torch.from_numpy(x).cuda()
        values, mask, begin, nnz = api.zvc_compress(t, process)
        buf = torch.full((n + 8,), -1.0, device="cuda")
        shift = 1 + case % 3
        api.GPUdecompression(values, buf[shift:shift + n], mask, begin, process)
        torch.cuda.synchronize()
        b = buf.cpu().numpy()
        want = np.where(x != 0, x, np.float32(0))
        assert np.array_equal(b[shift:shift + n].view(np.uint32), want.view(np.uint32)), tag
        assert (b[:shift] == -1).all() and (b[shift + n:] == -1).all(), tag


@pytest.mark.parametrize("nnz_per_chunk", [0, 1, 3, 255, 256, 257, 511, 512, 513, 1000])
def test_staged_compaction_ring_boundaries(torch_cuda, nnz_per_chunk):
    """The staged form writes a wave's ring out 256 values at a time: chunks whose
    counts sit on either side of one and two ring halves, so that every alignment of
    a chunk's first value (begin % 4) meets every fill level at the end of a chunk."""
    from cswap_amd._lib import lib

    E, chunks = 1024, 48
    rng = np.random.default_rng(nnz_per_chunk)
    x = np.zeros(E * chunks, dtype=np.float32)
    for c in range(chunks):
        k = min(E, max(0, nnz_per_chunk + (c % 5) - 2)) if nnz_per_chunk else 0
        idx = rng.choice(E, size=k, replace=False)
        x[c * E + idx] = rng.standard_normal(k).astype(np.float32) + 3.0
    before = lib().cswap_zvc_set_staged_compact_bytes(0)
    try:
        got = run_gpu(torch_cuda, x, chunks)
    finally:
        lib().cswap_zvc_set_staged_compact_bytes(before)
    check_against_oracle(x, got, chunks)


def test_staged_threshold_is_reported_and_restored(torch_cuda):
    from cswap_amd._lib import lib

    L = lib()
    default = L.cswap_zvc_set_staged_compact_bytes(12345)
    assert default == 192 << 20
    assert L.cswap_zvc_set_staged_compact_bytes(default) == 12345
