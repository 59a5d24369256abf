"""The low-level entry points allocate nothing and take the caller's stream, so
they can be recorded into a HIP graph.  Every replay is checked against the
eager result, with eager work and synchronisation between the replays."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_codec_calls_replay_correctly_from_a_hip_graph():
    import torch

    from cswap_amd import api
    from cswap_amd._lib import check, lib

    assert torch.cuda.is_available()
    L = lib()
    dev = torch.device("cuda")
    nz, ny, nx = 64, 32, 32
    n = nz * ny * nx
    P = L.cswap_zvc_pick_process(n)
    _, W, _ = api.zvc_geometry(n, P)
    x = torch.zeros(nz, ny, nx, device=dev)
    stream = torch.zeros(L.cswap_zfp_stream_capacity(nx, ny, nz, 512), dtype=torch.uint8, device=dev)
    dec = torch.zeros_like(x)
    values = torch.zeros(n, device=dev)
    mask = torch.zeros(W * P, dtype=torch.int32, device=dev)
    begin = torch.zeros(P, dtype=torch.int32, device=dev)
    nnz = torch.zeros(1, dtype=torch.int32, device=dev)
    back = torch.zeros_like(x)

    def work():
        st = torch.cuda.current_stream().cuda_stream
        check(L.cswap_zfp_compress_f32(x.data_ptr(), nx, ny, nz, 0, 0, 0, 512, stream.data_ptr(), st), "zfp c")
        check(L.cswap_zfp_decompress_f32(stream.data_ptr(), nx, ny, nz, 0, 0, 0, 512, dec.data_ptr(), st), "zfp d")
        check(L.cswap_zvc_compress(x.data_ptr(), n, P, begin.data_ptr(), nnz.data_ptr(), values.data_ptr(),
                                   mask.data_ptr(), st), "zvc c")
        check(L.cswap_zvc_expand(values.data_ptr(), mask.data_ptr(), begin.data_ptr(), n, P, back.data_ptr(), st),
              "zvc e")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                 # warm-up outside capture
        work()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        work()
    for seed in range(4):
        gen = torch.Generator(device=dev).manual_seed(seed)
        new = torch.relu(torch.randn(x.shape, generator=gen, device=dev) - 0.3 * seed)
        x.copy_(new)
        work()                                    # eager
        torch.cuda.synchronize()
        want = [t.clone() for t in (stream, dec, back, nnz)]
        k = int(nnz.item())
        want_vals = values[:k].clone()
        for t in (stream, dec, back, nnz, values):
            t.fill_(0)                            # eager work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for got, w in zip((stream, dec, back, nnz), want):
            assert torch.equal(got, w), seed
        assert torch.equal(values[:k], want_vals) and torch.equal(back, x)
        assert k == int((x != 0).sum())


@pytest.mark.parametrize("mib", [4, 96])
def test_static_workspace_compression_replays_from_a_hip_graph(mib):
    """cswap_zvc_compress_fused_static is meant for code under graph capture: it takes
    no workspace and allocates nothing, and both of its single-kernel forms keep their
    status words clean by themselves (the form for small tensors alternates between two
    count arrays from one run to the next, the pipeline kernel clears what it consumes),
    so a captured call can be replayed any number of times."""
    import torch

    from cswap_amd import api
    from cswap_amd._lib import check, lib

    assert torch.cuda.is_available()
    L = lib()
    dev = torch.device("cuda")
    P = 16384
    n = mib << 18
    assert L.cswap_zvc_takes_single_pass(n, P) == (2 if mib == 4 else 1)
    x = torch.zeros(n, device=dev)
    values = torch.zeros(n, device=dev)
    mask = torch.zeros(n // 32, dtype=torch.int32, device=dev)
    begin = torch.zeros(P, dtype=torch.int32, device=dev)
    nnz = torch.zeros(1, dtype=torch.int32, device=dev)
    back = torch.zeros_like(x)

    def work():
        st = torch.cuda.current_stream().cuda_stream
        check(L.cswap_zvc_compress_fused_static(x.data_ptr(), n, P, begin.data_ptr(), nnz.data_ptr(),
                                                values.data_ptr(), mask.data_ptr(), st), "fused static")
        check(L.cswap_zvc_expand(values.data_ptr(), mask.data_ptr(), begin.data_ptr(), n, P, back.data_ptr(), st),
              "expand")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                 # warm-up outside capture
        work()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        work()
    for seed in range(5):                         # an odd number of replays and eager calls in between
        gen = torch.Generator(device=dev).manual_seed(seed)
        x.copy_(torch.relu(torch.randn(n, generator=gen, device=dev) - 0.4 * seed))
        print("replay", seed, flush=True)
        for t in (back, nnz, values, mask, begin):
            t.fill_(0)                            # eager work between replays
        if seed % 2:
            work()                                # an eager call between two replays shares the static array
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        k = int(nnz.item())
        assert k == int((x != 0).sum()), seed
        assert torch.equal(values[:k], x[x != 0]) and torch.equal(back, x), seed
