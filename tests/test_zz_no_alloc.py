"""cswap_zvc_compress_fused_static: the single-pass compression with its status
words in the library's static device array.  Checked through the C ABI against
cswap_zvc_compress_fused (workspace from the caller) on the same inputs, bit for
bit, on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
P = 512 * 32


def _run(torch, L, x, process, static):
    from cswap_amd import api
    from cswap_amd._lib import check

    n = x.numel()
    W = L.cswap_zvc_chunk_words(n, process)
    values = torch.full((n,), -7.0, device="cuda")
    mask = torch.full((W * process,), -1, dtype=torch.int32, device="cuda")
    begin = torch.full((process,), -1, dtype=torch.int32, device="cuda")
    nnz = torch.full((1,), -5, dtype=torch.int32, device="cuda")
    if static:
        check(L.cswap_zvc_compress_fused_static(x.data_ptr(), n, process, begin.data_ptr(), nnz.data_ptr(),
                                                values.data_ptr(), mask.data_ptr(), None), "fused_static")
    else:
        ws = api.zvc_workspace(process)
        check(L.cswap_zvc_compress_fused(x.data_ptr(), n, process, ws.data_ptr(), begin.data_ptr(), nnz.data_ptr(),
                                         values.data_ptr(), mask.data_ptr(), None), "fused")
    torch.cuda.synchronize()
    k = int(nnz.item())
    return k, values[:max(k, 0)].cpu().numpy(), mask.cpu().numpy(), begin.cpu().numpy()


def test_static_scratch_entry_point_matches_the_workspace_one():
    import torch

    from cswap_amd._lib import lib

    assert torch.cuda.is_available(), "this test needs the GPU"
    L = lib()
    g = torch.Generator(device="cuda"); g.manual_seed(11)
    size_rule = L.cswap_zvc_set_single_pass_bytes(0)     # the single pass (the kernel that uses the scratch) at any size
    # later calls are smaller; the last shape is one the single pass does not take
    for n, process in ((P * 512 - 77, P), (P * 64 - 3, P), (300_001, 7)):
        assert L.cswap_zvc_takes_single_pass(n, process) == (process == P)
        x = torch.relu(torch.randn(n, generator=g, device="cuda"))
        print("static entry point: n", n, "process", process, flush=True)
        want = _run(torch, L, x, process, static=False)
        got = _run(torch, L, x, process, static=True)
        assert got[0] == want[0] == int((x != 0).sum().item())
        for a, b in zip(got[1:], want[1:]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(got[1], x[x != 0].cpu().numpy())
    # A run whose bounded waits run out (forced from the host: the first tile's count is never
    # published, the bound is a few re-reads) reports -1 and leaves the static array refused
    # until cswap_zvc_workspace_clear(NULL, ...) has prepared it again.
    n = P * 64
    x = torch.relu(torch.randn(n, generator=g, device="cuda"))
    L.cswap_zvc_debug_set_lookback(4, 1)
    try:
        print("static entry point: forced give-up", flush=True)
        assert _run(torch, L, x, P, static=True)[0] == -1
    finally:
        L.cswap_zvc_debug_set_lookback(0, 0)
    assert _run(torch, L, x, P, static=True)[0] == -1
    assert L.cswap_zvc_workspace_clear(None, 0, None) == 0
    got = _run(torch, L, x, P, static=True)
    assert got[0] == int((x != 0).sum().item())
    assert np.array_equal(got[1], x[x != 0].cpu().numpy())
    L.cswap_zvc_set_single_pass_bytes(size_rule)
    # beyond the static array: refused, nothing launched
    x = torch.zeros(1 << 20, device="cuda")
    big = 65536 * 2
    out = torch.zeros(big, dtype=torch.int32, device="cuda")
    assert L.cswap_zvc_compress_fused_static(x.data_ptr(), x.numel(), big, out.data_ptr(), out.data_ptr(),
                                             x.data_ptr(), out.data_ptr(), None) == -4
