"""Configurations 4 and 5 of the benchmark at their full sizes, through the C ABI.

Configuration 5: every tensor (hidden, FFN, attention probabilities) at 8 and 16
bits per value against the stock zfp 0.5.5 serial library on this machine's CPU
where it exists, and against the CPU checker on all cores: every stream byte
and every decoded value.

Configuration 4: the VGG-16 activation schedule at batch 128 through the swap
engine with the selector switched on: what the selector picks per kind of
tensor, the round trip against the codec's own round trip, and the latency of
every tensor it compressed against the raw swap of the same tensor.
"""
import time

import numpy as np
import pytest

from conftest import libzfp as _libzfp, libzfp_round_trip

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


@pytest.mark.parametrize("rate", [8, 16])
@pytest.mark.parametrize("name", ["hidden_gelu", "ffn_gelu", "attn_softmax"])
def test_config5_tensor_at_full_size(torch_cuda, name, rate):
    torch = torch_cuda
    import oracle
    from cswap_amd import api
    from cswap_amd.workloads import config5_tensor_torch, field_dims

    x = config5_tensor_torch(name, torch.device("cuda"), seed=0)
    nx, ny, nz = field_dims(x.shape)
    maxbits = 64 * rate
    print("config 5", name, "rate", rate, "field", (nx, ny, nz), flush=True)
    s = api.cuda_compress(x, maxbits)
    d = api.cuda_decompress(s, x.shape, maxbits)
    torch.cuda.synchronize()
    f = x.cpu().numpy().reshape(nz, ny, nx)
    got_stream = s.cpu().numpy()
    got_dec = d.cpu().numpy().reshape(f.shape).view(np.uint32)
    assert got_stream.size == f.size * rate // 8
    print("checker on all cores", flush=True)
    want = oracle.zfp_encode3(f, maxbits, omp=True)
    assert np.array_equal(got_stream.view(np.uint64), want)
    assert np.array_equal(got_dec, oracle.zfp_decode3(want, f.shape, maxbits, omp=True).view(np.uint32))
    Z = _libzfp()
    if Z is not None:
        print("zfp 0.5.5 library on one core", flush=True)
        zbits, zstream, zdec = libzfp_round_trip(Z, f, float(rate))
        assert zbits == maxbits
        assert np.array_equal(got_stream, zstream)
        assert np.array_equal(got_dec, zdec.view(np.uint32))


def _median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def test_config4_schedule_through_the_selector(torch_cuda):
    torch = torch_cuda
    import oracle
    from cswap_amd import swap
    from cswap_amd.workloads import config4_schedule, config4_tensor, dummy_layer_compute, field_dims

    sched = config4_schedule(128)
    assert len(sched) == 44
    biggest = max(int(np.prod(e["shape"])) for e in sched) * 4
    eng = swap.SwapEngine(pinned_bytes=2 * biggest + (64 << 20), device_bytes=2 * biggest + (64 << 20))
    eng.calibrate()
    a = torch.randn(2048, 2048, device="cuda")
    b = torch.randn(2048, 2048, device="cuda")
    picked = {"relu": [], "dense": [], "pool": []}
    try:
        for e in sched:
            xn = config4_tensor(e, 0)
            x = torch.from_numpy(xn).cuda()
            out = torch.full_like(x, -3.0)
            lat = {}
            for label, pol in (("none", swap.NONE), ("auto", swap.AUTO)):
                times = []
                for _ in range(5):
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    tk = eng.pre(x, pol)
                    dummy_layer_compute(a, b, 2)      # the layer's kernels, while the copy is in flight
                    eng.post(tk)
                    eng.swap_in(tk, out)
                    torch.cuda.synchronize()
                    times.append(time.perf_counter() - t0)
                    info = eng.info(tk)
                    eng.release(tk)
                lat[label] = _median(times)
            # `info` and `out` are those of the last selector-driven swap
            zeros = 1.0 - np.count_nonzero(xn) / xn.size
            mb = xn.nbytes / 1e6
            print(f"id {e['id']:2d} {e['kind']:5s} {mb:6.1f} MB zeros {zeros:.2f} -> {swap.POLICY_NAME[info.policy]:6s} "
                  f"raw {lat['none'] * 1e3:.3f} ms selector {lat['auto'] * 1e3:.3f} ms", flush=True)
            picked[e["kind"]].append((info.policy, mb, zeros))
            nx, ny, nz = field_dims(x.shape)
            got = out.cpu().numpy()
            if info.policy == swap.ZFP:
                f = xn.reshape(nz, ny, nx)
                want = oracle.zfp_decode3(oracle.zfp_encode3(f, 512, omp=True), f.shape, 512, omp=True)
                assert np.array_equal(got.reshape(f.shape).view(np.uint32), want.view(np.uint32))
                assert info.bytes_out == xn.size
            else:                                       # raw and ZVC are lossless
                assert np.array_equal(got.view(np.uint32), xn.view(np.uint32))
                if info.policy == swap.SPARSE:
                    assert info.nnz == np.count_nonzero(xn)
            if info.policy != swap.NONE:
                # the acceptance test of the path: a tensor the selector compresses swaps faster than raw.
                # Both arms are medians of five wall-clock timings on a shared host: 5 % of slack keeps
                # scheduler noise out of a parity suite; the strict figures are in the line printed above
                assert lat["auto"] <= 1.05 * lat["none"], (e, lat)
            else:
                assert lat["auto"] <= 1.25 * lat["none"] + 50e-6, (e, lat)
            del x, out
    finally:
        eng.close()
    # the assignment the reference's drivers write by hand (vgg16-cifar10.cpp:177-178,393-397):
    # sparse compaction for ReLU outputs, ZFP for dense and pooled tensors, small tensors left alone
    for pol, mb, zeros in picked["dense"]:
        assert pol != swap.SPARSE
        assert pol == swap.ZFP or mb < 8
    for pol, mb, zeros in picked["relu"]:
        assert pol != swap.NONE or mb < 8
        if zeros >= 0.6 and mb >= 8:
            assert pol == swap.SPARSE
    for pol, mb, zeros in picked["pool"]:
        assert pol in (swap.ZFP, swap.SPARSE) or mb < 8
    assert picked["pool"][-1][0] == swap.NONE          # [128,512,2,2]: blocks that are 3/4 padding, 1 MB
    assert sum(p == swap.SPARSE for p, _, _ in picked["relu"]) >= 5
    assert all(p == swap.ZFP for p, mb, _ in picked["dense"] if mb >= 8)
