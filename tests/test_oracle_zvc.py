"""Pins the CPU checker's ZVC restatement against numpy library routines
(boolean indexing, packbits, cumsum) -- independent statements of what the
reference format must contain (CSWAP+/zfp/compression.cu:134-239)."""
import numpy as np
import pytest

import oracle
from cswap_amd.workloads import config2_tensor

P = oracle.PROCESS


def flat_mask(x):
    return np.packbits(x != 0, bitorder="little")


@pytest.mark.parametrize("n", [P * 64, P * 512, P * 32 * 3])
def test_divisible_shapes_match_numpy(n):
    rng = np.random.default_rng(n)
    x = np.maximum(rng.standard_normal(n), 0).astype(np.float32)
    vals, mask, begin, nnz = oracle.zvc_compress(x)
    E, W, K = oracle.zvc_geometry(n)
    assert (E, W, K) == (n // P, n // P // 32, P)
    assert nnz == np.count_nonzero(x)
    assert np.array_equal(vals.view(np.uint32), x[x != 0].view(np.uint32))
    assert np.array_equal(mask.view(np.uint8), flat_mask(x))
    cnt = (x.reshape(P, E) != 0).sum(axis=1)
    assert np.array_equal(begin, np.concatenate([[0], np.cumsum(cnt)[:-1]]))
    assert np.array_equal(oracle.zvc_count(x), cnt)
    out = oracle.zvc_decompress(vals, mask, begin, n)
    assert np.array_equal(out.view(np.uint32), x.view(np.uint32))
    out2 = oracle.zvc_decompress(vals, mask, begin, n, reference_writes=True)
    assert np.array_equal(out2.view(np.uint32), x.view(np.uint32))


@pytest.mark.parametrize("n", [1, 31, 33, 1000, P - 1, P + 1, 1_000_003, P * 62 + 17])
def test_ragged_shapes(n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * (rng.random(n) < 0.4)).astype(np.float32)
    vals, mask, begin, nnz = oracle.zvc_compress(x)
    E, W, K = oracle.zvc_geometry(n)
    assert E == -(-n // P) and W == -(-E // 32) and K == -(-n // E)
    assert np.array_equal(vals.view(np.uint32), x[x != 0].view(np.uint32))
    # chunk-relative mask layout: chunk i's bits start at word i*W
    for i in list(range(min(K, 50))) + [K - 1]:
        c = x[i * E:(i + 1) * E]
        bits = np.unpackbits(mask[i * W:(i + 1) * W].view(np.uint8), bitorder="little")
        assert np.array_equal(bits[: c.size], (c != 0).astype(np.uint8))
        assert not bits[c.size:].any()
        assert begin[i] == np.count_nonzero(x[: i * E])
    out = oracle.zvc_decompress(vals, mask, begin, n)
    want = np.where(x != 0, x, np.float32(0))     # -0.0 is dropped and comes back +0.0
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def test_special_values():
    x = np.zeros(P * 64, dtype=np.float32)
    x[3] = -0.0
    x[10] = np.nan
    x[11] = np.inf
    x[12] = -np.inf
    x[13] = np.float32(1e-45)   # subnormal: kept
    x[70] = -2.5
    vals, mask, begin, nnz = oracle.zvc_compress(x)
    assert nnz == 5
    assert np.array_equal(vals.view(np.uint32), x[[10, 11, 12, 13, 70]].view(np.uint32))
    out = oracle.zvc_decompress(vals, mask, begin, x.size)
    want = x.copy(); want[3] = 0.0          # -0.0 comes back as +0.0
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def test_all_zero_and_all_nonzero():
    n = P * 64
    z = np.zeros(n, np.float32)
    vals, mask, begin, nnz = oracle.zvc_compress(z)
    assert nnz == 0 and not mask.any() and not begin.any()
    assert not oracle.zvc_decompress(vals, mask, begin, n).any()
    o = np.arange(1, n + 1, dtype=np.float32)
    vals, mask, begin, nnz = oracle.zvc_compress(o)
    assert nnz == n and np.all(mask == 0xffffffff) and np.array_equal(vals, o)
    assert np.array_equal(oracle.zvc_decompress(vals, mask, begin, n), o)


@pytest.mark.parametrize("pct", [30, 50, 70, 90])
def test_config2_sparsity_sweep(pct):
    x = config2_tensor(pct).reshape(-1)
    vals, mask, begin, nnz = oracle.zvc_compress(x)
    assert abs((1 - nnz / x.size) * 100 - pct) < 0.2
    assert np.array_equal(mask.view(np.uint8), flat_mask(x))
    assert np.array_equal(vals, x[x != 0])
    assert mask.nbytes == oracle.lib().orc_zvc_mask_bytes(x.size, P) == x.size // 8


def test_omp_build_matches_serial():
    x = config2_tensor(50, shape=(16, 64, 16, 16)).reshape(-1)
    a = oracle.zvc_compress(x)
    b = oracle.zvc_compress(x, omp=True)
    for u, v in zip(a[:3], b[:3]):
        assert np.array_equal(u, v)
