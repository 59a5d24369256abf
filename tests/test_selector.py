"""Host-only tests of the selector.  The reference ships no selector (its
PolicyMaker is in an absent patched PyTorch), so these pin invariants, not
values: monotone in sparsity and in size, never sparse without a gain, never
lossy when forbidden, nothing compressed below the size floor, and the outcome
the reference's hand-written policy vectors encode (ZVC for ReLU outputs, ZFP for
dense/pooled tensors, CSWAP+/vgg16-cifar10.cpp:177-178,393-397)."""
import ctypes as C

import pytest

from cswap_amd import swap
from cswap_amd._lib import lib

NONE, SPARSE, ZFP = swap.NONE, swap.SPARSE, swap.ZFP


def test_policy_bytes_closed_forms():
    L = lib()
    n = 128 * 256 * 16 * 16
    assert L.cswap_policy_bytes(NONE, n, 0, 512, 16384, 0, 0, 0) == 4 * n
    assert L.cswap_policy_bytes(SPARSE, n, n // 2, 512, 16384, 0, 0, 0) == 4 * (n // 2) + n // 8 + 65536
    assert L.cswap_policy_bytes(ZFP, n, 0, 512, 16384, 0, 0, 0) == n
    assert L.cswap_policy_bytes(ZFP, 0, 0, 512, 16384, 2, 2, 65536) == 16384 * 64   # partial blocks pay full rate


def test_sparse_chosen_for_relu_zfp_for_dense_none_for_tiny():
    n = 128 * 64 * 32 * 32
    assert swap.select(n, int(0.4 * n)).policy == SPARSE           # ReLU output, 60 % zeros
    assert swap.select(n, n).policy == ZFP                         # dense pre-activation
    assert swap.select(n, int(0.85 * n)).policy == ZFP             # few zeros: ZVC barely helps, ZFP >2x faster
    assert swap.select(1024, 100).policy == NONE                   # below the size floor
    c = swap.default_costs(); c.allow_lossy = 0
    assert swap.select(n, n, costs=c).policy == NONE               # dense + lossless only -> raw swap
    assert swap.select(n, int(0.4 * n), costs=c).policy == SPARSE


def test_monotone_in_sparsity():
    n = 1 << 24
    c = swap.default_costs(); c.allow_lossy = 0
    last_t, seen_sparse = None, False
    for zeros_pct in range(0, 101, 2):
        nnz = n * (100 - zeros_pct) // 100
        ch = swap.select(n, nnz, costs=c)
        if ch.t_sparse_us >= 0:
            assert last_t is None or ch.t_sparse_us <= last_t + 1e-9
            last_t = ch.t_sparse_us
        if seen_sparse:
            assert ch.policy == SPARSE, "once sparse wins it keeps winning as zeros increase"
        seen_sparse |= ch.policy == SPARSE
    assert seen_sparse


def test_never_sparse_without_gain():
    n = 1 << 22
    c = swap.default_costs()
    for nnz in (n, n - 1, int(0.97 * n)):
        ch = swap.select(n, nnz, costs=c)
        assert ch.policy != SPARSE
        assert ch.t_sparse_us == -1.0 or lib().cswap_policy_bytes(SPARSE, n, nnz, 512, 16384, 0, 0, 0) < 0.9 * 4 * n


def test_monotone_in_size():
    c = swap.default_costs()
    for density in (0.3, 1.0):
        compressed = False
        for logn in range(10, 30):
            n = 1 << logn
            ch = swap.select(n, int(density * n), costs=c)
            if compressed:
                assert ch.policy != NONE, (density, logn)
            compressed |= ch.policy != NONE
        assert compressed


def test_chosen_option_never_modelled_slower_than_raw():
    c = swap.default_costs()
    for n in (1 << 16, 1 << 20, 1 << 26):
        for d in (0.05, 0.5, 0.95, 1.0):
            ch = swap.select(n, int(d * n), costs=c)
            t = {NONE: ch.t_none_us, SPARSE: ch.t_sparse_us, ZFP: ch.t_zfp_us}[ch.policy]
            assert 0 <= t <= ch.t_none_us
            if ch.policy == ZFP and ch.t_sparse_us >= 0 and ch.t_sparse_us < ch.t_none_us:
                assert ch.t_zfp_us < c.lossy_min_gain * ch.t_sparse_us


def test_partial_block_fields_pay_full_rate():
    """A 2x2xN field (the [128,512,2,2] activation) fills only 1/4 of every 4x4x4
    block: rate 8 gives no size gain, so ZFP must not be chosen for it."""
    ch = swap.select_field(2, 2, 65536, 2 * 2 * 65536)
    assert ch.policy == NONE
    flat = swap.select(2 * 2 * 65536, 2 * 2 * 65536)
    assert flat.bytes_out in (2 * 2 * 65536, 4 * 2 * 2 * 65536)
    big = swap.select_field(2, 2, 1 << 24, 4 << 24)
    assert big.policy == NONE and big.t_zfp_us == -1.0


def test_margin_and_probe_cost_keep_small_tensors_raw():
    c = swap.default_costs()
    n = 1 << 20                                   # 4 MiB: the inbound copy takes ~85 us, the probe ~30 us
    assert swap.select(n, n, costs=c).policy == NONE
    assert swap.select(1 << 22, 1 << 22, costs=c).policy == ZFP    # 16 MiB pays
    c.probe_latency_us = 0.0
    c.min_gain = 1.0
    assert swap.select(n, n, costs=c).policy == ZFP
    c.min_gain = 0.1                              # demand a 10x gain: nothing qualifies
    assert swap.select(1 << 26, 1 << 26, costs=c).policy == NONE


def test_ties_stay_lossless():
    c = swap.default_costs()
    # an infinitely fast link makes all options equal up to kernel time: raw wins
    c.bw_d2h_gbs = c.bw_h2d_gbs = 1e12
    c.copy_latency_us = 0.0
    assert swap.select(1 << 24, 1 << 20, costs=c).policy == NONE


def test_bad_arguments():
    ch = swap.Choice()
    assert lib().cswap_select(0, 0, 512, None, C.byref(ch)) == -1
    assert lib().cswap_select(10, 11, 512, None, C.byref(ch)) == -1
    assert lib().cswap_select(10, 1, 512, None, None) == -1


def test_chunk_count_rule():
    """About 1024 elements per chunk, a power of two between 1024 and 16384."""
    from cswap_amd._lib import lib

    L = lib()
    assert L.cswap_zvc_pick_process(1) == 1024
    assert L.cswap_zvc_pick_process(262144) == 1024          # 1 MiB
    assert L.cswap_zvc_pick_process(4 << 20) == 4096         # 16 MiB
    assert L.cswap_zvc_pick_process(8 << 20) == 8192         # 32 MiB
    assert L.cswap_zvc_pick_process(64 << 20) == 16384       # 256 MiB
    assert L.cswap_zvc_pick_process(2**31 - 1) == 16384
    prev = 0
    for k in range(10, 31):
        p = L.cswap_zvc_pick_process(1 << k)
        assert p >= prev and p & (p - 1) == 0 and 1024 <= p <= 16384
        prev = p
