"""The planner has no implementation in the reference's tree (c10::PolicyMaker
belongs to a patched PyTorch), so its results are pinned by invariants: what a
plan may and may not contain, how it moves with the target and with the cost
model, and two tiny schedules worked out by hand."""
import os
import subprocess
import tempfile

import pytest

from conftest import ROOT


def costs(**kw):
    from cswap_amd import swap

    c = swap.default_costs()
    c.bw_d2h_gbs = c.bw_h2d_gbs = 50.0
    c.copy_latency_us = 10.0
    c.kernel_latency_us = 4.0
    c.zfp_latency_us = 4.0
    c.size_floor_bytes = 0
    for k, v in kw.items():
        setattr(c, k, v)
    return c


def vgg_like(pm, n_ops=20, mb=64, relu_every=3, nnz_share=0.4, comptime=300.0):
    """A chain: op i consumes tensor i-1 and produces tensor i."""
    for i in range(n_ops):
        pm.add_comptime(comptime)
        pm.add_tensor(i, mb << 20)
        pm.add_stepdep([i - 1, i])
        pm.set_field(i, 32, 32, (mb << 20) // 4 // 1024)
        if i % relu_every == 2:
            pm.set_nnz(i, int(nnz_share * ((mb << 20) // 4)))


def test_nothing_is_planned_for_ratio_zero_and_time_is_the_base_time():
    from cswap_amd.planner import PolicyMaker

    pm = PolicyMaker(costs())
    vgg_like(pm)
    pm.init(0.0)
    pol, t = pm.make_policy(20)
    assert pol == [0] * 20
    assert t == pytest.approx(20 * 300.0 * 3)         # forward + 2x backward
    assert pm.summary.base_time_us == t and pm.summary.target_met == 1
    assert pm.begin_stage[:19] == list(range(1, 20))  # a chain: tensor i is last used by op i+1


def test_plan_meets_the_target_and_grows_with_it():
    from cswap_amd.planner import PolicyMaker

    pm = PolicyMaker(costs())
    vgg_like(pm)
    prev_moved, prev_time, prev_set = 0, 0.0, set()
    for ratio in (0.1, 0.3, 0.5, 0.7, 0.85):
        pm.init(ratio)
        pol, t = pm.make_policy(20)
        s = pm.summary
        chosen = {i for i, p in enumerate(pol) if p}
        assert s.target_met and s.bytes_moved >= ratio * s.bytes_total
        assert s.bytes_moved - (64 << 20) < ratio * s.bytes_total      # stops at the first tensor that meets it
        assert s.bytes_moved >= prev_moved and t >= prev_time and chosen >= prev_set
        assert set(pol) <= {0, 2, 3, 6}
        assert t >= s.base_time_us
        prev_moved, prev_time, prev_set = s.bytes_moved, t, chosen
    # the last tensor (no consumer) and the one consumed by the last op are never taken
    pm.init(1.0)
    pol, _ = pm.make_policy(20)
    assert pol[19] == 0 and pol[18] == 0 and pm.summary.target_met == 0
    assert all(p != 0 for p in pol[:18])


def test_actions_follow_the_cost_model():
    from cswap_amd.planner import PolicyMaker

    # slow link, fast kernels: compression pays; sparse tensors go ZVC unless ZFP wins by the lossy margin
    pm = PolicyMaker(costs(lossy_min_gain=0.0))          # lossy never preferred over a lossless option
    vgg_like(pm, nnz_share=0.3)
    pm.init(1.0)
    pol, _ = pm.make_policy(20)
    assert all(pol[i] == 3 for i in range(18) if i % 3 == 2)
    assert all(pol[i] == 2 for i in range(18) if i % 3 != 2)
    # lossy allowed and clearly cheaper for dense tensors
    pm2 = PolicyMaker(costs(lossy_min_gain=0.9))
    vgg_like(pm2, nnz_share=0.3)
    pm2.init(1.0)
    pol2, t2 = pm2.make_policy(20)
    assert all(pol2[i] == 6 for i in range(18) if i % 3 != 2)
    # lossy forbidden
    pm3 = PolicyMaker(costs(allow_lossy=0))
    vgg_like(pm3, nnz_share=0.3)
    pm3.init(1.0)
    pol3, t3 = pm3.make_policy(20)
    assert 6 not in pol3 and t3 >= t2
    # a link so fast that the copies hide under the compute: raw swap is free, nothing gets compressed
    pm4 = PolicyMaker(costs(bw_d2h_gbs=5000.0, bw_h2d_gbs=5000.0))
    vgg_like(pm4, nnz_share=0.3)
    pm4.init(1.0)
    pol4, t4 = pm4.make_policy(20)
    assert set(pol4[:18]) == {2} and t4 == pytest.approx(pm4.summary.base_time_us)
    # nearly dense "sparse" tensors are not worth ZVC
    pm5 = PolicyMaker(costs(allow_lossy=0))
    vgg_like(pm5, nnz_share=0.95)
    pm5.init(1.0)
    pol5, _ = pm5.make_policy(20)
    assert 3 not in pol5


def test_omitted_small_and_unconsumed_tensors_stay():
    from cswap_amd.planner import PolicyMaker

    pm = PolicyMaker(costs(size_floor_bytes=1 << 20))
    vgg_like(pm)
    pm.add_omitid(4)
    pm.add_tensor(7, 1000 * 4)           # below the size floor
    pm.add_tensor(30, 64 << 20)          # recorded but never consumed
    pm.init(1.0)
    pol, _ = pm.make_policy(40)
    assert pol[4] == 0 and pol[7] == 0 and pol[30] == 0
    assert pm.begin_stage[30] == 31      # Execution's default


def test_capuchin_baseline_is_raw_only_and_never_cheaper():
    from cswap_amd.planner import PolicyMaker

    pm = PolicyMaker(costs())
    vgg_like(pm)
    for ratio in (0.2, 0.5, 0.8):
        pm.init(ratio)
        pol, t = pm.make_policy(20)
        moved = pm.summary.bytes_moved
        cap, tc = pm.capuchin(20)
        assert set(cap) <= {0, 2} and pm.summary.bytes_moved >= ratio * pm.summary.bytes_total
        assert tc >= t - 1e-6
        # longest absence first: the earliest tensors of the chain
        k = sum(1 for p in cap if p)
        assert [i for i, p in enumerate(cap) if p] == list(range(k))
        assert pm.summary.bytes_moved == moved


def test_hand_worked_schedule():
    """Three ops of 1000 us, tensors of 100 MB, link 50 GB/s (2010 us per raw copy
    with the 10 us latency), backward factor 2.  Tensor 0 is consumed by op 1:
    out-copy 2010 - 1000 covered = 1010 exposed; in-copy covered by the backward
    of op 2 (2000): 10 exposed.  Raw overhead 1020 us.  ZFP at rate 8 (25 MB):
    copies of 510 us hide completely; kernels 4 + 100e6/2.1e6 = 51.6 and
    4 + 100e6/1.9e6 = 56.6 us -> 108.2 us."""
    from cswap_amd.planner import PolicyMaker

    c = costs(zfp_compress_gbs=2100.0, zfp_decompress_gbs=1900.0)
    pm = PolicyMaker(c)
    for i in range(3):
        pm.add_comptime(1000.0)
        pm.add_tensor(i, 100_000_000)
        pm.add_stepdep([i - 1, i])
        pm.set_field(i, 100, 100, 2500)
    pm.init(0.3)
    pol, t = pm.make_policy(3)
    assert pol == [6, 0, 0]
    assert t == pytest.approx(9000.0 + 4 + 100e6 / 2.1e6 + 4 + 100e6 / 1.9e6, rel=1e-9)
    cap, tc = pm.capuchin(3)
    assert cap == [2, 0, 0]
    assert tc == pytest.approx(9000.0 + 1010.0 + 10.0, rel=1e-9)
    assert pm.summary.bytes_on_link == 100_000_000


def test_multi_consumer_tensor_leaves_at_its_last_use():
    from cswap_amd.planner import PolicyMaker

    pm = PolicyMaker(costs())
    for i in range(6):
        pm.add_comptime(500.0)
        pm.add_tensor(i, 32 << 20)
        pm.add_stepdep([i - 1, i])
    pm.add_stepdep([1, 4])               # a skip connection: tensor 1 feeds op 2 and op 4
    pm.init(1.0)
    pol, _ = pm.make_policy(6)
    assert pm.begin_stage[1] == 4 and pm.begin_stage[0] == 1
    assert pol[1] != 0 and pol[4] == 0 and pol[5] == 0


def test_argument_errors():
    from cswap_amd._lib import lib

    L = lib()
    p = L.cswap_planner_create(None, 0)
    assert p
    assert L.cswap_planner_init(p, 1.5) == -1 and L.cswap_planner_init(p, -0.1) == -1
    assert L.cswap_planner_add_tensor(p, -1, 10) == -1
    assert L.cswap_planner_add_comptime(p, -1.0) == -1
    assert L.cswap_planner_make_policy(p, None, None, 4, None) == -1
    assert L.cswap_planner_add_stepdep(p, -1, 0) == 0     # untracked input
    L.cswap_planner_destroy(p)


SRC = r"""
#include "cswap_policy_maker.hpp"
#include "cswap_execution.hpp"
#include <stdio.h>
int main() {
  cswap::PolicyMaker pm;
  for (int i = 0; i < 10; i++) {
    pm.add_comptime(400.0);
    pm.add_tensor(i, (size_t)64 << 20);
    pm.add_stepdep({i - 1, i});
  }
  pm.add_omitid(3);
  pm.init(0.4);
  int time_ = 0;
  std::vector<int> policy1 = pm.make_policy(time_, 10);
  int tc = 0;
  std::vector<int> policy2 = pm.capuchin(tc, 10);
  cswap::Execution exe(nullptr);
  exe.init_(10);
  exe.policy = policy1;
  exe.begin_stage = pm.begin_stage();
  int moved = 0;
  for (int p : policy1) moved += p != 0;
  printf("%d %d %d %d\n", time_, tc, moved, policy1[3]);
  return (policy1.size() == 10 && policy1[3] == 0 && moved >= 4 && time_ >= 12000 && tc >= time_) ? 0 : 1;
}
"""


def test_policy_maker_header_compiles_and_plans():
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.cpp")
        exe = os.path.join(d, "t")
        open(src, "w").write(SRC)
        lib = os.path.join(ROOT, "cswap_amd", "libcswap_hip.so")
        subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), src, lib,
                               "-Wl,-rpath," + os.path.dirname(lib), "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib",
                               "-lamdhip64", "-o", exe])
        subprocess.check_call([exe])


def test_backward_factor_scales_the_base_time_and_the_room_to_hide_copies():
    """set_backward_factor: backward of op i takes factor x its forward time.  The
    base time is (1 + factor) x the forward time, and a longer backward hides more
    of every inbound copy, so the planned overhead cannot grow with it."""
    from cswap_amd.planner import PolicyMaker

    over = []
    for factor in (0.5, 1.0, 2.0, 4.0):
        pm = PolicyMaker(costs())
        pm.set_backward_factor(factor)
        vgg_like(pm, comptime=200.0)
        pm.init(0.5)
        pol, t = pm.make_policy(20)
        s = pm.summary
        assert s.base_time_us == pytest.approx(20 * 200.0 * (1.0 + factor))
        assert s.target_met
        over.append(t - s.base_time_us)
    assert all(b <= a + 1e-6 for a, b in zip(over, over[1:])), over
    assert over[0] > over[-1]
