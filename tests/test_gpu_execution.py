"""The Execution mirror on a VGG-16-shaped forward walk with the policy vector of
the reference driver (ZVC for ReLU outputs, ZFP for pooled outputs,
CSWAP+/vgg16-cifar10.cpp:177-178 and the commented mix at :393-394)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_vgg_walk_with_reference_policy_vector():
    import torch

    import oracle
    from cswap_amd import swap
    from cswap_amd.execution import ACT, Execution

    assert torch.cuda.is_available()
    torch.manual_seed(0)
    # first 14 ops of VGG-16 (types as in vgg16-cifar10.cpp:177-178), small batch
    ops = [("conv", 3, 64), ("bn", 64), ("relu",), ("conv", 64, 64), ("bn", 64), ("relu",), ("pool",),
           ("conv", 64, 128), ("bn", 128), ("relu",), ("conv", 128, 128), ("bn", 128), ("relu",), ("pool",)]
    mods = []
    for o in ops:
        if o[0] == "conv":
            mods.append(torch.nn.Conv2d(o[1], o[2], 3, padding=1).cuda())
        elif o[0] == "bn":
            mods.append(torch.nn.BatchNorm2d(o[1]).cuda())
        elif o[0] == "relu":
            mods.append(torch.nn.ReLU())
        else:
            mods.append(torch.nn.MaxPool2d(2))
    eng = swap.SwapEngine(pinned_bytes=512 << 20, device_bytes=512 << 20)
    exe = Execution(eng)
    exe.init_(50)
    for i in (2, 9):
        exe.policy[i] = 3        # ReLU outputs feeding a conv: ZVC
    for i in (6, 13):
        exe.policy[i] = 6        # pool outputs: ZFP
    exe.policy[5] = 2            # one raw swap (vDNN style)
    exe.policy[12] = -1          # and one left to the selector

    x = torch.randn(32, 3, 64, 64, device="cuda")
    kept = {}
    with torch.no_grad():
        exe.preforward()
        pre, pre_id = x, -1
        for m in mods:
            exe.pre(pre, pre_id, ACT)
            out = m(pre)
            out_id = exe.post()
            if exe.swapped(pre_id):
                kept[pre_id] = pre.clone()     # what the device copy held when it was swapped out
            pre, pre_id = out, out_id
        # the consumer of the last tensor (the next conv in the real model)
        exe.pre(pre, pre_id, ACT)
        exe.post()
        if exe.swapped(pre_id):
            kept[pre_id] = pre.clone()
        exe.postforward()
    assert exe.index == len(mods)
    assert sorted(kept) == [2, 5, 6, 9, 12, 13]
    assert exe.com_and_tran(2) == 3 and exe.com_and_tran(6) == 6 and exe.com_and_tran(5) == 2
    assert exe.com_and_tran(12) in (2, 3, 6) and exe.com_and_tran(0) == 0

    order = sorted(kept, reverse=True)           # backward order
    for k, tid in enumerate(order):
        tag = exe.com_and_tran(tid)
        if k + 1 < len(order):
            exe.prefetch(order[k + 1])           # the next one comes in under this layer's backward
        back = exe.fetch(tid)
        torch.cuda.synchronize()
        ref = kept[tid]
        if tag == 6:
            f = ref.cpu().numpy().reshape(-1, ref.shape[-2], ref.shape[-1])
            want = oracle.zfp_decode3(oracle.zfp_encode3(f, 512, omp=True), f.shape, 512, omp=True)
            assert np.array_equal(back.cpu().numpy().reshape(f.shape).view(np.uint32), want.view(np.uint32))
        else:
            assert torch.equal(back, ref)
        assert not exe.swapped(tid)
    eng.close()


def test_op_with_several_inputs_swaps_each_under_its_own_policy():
    """Vector form of pre/post (Execution.h:135-212,311-401): a residual add whose
    two inputs are both consumed by that op, one as ZVC and one as ZFP, plus an
    untracked third input."""
    import torch

    import oracle
    from cswap_amd import swap
    from cswap_amd.execution import ACT, Execution

    torch.manual_seed(1)
    eng = swap.SwapEngine(pinned_bytes=256 << 20, device_bytes=256 << 20)
    exe = Execution(eng)
    exe.init_(8)
    exe.policy[0] = 3
    exe.policy[1] = 6
    exe.begin_stage[0] = 2            # both are consumed by op 2, the add
    exe.begin_stage[1] = 2
    a = torch.relu(torch.randn(16, 64, 32, 32, device="cuda"))      # output of op 0
    b = torch.randn(16, 64, 32, 32, device="cuda")                  # output of op 1
    c = torch.randn(16, 64, 32, 32, device="cuda")                  # not tracked
    exe.preforward()
    exe.pre(a, -1); exe.post()        # op 0
    exe.pre(a, -1); exe.post()        # op 1
    exe.pre([(a, 0), (b, 1), (c, -1)], layer_type=ACT)              # op 2
    s = a + b + c
    assert exe.post() == 2
    exe.postforward()
    assert exe.swapped(0) and exe.swapped(1) and exe.com_and_tran(0) == 3 and exe.com_and_tran(1) == 6
    exe.prefetch(0)
    back_b = exe.fetch(1)
    back_a = exe.fetch(0)
    torch.cuda.synchronize()
    assert torch.equal(back_a, a)
    f = b.cpu().numpy().reshape(-1, 32, 32)
    want = oracle.zfp_decode3(oracle.zfp_encode3(f, 512, omp=True), f.shape, 512, omp=True)
    assert np.array_equal(back_b.cpu().numpy().reshape(f.shape).view(np.uint32), want.view(np.uint32))
    assert torch.equal(s, a + b + c)
    eng.close()


def test_planned_iteration_restores_every_swapped_tensor():
    """Profile -> make_policy -> Execution walk with prefetch: every tensor the plan
    moved comes back as its codec round trip (lossless actions: bit-identical)."""
    import torch

    from cswap_amd import api, swap
    from cswap_amd.planner import PolicyMaker, run_planned_iteration
    from cswap_amd.workloads import vgg16_modules

    torch.manual_seed(0)
    dev = torch.device("cuda")
    mods = [m.eval() for m in vgg16_modules(torch, dev)][:17]
    x = torch.randn(16, 3, 64, 64, device=dev)
    costs = swap.default_costs()
    costs.allow_lossy = 0
    costs.size_floor_bytes = 0
    pm = PolicyMaker(costs)
    with torch.no_grad():
        t, tid = x, -1
        for i, m in enumerate(mods):
            out = m(t)
            pm.add_comptime(100.0)
            pm.add_tensor(i, out.numel() * 4)
            pm.add_stepdep([tid, i])
            pm.set_nnz(i, int(api.probe_nnz(out).item()))
            t, tid = out, i
    pm.init(0.6)
    pol, _ = pm.make_policy(len(mods))
    assert 3 in pol and 2 in pol and 6 not in pol
    eng = swap.SwapEngine(pinned_bytes=1 << 30, device_bytes=512 << 20)
    seen, kept = [], {}

    def check(tid, back):
        seen.append(tid)
        assert torch.equal(back, kept[tid]), tid

    run_planned_iteration(eng, mods, x, pol, pm.begin_stage, check=check, keep=kept)
    assert sorted(seen) == [i for i, p in enumerate(pol) if p]
    eng.close()
    pm.close()


def test_cpp_driver_with_policy_maker_and_execution():
    """tests/cpp_schedule_walk.cpp: a driver in the style of the reference's model
    files, written against the two header-only mirrors and the C ABI only (no
    Python, no torch): calibrate, plan most of the activation bytes with
    cswap::PolicyMaker, walk forward with cswap::Execution::pre/post, walk backward
    with prefetch/fetch, and compare every tensor that comes back byte for byte."""
    out = _build_and_run_cpp("cpp_schedule_walk")
    assert out.returncode == 0, out.stdout
    tag, swapped, link = out.stdout.split()[-3:]
    assert tag == "OK" and int(swapped) >= 3 and int(link) > 0
    policy = [int(v) for v in out.stdout.split("policy:")[1].split("OK")[0].split()]
    assert 3 in policy and 2 in policy                       # ZVC for the ReLU-like tensors, raw for the (de-ZFP-ed) dense ones


def _build_and_run_cpp(name, timeout=100):
    import os
    import subprocess
    import tempfile

    from conftest import ROOT

    src = os.path.join(ROOT, "tests", name + ".cpp")
    lib = os.path.join(ROOT, "cswap_amd", "libcswap_hip.so")
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, name)
        subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"),
                               "-I/opt/rocm/include", src, lib, "-Wl,-rpath," + os.path.dirname(lib),
                               "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib", "-lamdhip64", "-o", exe])
        out = subprocess.run([exe], capture_output=True, text=True, timeout=timeout)
    print(out.stdout, out.stderr, flush=True)
    return out


def test_cpp_selector_memo_skips_the_probe_for_remembered_decisions():
    """tests/cpp_selector_memo.cpp: with policy[] = -1 the C++ mirror asks the
    selector in the first iteration and reuses a ZFP or raw decision afterwards
    without the counting pass and its host round trip (Execution.h:89-92), until
    `recheck` reuses are spent; a ZVC tensor is probed every time."""
    out = _build_and_run_cpp("cpp_selector_memo")
    assert out.returncode == 0, out.stdout
    assert out.stdout.split()[-6:] == ["OK", "2", "1", "1", "2", "1"]


def test_python_mirror_selector_memo_and_global_modes():
    """The Python twin: the same memo, and the reference's global modes -- under
    policy_ = 3 (vDNN) every input of a convolution goes out raw whatever its
    entry says, under policy_ = 4 (SuperNeurons) everything else is dropped
    (Execution.h:70,243)."""
    import torch

    from cswap_amd import swap
    from cswap_amd.execution import ACT, CONV, Execution

    eng = swap.SwapEngine(pinned_bytes=256 << 20, device_bytes=256 << 20)
    dense = torch.randn(64, 64, 32, 32, device="cuda")
    relu = torch.relu(torch.randn(64, 64, 32, 32, device="cuda") - 0.6)
    exe = Execution(eng)
    exe.init_(4)
    exe.policy = [-1, -1, 0, 0]
    exe.recheck = 3
    per_iter = []
    for _ in range(3):
        before = eng.probe_count()
        exe.preforward()
        exe.pre(dense, -1); exe.post()
        exe.pre(dense, 0); exe.post()
        exe.pre(relu, 1); exe.post()
        exe.postforward()
        per_iter.append(eng.probe_count() - before)
        assert exe.com_and_tran(0) == swap.ZFP and exe.com_and_tran(1) == swap.SPARSE
        back = exe.fetch(1)
        assert torch.equal(back, relu)
        assert float((exe.fetch(0) - dense).abs().max()) < 0.5
    assert per_iter == [2, 1, 1] and exe.memo_hits == 2

    # global modes
    exe = Execution(eng)
    exe.init_(4)
    exe.policy = [3, 6, 2, 0]
    exe.policy_ = 3
    exe.preforward()
    exe.pre(dense, -1, CONV); exe.post()
    exe.pre(relu, 0, CONV); exe.post()          # entry 3, but a convolution consumes it under vDNN: raw
    exe.pre(dense, 1, ACT); exe.post()          # entry 6, consumer is not a convolution: ZFP as written
    assert exe.com_and_tran(0) == 2 and exe.com_and_tran(1) == 6
    assert torch.equal(exe.fetch(0), relu)
    exe.fetch(1)
    exe.policy_ = 4
    exe.preforward()
    exe.pre(dense, -1, CONV); exe.post()
    exe.pre(relu, 0, ACT); exe.post()           # SuperNeurons: not a convolution input -> dropped
    exe.pre(dense, 1, CONV); exe.post()         # convolution input -> raw swap
    exe.pre(relu, 2, ACT); exe.post()           # entry 2, still dropped: the drop branch comes first
    assert exe.com_and_tran(0) == 1 and exe.dropped(0) and not exe.swapped(0)
    assert exe.com_and_tran(1) == 2 and exe.com_and_tran(2) == 1
    assert torch.equal(exe.fetch(1), dense)
    with pytest.raises(KeyError):
        exe.fetch(0)                            # nothing to bring back: the caller recomputes it
    eng.close()
