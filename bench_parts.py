"""The measurements of bench.py beyond its headline: drivers that walk the swap engine, the
saved-tensor hooks and the planner over synthetic workloads and time them.  They use the
package as a caller would; nothing in the package imports this file."""
from __future__ import annotations

import time

import torch

from cswap_amd import api, swap
from cswap_amd._lib import Costs
from cswap_amd.hooks import swap_saved_tensors
from cswap_amd.planner import PolicyMaker, run_planned_iteration
from cswap_amd.workloads import dummy_layer_compute, vgg16_modules


def _median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def bench_schedule(dev, batch: int = 128, seed: int = 0) -> dict:
    """Configuration 4: walk the VGG-16 activation schedule; per tensor, swap out (probe + select +
    compress + D2H on the copy stream, overlapped with a dummy compute stream) and back in,
    against the raw (policy 2) swap.  Three arms per tensor, best of five each:
      none        the raw swap
      auto        the selector on a tensor it sees for the first time
      remembered  the selector from the second training iteration on, as the saved-tensor hooks and
                  the Execution mirrors drive it: a remembered ZFP or raw choice is requested outright
                  (no probe), a remembered ZVC choice goes in as CSWAP_POLICY_AUTO_SPARSE (the
                  single-kernel compaction is the probe)
    The latencies are wall clock around the calls; the engine's own phase times (its events) are
    reported beside them for the remembered arm."""
    from cswap_amd.workloads import config4_schedule, config4_tensor

    sched = config4_schedule(batch)
    biggest = max(int(torch.tensor(e["shape"]).prod()) for e in sched) * 4
    eng = swap.SwapEngine(pinned_bytes=2 * biggest + (64 << 20), device_bytes=2 * biggest + (64 << 20), timing=True)
    costs = eng.calibrate()
    a = torch.randn(2048, 2048, device=dev)
    b = torch.randn(2048, 2048, device=dev)
    rows = []
    tot = {"auto": 0.0, "none": 0.0, "remembered": 0.0}
    worst = {"auto": 0.0, "remembered": 0.0}
    for e in sched:
        x = torch.from_numpy(config4_tensor(e, seed)).to(dev)
        out = torch.empty_like(x)
        lat, chosen, phases = {}, None, None
        for label in ("none", "auto", "remembered"):
            if label == "none":
                pol = swap.NONE
            elif label == "auto":
                pol = swap.AUTO
            else:
                pol = swap.AUTO_SPARSE if chosen.policy == swap.SPARSE else chosen.policy
            best = None
            for _ in range(5):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                tk = eng.pre(x, pol)
                dummy_layer_compute(a, b, 2)
                eng.post(tk)
                eng.swap_in(tk, out)
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                info = eng.info(tk)
                tm = eng.timing(tk)
                eng.release(tk)
                if best is None or t1 - t0 < best:
                    best = t1 - t0
                    if label == "remembered":
                        phases = tm
            lat[label] = best * 1e3
            if label == "auto":
                chosen = info
        # dummy compute alone, to report how much of it the swap hides
        torch.cuda.synchronize()
        t0 = time.perf_counter(); dummy_layer_compute(a, b, 2); torch.cuda.synchronize()
        comp_ms = (time.perf_counter() - t0) * 1e3
        rows.append({"id": e["id"], "kind": e["kind"], "shape": list(e["shape"]), "MB": round(x.numel() * 4 / 1e6, 1),
                     "policy": swap.POLICY_NAME[chosen.policy], "ratio": round(chosen.bytes_out / chosen.bytes_in, 4),
                     "none_ms": round(lat["none"], 3), "auto_ms": round(lat["auto"], 3),
                     "remembered_ms": round(lat["remembered"], 3), "compute_ms": round(comp_ms, 3),
                     "engine_us": {"compress": round(phases.compress_us, 1), "copy_out": round(phases.copy_out_us, 1),
                                   "copy_in": round(phases.copy_in_us, 1), "decompress": round(phases.decompress_us, 1)}})
        for k in tot:
            tot[k] += lat[k]
        if chosen.policy != swap.NONE:
            for k in worst:
                worst[k] = max(worst[k], lat[k] / lat["none"])
        del x, out
    eng.close()
    return {"costs": {k: round(getattr(costs, k), 2) for k, _ in Costs._fields_ if k.endswith(("gbs", "us"))},
            "total_none_ms": round(tot["none"], 2), "total_auto_ms": round(tot["auto"], 2),
            "total_remembered_ms": round(tot["remembered"], 2),
            "worst_compressed_over_raw": round(worst["auto"], 3),
            "worst_compressed_over_raw_remembered": round(worst["remembered"], 3), "tensors": rows}


def bench_backward(dev, batch: int = 128, seed: int = 0, compute_reps: int = 2) -> dict:
    """Configuration 4, backward side: every swapped tensor of the schedule is
    already on the host; walk them in reverse (the order backward asks for them),
    each followed by a dummy layer backward on the compute stream.  Compared:
    raw tensors fetched on demand, compressed tensors fetched on demand, and
    compressed tensors with the next one prefetched under the current layer."""
    from cswap_amd.workloads import config4_schedule, config4_tensor

    sched = [e for e in config4_schedule(batch) if e["kind"] != "dense"]   # the swapped ones: ReLU and pool outputs
    total = sum(int(torch.tensor(e["shape"]).prod()) * 4 for e in sched)
    biggest = max(int(torch.tensor(e["shape"]).prod()) for e in sched) * 4
    eng = swap.SwapEngine(pinned_bytes=total + (64 << 20), device_bytes=4 * biggest + (64 << 20))
    eng.calibrate()
    a = torch.randn(2048, 2048, device=dev)
    b = torch.randn(2048, 2048, device=dev)
    xs = [torch.from_numpy(config4_tensor(e, seed)).to(dev) for e in sched]
    outs = [torch.empty_like(x) for x in xs]
    res = {}
    for label, pol, ahead in (("raw_on_demand", swap.NONE, 0), ("compressed_on_demand", swap.AUTO, 0),
                              ("compressed_prefetch_1", swap.AUTO, 1), ("raw_prefetch_1", swap.NONE, 1)):
        best = None
        for _ in range(3):
            tks = []
            for x in xs:
                tk = eng.pre(x, pol)
                eng.post(tk)
                tks.append(tk)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            order = list(range(len(xs)))[::-1]
            if ahead:
                eng.prefetch(tks[order[0]])
            for k, i in enumerate(order):
                if k >= 2:
                    eng.release(tks[order[k - 2]])      # its decompression finished a layer ago
                for j in order[k + 1:k + 1 + ahead]:
                    eng.prefetch(tks[j])
                eng.swap_in(tks[i], outs[i])
                dummy_layer_compute(a, b, compute_reps)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            for i in order[-2:]:
                eng.release(tks[i])
            best = dt if best is None else min(best, dt)
        res[label + "_ms"] = round(best * 1e3, 2)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in xs:
        dummy_layer_compute(a, b, compute_reps)
    torch.cuda.synchronize()
    res["compute_only_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
    res["tensors"] = len(xs)
    res["MB"] = round(total / 1e6, 1)
    eng.close()
    return res


def bench_planner(dev, batch: int = 128, ratio: float = 0.5) -> dict:
    """Profile a VGG-16 forward at 3x64x64, plan with the calibrated cost model,
    run the planned iteration and compare predicted with measured overhead, for
    make_policy and for the raw-swap baseline."""
    import time

    import torch

    
    torch.manual_seed(0)
    mods = vgg16_modules(torch, dev)
    for m in mods:
        m.eval()
    x = torch.randn(batch, 3, 64, 64, device=dev)
    n = len(mods)
    eng = swap.SwapEngine(pinned_bytes=3 << 30, device_bytes=1 << 30)
    costs = eng.calibrate()
    pm = PolicyMaker(costs)
    with torch.no_grad():
        for _ in range(2):                      # warm up kernels and allocator
            t = x
            for m in mods:
                t = m(t)
        t, tid = x, -1
        for i, m in enumerate(mods):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = m(t)
            torch.cuda.synchronize()
            pm.add_comptime((time.perf_counter() - t0) * 1e6)
            pm.add_tensor(i, out.numel() * 4)
            pm.add_stepdep([tid, i])
            nx, ny, nz = swap.field_dims(out.shape)
            pm.set_field(i, nx, ny, nz)
            pm.set_nnz(i, int(api.probe_nnz(out).item()))
            t, tid = out, i
    pm.init(ratio)
    res = {"ratio": ratio, "ops": n}
    none_s = min(run_planned_iteration(eng, mods, x, [0] * n, list(range(1, n + 1))) for _ in range(3))
    res["measured_none_ms"] = round(none_s * 1e3, 2)
    for label, fn in (("make_policy", pm.make_policy), ("capuchin", pm.capuchin)):
        pol, t_us = fn(n)
        s = pm.summary
        best = min(run_planned_iteration(eng, mods, x, pol, pm.begin_stage) for _ in range(3))
        res[label] = {"policy": pol, "predicted_overhead_ms": round((t_us - s.base_time_us) / 1e3, 2),
                      "measured_overhead_ms": round((best - none_s) * 1e3, 2),
                      "moved_MB": round(s.bytes_moved / 1e6, 1), "link_MB": round(s.bytes_on_link / 1e6, 1),
                      "selected": s.n_selected}
    res["base_predicted_ms"] = round(pm.summary.base_time_us / 1e3, 2)
    eng.close()
    pm.close()
    return res


def _measure_step(step, params, make_ctx, reps=5):
    """Median and best wall time of ``step(ctx)`` over ``reps`` runs after two warm-up
    runs (a step whose copies overlap compute differently from run to run has a
    spread worth showing), the step's peak in torch's allocator above what is
    allocated before it, and the hook statistics of the last run."""
    import time

    for _ in range(2):
        step(make_ctx())
    for p in params:
        p.grad = None
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()     # weights, input and whatever else the process holds
    torch.cuda.reset_peak_memory_stats()
    times = []
    stats = None
    for _ in range(reps):
        ctx = make_ctx()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step(ctx)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) * 1e3)
        stats = ctx.stats if ctx is not None else None
    times.sort()
    return (times[len(times) // 2], times[0]), (torch.cuda.max_memory_allocated() - base) / 1e6, stats


def _swap_rows(res, eng, step, params, min_bytes, reps):
    memo = {}        # the selector's decisions, kept across the iterations of the last row
    for label, pol, kw in (("raw_swap", swap.NONE, {}), ("selector", swap.AUTO, {}),
                           ("selector_remembered", swap.AUTO, {"memo": memo})):
        ms, mb, st = _measure_step(step, params,
                                   lambda: swap_saved_tensors(eng, policy=pol, min_bytes=min_bytes, **kw), reps)
        res[label] = {"step_ms": round(ms[0], 2), "step_ms_best": round(ms[1], 2), "step_peak_MB": round(mb, 1),
                      "swapped_tensors": st["swapped"],
                      "swapped_MB": round(st["bytes_in"] / 1e6, 1), "link_MB": round(st["bytes_out"] / 1e6, 1),
                      "shared": st["shared"], "by_policy": dict(st.get("by_policy", {})),
                      "prefetched": st.get("prefetched", 0), "resident": st.get("resident", 0),
                      "kept_no_room": st.get("kept_no_room", 0), "memo_hits": st.get("memo_hits", 0),
                      "memo_sparse": st.get("memo_sparse", 0)}


def bench_training_step(dev, batch: int = 128, image: int = 64, min_bytes: int = 8 << 20) -> dict:
    """Forward + backward of a VGG-16 (conv/BN/ReLU x13, 5 pools, linear head) on
    random data with and without activation swapping through the saved-tensor
    hooks: step time and peak device memory of the step (torch's allocator, above
    what is allocated before the step).  Stock autograd, nothing patched."""

    

    torch.manual_seed(0)
    feats = torch.nn.Sequential(*vgg16_modules(torch, dev))
    head = torch.nn.Linear(512 * (image // 32) ** 2, 10).to(dev)
    x = torch.randn(batch, 3, image, image, device=dev)
    params = list(feats.parameters()) + list(head.parameters())

    def step(ctx):
        for p in params:
            p.grad = None
        if ctx is None:
            loss = head(feats(x).flatten(1)).square().mean()
        else:
            with ctx:
                loss = head(feats(x).flatten(1)).square().mean()
        loss.backward()
        if ctx is not None:
            ctx.close()
        return loss

    res = {"model": f"VGG-16 BN, batch {batch}, 3x{image}x{image}", "min_bytes": min_bytes}
    base_ms, base_mb, _ = _measure_step(step, params, lambda: None)
    res["no_swap"] = {"step_ms": round(base_ms[0], 2), "step_peak_MB": round(base_mb, 1)}
    staging = 192 << 20
    eng = swap.SwapEngine(pinned_bytes=4 << 30, device_bytes=staging)
    eng.calibrate()
    res["staging_pool_MB"] = round(staging / 1e6, 1)    # device memory the engine holds besides torch's allocator
    _swap_rows(res, eng, step, params, min_bytes, 9)
    eng.close()
    return res


def bench_transformer_step(dev, layers: int = 4, batch: int = 32, seq: int = 512, hidden: int = 768, heads: int = 12,
                           min_bytes: int = 8 << 20) -> dict:
    """Forward + backward of a BERT-base-shaped encoder stack (attention written
    out, so the [batch, heads, seq, seq] probabilities are saved as in
    configuration 5; GELU feed-forward of 4 x hidden) with and without swapping
    through the saved-tensor hooks.  No ReLU anywhere: the selector has only ZFP
    and raw to choose from."""
    import math

    torch.manual_seed(0)

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.qkv = torch.nn.Linear(hidden, 3 * hidden)
            self.proj = torch.nn.Linear(hidden, hidden)
            self.ln1 = torch.nn.LayerNorm(hidden)
            self.ln2 = torch.nn.LayerNorm(hidden)
            self.fc1 = torch.nn.Linear(hidden, 4 * hidden)
            self.fc2 = torch.nn.Linear(4 * hidden, hidden)

        def forward(self, x):
            b, s, h = x.shape
            q, k, v = self.qkv(self.ln1(x)).view(b, s, 3, heads, h // heads).permute(2, 0, 3, 1, 4)
            p = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(h // heads), dim=-1)
            x = x + self.proj((p @ v).transpose(1, 2).reshape(b, s, h))
            return x + self.fc2(torch.nn.functional.gelu(self.fc1(self.ln2(x))))

    net = torch.nn.Sequential(*[Block() for _ in range(layers)]).to(dev)
    x = torch.randn(batch, seq, hidden, device=dev)
    params = list(net.parameters())

    def step(ctx):
        for p in params:
            p.grad = None
        if ctx is None:
            loss = net(x).square().mean()
        else:
            with ctx:
                loss = net(x).square().mean()
        loss.backward()
        if ctx is not None:
            ctx.close()

    res = {"model": f"{layers} encoder blocks, batch {batch}, seq {seq}, hidden {hidden}, {heads} heads",
           "min_bytes": min_bytes}
    ms, mb, _ = _measure_step(step, params, lambda: None, 5)
    res["no_swap"] = {"step_ms": round(ms[0], 2), "step_peak_MB": round(mb, 1)}
    staging = 768 << 20
    eng = swap.SwapEngine(pinned_bytes=12 << 30, device_bytes=staging)
    eng.calibrate()
    res["staging_pool_MB"] = round(staging / 1e6, 1)
    _swap_rows(res, eng, step, params, min_bytes, 9)
    eng.close()
    return res
