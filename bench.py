#!/usr/bin/env python3
"""Benchmark of the compression-before-swap hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one synthetic batch: ZFP fixed-rate
8 bits/value compress followed by decompress of the BERT-base attention
probability tensor fp32 [32,12,512,512] (402,653,184 B; the >=256 MB tensor the
throughput target is quoted on), already resident in HBM.  ``value`` is GB/s of
uncompressed fp32 pushed through the compress+decompress pair:
4*N bytes / (t_compress + t_decompress).

Before the W warm-up steps the same step runs, untimed, for CLOCK_SETTLE_S
seconds: after an idle gap the GPU needs about 25 ms of continuous work to
return to its steady clocks, and a training loop never leaves it idle.

The last line of stdout is ONE short JSON object (cut to 1480 characters if need be: fit_line) that
also carries
  roofline      HBM-roofline figures of the dominant (slower) ZFP kernel, from
                HIP-event timing of that kernel inside the timed region (events
                around both kernels of every few steps)
  cpu_baseline  the CPU checker (a port of the reference algorithm) timed on a
                bounded sample of the same tensor on this host
  also          a handful of roofline fractions of the other kernels of the path.
Everything else that is measured (ZVC compact/expand, probe, other rates and
tensors, swap latency, the training steps, the per-kernel details of the two
objects above) goes to the file named by ``extra_file`` -- reported, not the
headline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the two ZFP kernels on this workload, from two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE), each scaled by what the counter reads for a plain copy of the same tensor
# (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000); the summary of those runs is kept under profiles/
HBM_TRAFFIC_BYTES_PER_LAUNCH = {"zfp_encode3_f32_kernel": 503500800, "zfp_decode3_f32_kernel": 503787520}
ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


# After an idle gap of more than a few milliseconds the GPU's clocks take about
# 25 ms of continuous work to come back to their steady level (the first
# hundred launches of a 0.12 ms kernel run 10-30 % slow).  A training loop keeps
# the GPU busy, so every figure here is taken in that steady state: the
# workload itself is run, untimed, for this long before the warm-up steps.
CLOCK_SETTLE_S = 0.3


def settle(torch, fn, seconds):
    """Run fn() back to back, untimed, for about ``seconds`` of GPU time."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(16):
            fn()
        torch.cuda.synchronize()


def ev_ms(torch, fn, reps, settle_s=0.03):
    """Average duration of fn() in ms from HIP events on the current stream,
    after ``settle_s`` seconds of the same work."""
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    settle(torch, fn, settle_s)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) / reps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--extra-file", default=os.path.join(ROOT, "gpurun_out", "bench_extra.json"),
                    help="where the figures beyond the headline line are written")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one plain copy kernel of the same tensor (known traffic: 4N read, 4N "
                         "written) so that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE can be scaled")
    ap.add_argument("--swap-only", action="store_true",
                    help="run only the swap schedule of configuration 4 and its backward walk (for profiling)")
    ap.add_argument("--zvc-only", action="store_true",
                    help="run only one ReLU zero-value-compaction case (for profiling); prints its figures")
    ap.add_argument("--zvc-mib", type=int, default=256, help="size of the --zvc-only tensor in MiB")
    ap.add_argument("--zfp-only", choices=sorted(ZFP_ONLY_CASES),
                    help="run only the ZFP kernels on one of the smaller workloads, each in a loop of its own "
                         "(for profiling); prints its figures")
    ap.add_argument("--zfp-form", choices=["shipped", "lane", "pair"], default="shipped",
                    help="with --zfp-only: the kernel form, as shipped (by field size), one lane per block, "
                         "or the pair form wherever the shape allows")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is built and measured on ONE GPU; run with --gpus 1 "
              "(blocks and chunks are independent, so it would shard by splitting the field along nz "
              "or the tensor by chunk ranges, with no exchange)", file=sys.stderr)
        sys.exit(2)

    import torch

    from cswap_amd import api
    from cswap_amd.workloads import CONFIG5_SHAPES, config5_tensor_torch, field_dims

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.zvc_only:
        print(json.dumps(extras(torch, api, dev, zvc_only=args.zvc_mib)))
        return
    if args.zfp_only:
        print(json.dumps(zfp_only(torch, api, dev, args.zfp_only, args.zfp_form)))
        return
    if args.swap_only:
        import bench_parts
        print(json.dumps({"swap": bench_parts.bench_schedule(dev), "swap_backward": bench_parts.bench_backward(dev)}))
        return

    rate = 8
    maxbits = 64 * rate
    name = "attn_softmax"
    x = config5_tensor_torch(name, dev, seed=0)
    n = x.numel()
    nx, ny, nz = field_dims(x.shape)
    stream = torch.empty(api.zfp_stream_capacity(nx, ny, nz, maxbits), dtype=torch.uint8, device=dev)
    out = torch.empty_like(x)

    def step():
        api.cuda_compress(x, maxbits, out=stream)
        api.cuda_decompress(stream, x.shape, maxbits, out=out)

    if args.copy_probe:
        out.copy_(x)
        torch.cuda.synchronize()
    # the events of the timed region exist before the GPU is brought to its steady
    # clocks, so that nothing but a synchronize separates the warm-up from the timed steps
    # an event record costs about 4 us of GPU time between two launches, so only every
    # `stride`-th step of the timed region carries the events that time its two kernels
    stride = max(1, min(10, args.steps // 5))
    sampled = list(range(0, args.steps, stride))
    evs = {k: [torch.cuda.Event(enable_timing=True) for _ in range(3)] for k in sampled}
    settle(torch, step, CLOCK_SETTLE_S)
    for _ in range(args.warmup):
        step()

    # ---- timed region: exactly K steps, per-kernel HIP events inside it
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        e = evs.get(k)
        if e is None:
            api.cuda_compress(x, maxbits, out=stream)
            api.cuda_decompress(stream, x.shape, maxbits, out=out)
        else:
            e[0].record()
            api.cuda_compress(x, maxbits, out=stream)
            e[1].record()
            api.cuda_decompress(stream, x.shape, maxbits, out=out)
            e[2].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    enc_ms = sum(e[0].elapsed_time(e[1]) for e in evs.values()) / len(evs)
    dec_ms = sum(e[1].elapsed_time(e[2]) for e in evs.values()) / len(evs)
    value = 4.0 * n / (ms_per_step * 1e-3) / 1e9

    bytes_per_value = 4.0 + rate / 8.0          # read 4 B, write rate/8 B (or the reverse)
    dom = "zfp_encode3_f32_kernel" if enc_ms >= dec_ms else "zfp_decode3_f32_kernel"
    dom_ms = max(enc_ms, dec_ms)
    achieved = bytes_per_value * n / (dom_ms * 1e-3) / 1e9

    def frac(ms):
        return round(bytes_per_value * n / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)

    roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": HBM_TRAFFIC_BYTES_PER_LAUNCH.get(dom),
                "algorithmic_bytes_per_launch": int(bytes_per_value * n), "avg_launch_ms": round(dom_ms, 4),
                "compress_frac": frac(enc_ms), "decompress_frac": frac(dec_ms)}

    result = {
        "metric": "compress+decompress GB/s (fp32 in), ZFP fixed-rate 8 bits/value, 1xMI355X",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp32", "data": "synthetic",
        "config": {"workload": "config5 attention probabilities fp32 [32,12,512,512]=softmax(N(0,1)), "
                               "field 512x512x384, rate 8, compress then decompress",
                   "bytes_in": 4 * n},
        "roofline": roofline,
    }
    detail = {"clock_settle_s": CLOCK_SETTLE_S, "kernel_event_samples": len(evs),
              "compress_ms": round(enc_ms, 4), "decompress_ms": round(dec_ms, 4)}

    if not args.no_cpu:
        cb = cpu_baseline(x, maxbits)
        detail["cpu_baseline"] = cb
        result["cpu_baseline"] = {k: cb[k] for k in ("value", "unit", "cores", "kind", "sample")}
    if not args.no_extra:
        ex = extras(torch, api, dev, cpu=not args.no_cpu)
        detail["extra"] = ex
        result["also"] = headline_fractions(ex)
    if not args.no_extra or not args.no_cpu:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.extra_file)), exist_ok=True)
            with open(args.extra_file, "w") as fh:
                json.dump(dict(result, **detail), fh, indent=1)
            result["extra_file"] = os.path.relpath(args.extra_file, ROOT)
        except OSError as err:      # a read-only tree: the figures above are still printed
            print(f"bench.py: could not write {args.extra_file}: {err}", file=sys.stderr)
    print(fit_line(result))


LINE_LIMIT = 1480   # characters; the driver keeps a 2000-character tail of stdout


def fit_line(result, limit=LINE_LIMIT):
    """The result as one JSON line of at most `limit` characters.  What does not fit goes,
    least important first: the name of the file with the rest of the figures when it is a
    long path, then the entries of `also` from its end; the contract's own keys always stay.
    (Everything dropped here is still in that file.)"""
    line = json.dumps(result)
    if len(line) <= limit:
        return line
    result = dict(result)
    if len(str(result.get("extra_file", ""))) > 40:
        result["extra_file"] = os.path.basename(result["extra_file"])
    also = dict(result.get("also") or {})
    while len(json.dumps(result)) > limit and also:
        also.popitem()
        result["also"] = also
    if not also:
        result.pop("also", None)
    return json.dumps(result)


def zfp_cold_pair(torch, api, t, rate, copies, reps):
    """[compress, decompress] in ms with nothing of a launch's operands left in the memory-side
    cache (256 MB) from the launches before it: the loop rotates over `copies` separate fields,
    streams and outputs, so that between two uses of a buffer more than the cache's size in
    other traffic has gone by.  A timing loop over one tensor re-reads what the previous launch
    left behind; in a swap the encoder's field was written by the producing layer a while ago
    and the decoder's stream has just come over the link."""
    from cswap_amd.workloads import field_dims

    nx, ny, nz = field_dims(t.shape)
    mb = 64 * rate
    fields = [t] + [t.clone() for _ in range(copies - 1)]
    streams = [torch.empty(api.zfp_stream_capacity(nx, ny, nz, mb), dtype=torch.uint8, device=t.device)
               for _ in range(copies)]
    outs = [torch.empty_like(t) for _ in range(copies)]
    for f, s_ in zip(fields, streams):
        api.cuda_compress(f, mb, out=s_)
    state = {"i": 0}

    def enc():
        k = state["i"] % copies
        state["i"] += 1
        api.cuda_compress(fields[k], mb, out=streams[k])

    def dec():
        k = state["i"] % copies
        state["i"] += 1
        api.cuda_decompress(streams[k], t.shape, mb, out=outs[k])

    return ev_ms(torch, enc, reps), ev_ms(torch, dec, reps)


# --zfp-only: name -> (what it is, rate)
ZFP_ONLY_CASES = {"config1": ("config 1, PReLU(N(0,1)) fp32 [64,64,32,32], 16.8 MB", 8),
                  "config3_34MB": ("config 3, fp32 [128,64,32,32], 33.6 MB", 8),
                  "hidden50MB": ("config 5, GELU(N(0,1)) fp32 [32,512,768], 50.3 MB", 8),
                  "ffn201MB_r16": ("config 5, GELU(N(0,1)) fp32 [32,512,3072], 201.3 MB, 16 bits per value", 16)}


def zfp_only(torch, api, dev, name, form):
    """One of the smaller ZFP workloads, compress and decompress each in a loop of its own."""
    import ctypes as C

    from cswap_amd._lib import lib
    from cswap_amd.workloads import config1_field, config3_fields, config5_tensor_torch, field_dims

    if form != "shipped":
        big = C.c_size_t(-1).value
        lib().cswap_zfp_set_pair_bytes(big if form == "pair" else 0, big if form == "pair" else 0, None)
    what, rate = ZFP_ONLY_CASES[name]
    if name == "config1":
        t = torch.from_numpy(config1_field()).to(dev)
    elif name == "config3_34MB":
        t = torch.from_numpy(config3_fields(batch=128)["64x32x32"]).to(dev)
    else:
        t = config5_tensor_torch("hidden_gelu" if name == "hidden50MB" else "ffn_gelu", dev, seed=0)
    n = t.numel()
    nx, ny, nz = field_dims(t.shape)
    mb = 64 * rate
    s = torch.empty(api.zfp_stream_capacity(nx, ny, nz, mb), dtype=torch.uint8, device=dev)
    o = torch.empty_like(t)
    api.cuda_compress(t, mb, out=s); api.cuda_decompress(s, t.shape, mb, out=o)
    e = ev_ms(torch, lambda: api.cuda_compress(t, mb, out=s), 2000, settle_s=0.1)
    d = ev_ms(torch, lambda: api.cuda_decompress(s, t.shape, mb, out=o), 2000, settle_s=0.1)
    bpv = 4 + rate / 8
    return {"workload": what, "form": form, "rate": rate, "compress_us": round(e * 1e3, 2), "decompress_us": round(d * 1e3, 2),
            "compress_hbm_frac": round(bpv * n / e / 1e6 / HBM_PEAK_GBS, 4),
            "decompress_hbm_frac": round(bpv * n / d / 1e6 / HBM_PEAK_GBS, 4)}


def headline_fractions(ex):
    """A few fractions of the 8 TB/s HBM roofline (algorithmic bytes) picked from
    the extra figures, short enough for the one-line record:
    [compress, decompress] for ZFP, [count+scan+compact, expand] for ZVC."""
    def pick(key, a, b):
        row = ex.get(key)
        return [round(row[a], 3), round(row[b], 3)] if row and a in row else None

    also = {
        "zfp_r16_attn402MB": pick("zfp_attn_402MB_r16", "compress_hbm_frac", "decompress_hbm_frac"),
        "zfp_r8_ffn201MB": pick("zfp_config5_ffn_gelu_r8", "compress_hbm_frac", "decompress_hbm_frac"),
        "zfp_r8_hidden50MB": pick("zfp_config5_hidden_gelu_r8", "compress_hbm_frac", "decompress_hbm_frac"),
        "zfp_r8_c3_34MB": pick("zfp_config3_64x32x32_r8", "compress_hbm_frac", "decompress_hbm_frac"),
        "zfp_r8_c1_16MB": pick("zfp_config1_16MB_r8", "compress_hbm_frac", "decompress_hbm_frac"),
        # the same three tensors with every launch's operands cold in the memory-side cache
        "cold": {k: v for k, v in (("attn402MB", pick("zfp_attn_402MB_r8", "compress_hbm_frac_cold", "decompress_hbm_frac_cold")),
                                   ("ffn201MB", pick("zfp_config5_ffn_gelu_r8", "compress_hbm_frac_cold", "decompress_hbm_frac_cold")),
                                   ("hidden50MB", pick("zfp_config5_hidden_gelu_r8", "compress_hbm_frac_cold", "decompress_hbm_frac_cold")))
                 if v is not None} or None,
        "zvc_256MiB": pick("zvc_relu_256MiB", "compress_total_hbm_frac", "expand_hbm_frac"),
        "zvc_512MiB": pick("zvc_relu_512MiB", "compress_total_hbm_frac", "expand_hbm_frac"),
        "zvc_c2_50pct": pick("zvc_config2_s50", "compress_total_hbm_frac", "expand_hbm_frac"),
    }
    zc = (ex.get("zvc_relu_256MiB") or {}).get("cpu_baseline")
    if zc:     # the CPU sparse path on the 256 MiB tensor, one core: [compress, expand] GB/s of fp32
        also["zvc_256MiB_cpu_GBs"] = [zc["one_core"]["compress_GBs_fp32"], zc["one_core"]["expand_GBs_fp32"]]
    if ex.get("box_memory_GBs"):
        also["box_copy_GBs"] = ex["box_memory_GBs"]["copy_read_plus_write"]
    sw = ex.get("swap")
    if sw and "total_none_ms" in sw:
        # sums over the 44 tensors: raw, selector on first sight, selector with remembered decisions; and the
        # largest compressed / raw latency ratio among the tensors the selector compressed (target: below 1)
        also["swap_c4_ms"] = {"raw": sw["total_none_ms"], "auto": sw["total_auto_ms"],
                              "memo": sw["total_remembered_ms"], "worst_vs_raw": sw["worst_compressed_over_raw"]}
    # most important first: fit_line() drops from the end when the line would get too long
    order = ["zfp_r8_c1_16MB", "zfp_r8_c3_34MB", "zfp_r8_hidden50MB", "zfp_r8_ffn201MB", "cold", "swap_c4_ms",
             "zvc_256MiB", "zvc_512MiB", "zvc_c2_50pct", "zfp_r16_attn402MB", "box_copy_GBs", "zvc_256MiB_cpu_GBs"]
    return {k: also[k] for k in order if also.get(k) is not None}


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def cpu_baseline(x, maxbits):
    """The CPU checker (port of the reference algorithm) on the whole tensor of
    the workload: compress + decompress, one warm-up and the median of five runs
    (about 15 s of CPU work on one core), then the same on all cores."""
    import oracle

    sample = x.cpu().numpy().reshape(-1, x.shape[-2], x.shape[-1])
    nbytes = sample.nbytes

    def pair(omp, runs):
        times = []
        for i in range(runs + 1):
            t0 = time.perf_counter()
            s = oracle.zfp_encode3(sample, maxbits, omp=omp)
            t1 = time.perf_counter()
            oracle.zfp_decode3(s, sample.shape, maxbits, omp=omp)
            t2 = time.perf_counter()
            if i:                                  # the first run is the warm-up
                times.append((t2 - t0, t1 - t0, t2 - t1))
        return tuple(median([t[j] for t in times]) for j in range(3))

    ser = pair(False, 5)
    par = pair(True, 5)
    threads = oracle.lib(True).orc_threads()
    res = {"value": round(nbytes / ser[0] / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": "the whole 402.7 MB tensor, compress+decompress, 1 warm-up + median of 5",
           "compress_GBs": round(nbytes / ser[1] / 1e9, 4), "decompress_GBs": round(nbytes / ser[2] / 1e9, 4),
           "all_cores": {"value": round(nbytes / par[0] / 1e9, 4), "cores": threads}}
    z = zfp_library_pair(sample, maxbits)
    if z is not None:
        res["zfp_0_5_5_library"] = {"value": round(nbytes / z[0] / 1e9, 4), "cores": 1,
                                    "compress_GBs": round(nbytes / z[1] / 1e9, 4),
                                    "decompress_GBs": round(nbytes / z[2] / 1e9, 4),
                                    "note": "stock serial codec of the image, same tensor, best of 3"}
    return res


def zfp_library_pair(sample, maxbits):
    """The stock zfp 0.5.5 serial codec (the version the reference snapshots), if
    this machine has the library: (pair, compress, decompress) seconds, best of 3."""
    import ctypes as C

    import numpy as np

    path = "/opt/conda/lib/libzfp.so.0.5.5"
    if not os.path.exists(path):
        return None
    try:
        Z = C.CDLL(path)
    except OSError:
        return None
    vp = C.c_void_p
    Z.stream_open.restype = vp; Z.stream_open.argtypes = [vp, C.c_size_t]
    Z.stream_close.argtypes = [vp]
    Z.zfp_stream_open.restype = vp; Z.zfp_stream_open.argtypes = [vp]
    Z.zfp_stream_close.argtypes = [vp]
    Z.zfp_stream_set_rate.restype = C.c_double
    Z.zfp_stream_set_rate.argtypes = [vp, C.c_double, C.c_int, C.c_uint, C.c_int]
    Z.zfp_stream_rewind.argtypes = [vp]
    Z.zfp_field_3d.restype = vp; Z.zfp_field_3d.argtypes = [vp, C.c_int, C.c_uint, C.c_uint, C.c_uint]
    Z.zfp_field_free.argtypes = [vp]
    Z.zfp_compress.restype = C.c_size_t; Z.zfp_compress.argtypes = [vp, vp]
    Z.zfp_decompress.restype = C.c_size_t; Z.zfp_decompress.argtypes = [vp, vp]
    nz, ny, nx = sample.shape
    buf = np.zeros(sample.nbytes + 4096, dtype=np.uint8)
    out = np.empty_like(sample)
    bs = Z.stream_open(buf.ctypes.data, buf.size)
    zs = Z.zfp_stream_open(bs)
    Z.zfp_stream_set_rate(zs, maxbits / 64.0, 3, 3, 0)
    fi = Z.zfp_field_3d(sample.ctypes.data, 3, nx, ny, nz)
    fo = Z.zfp_field_3d(out.ctypes.data, 3, nx, ny, nz)
    best = None
    for _ in range(3):
        Z.zfp_stream_rewind(zs)
        t0 = time.perf_counter()
        n = Z.zfp_compress(zs, fi)
        t1 = time.perf_counter()
        Z.zfp_stream_rewind(zs)
        Z.zfp_decompress(zs, fo)
        t2 = time.perf_counter()
        if n == 0:
            best = None
            break
        cur = (t2 - t0, t1 - t0, t2 - t1)
        best = cur if best is None or cur[0] < best[0] else best
    for f in (fi, fo):
        Z.zfp_field_free(f)
    Z.zfp_stream_close(zs)
    Z.stream_close(bs)
    return best


def zvc_cpu_baseline(t, process):
    """The CPU checker's sparse path (count, prefix sum, compaction; expansion) on the
    same tensor: one warm-up and the median of three runs, on one core and on all."""
    import oracle

    x = t.cpu().numpy().reshape(-1)
    res = {"kind": "port", "sample": "the whole tensor, 1 warm-up + median of 3"}
    for key, omp in (("one_core", False), ("all_cores", True)):
        times = []
        for i in range(4):
            t0 = time.perf_counter()
            values, mask, begin, nnz = oracle.zvc_compress(x, process, omp=omp)
            t1 = time.perf_counter()
            oracle.zvc_decompress(values, mask, begin, x.size, process, omp=omp)
            t2 = time.perf_counter()
            if i:
                times.append((t1 - t0, t2 - t1))
        c, e = median([a for a, _ in times]), median([b for _, b in times])
        res[key] = {"compress_GBs_fp32": round(x.nbytes / c / 1e9, 3), "expand_GBs_fp32": round(x.nbytes / e / 1e9, 3),
                    "cores": oracle.lib(True).orc_threads() if omp else 1}
    return res


def zvc_extras(torch, api, dev, ex, config2_tensor, only_mib=0, cpu=False):
    only_256 = bool(only_mib)
    # ---- ZVC compact / expand / probe
    def zvc_case(label, t):
        n = t.numel()
        values, mask, begin, nnz = api.zvc_compress(t)
        o = torch.empty_like(t)
        api.GPUdecompression(values, o, mask, begin)
        torch.cuda.synchronize()
        k = int(nnz.item())
        dens = k / n
        reps = 40 if n > 1 << 24 else 200
        from cswap_amd._lib import lib
        L = lib()
        st = torch.cuda.current_stream().cuda_stream
        three = ev_ms(torch, lambda: L.cswap_zvc_compress(t.data_ptr(), n, api.PROCESS, begin.data_ptr(),
                                                          nnz.data_ptr(), values.data_ptr(), mask.data_ptr(), st), reps)
        ws = api.zvc_workspace(api.PROCESS, dev)
        # count + scan + compact as one operation, as the swap engine runs it for a ZVC request: the
        # single pass from 64 MiB on, the three kernels below
        full = ev_ms(torch, lambda: L.cswap_zvc_compress_fused(t.data_ptr(), n, api.PROCESS, ws.data_ptr(),
                                                               begin.data_ptr(), nnz.data_ptr(),
                                                               values.data_ptr(), mask.data_ptr(), st), reps)
        single = bool(L.cswap_zvc_takes_single_pass(n, api.PROCESS))
        cnt = torch.zeros(api.PROCESS, dtype=torch.int32, device=dev)
        count = ev_ms(torch, lambda: L.cswap_zvc_count(t.data_ptr(), n, api.PROCESS, cnt.data_ptr(), st), reps)
        compact = ev_ms(torch, lambda: L.cswap_zvc_compact(t.data_ptr(), n, api.PROCESS, begin.data_ptr(),
                                                           values.data_ptr(), mask.data_ptr(), st), reps)
        expand = ev_ms(torch, lambda: api.GPUdecompression(values, o, mask, begin), reps)
        pr = torch.zeros(1, dtype=torch.int64, device=dev)
        probe = ev_ms(torch, lambda: api.probe_nnz(t, out=pr), reps)
        bpv = 4 + 1 / 8 + 4 * dens
        ex[f"zvc_{label}"] = {
            "density": round(dens, 4), "ratio": round((4 * k + n / 8 + 4 * api.PROCESS) / (4 * n), 4),
            "count_ms": round(count, 4), "compact_ms": round(compact, 4), "compress_total_ms": round(full, 4),
            "compress_total_is_single_pass": single,
            "compress_three_kernels_ms": round(three, 4),
            "compress_three_kernels_hbm_frac": round(bpv * n / three / 1e6 / HBM_PEAK_GBS, 4),
            "expand_ms": round(expand, 4), "probe_ms": round(probe, 4),
            "compact_GBs_fp32": round(4 * n / compact / 1e6, 1), "expand_GBs_fp32": round(4 * n / expand / 1e6, 1),
            "compact_hbm_frac": round(bpv * n / compact / 1e6 / HBM_PEAK_GBS, 4),
            "compress_total_hbm_frac": round(bpv * n / full / 1e6 / HBM_PEAK_GBS, 4),
            "expand_hbm_frac": round(bpv * n / expand / 1e6 / HBM_PEAK_GBS, 4),
            "probe_hbm_frac": round(4 * n / probe / 1e6 / HBM_PEAK_GBS, 4)}

    if not only_256:
        for pct in (30, 50, 70, 90):
            zvc_case(f"config2_s{pct}", torch.from_numpy(config2_tensor(pct)).to(dev))

    # ---- ZVC chunk count: the reference's 512*32 against the size rule the engine uses
    def geometry_case(mib):
        from cswap_amd._lib import lib
        L = lib()
        n = mib * 1024 * 1024 // 4
        t = torch.relu(torch.randn(n, device=dev))
        o = torch.empty_like(t)
        st = torch.cuda.current_stream().cuda_stream
        row = {}
        for label, process in (("reference_16384", api.PROCESS), ("size_rule", L.cswap_zvc_pick_process(n))):
            _, W, _ = api.zvc_geometry(n, process)
            values = torch.empty(n, device=dev)
            mask = torch.empty(W * process, dtype=torch.int32, device=dev)
            begin = torch.zeros(process, dtype=torch.int32, device=dev)
            nnz = torch.zeros(1, dtype=torch.int32, device=dev)
            c = ev_ms(torch, lambda: L.cswap_zvc_compress(t.data_ptr(), n, process, begin.data_ptr(), nnz.data_ptr(),
                                                          values.data_ptr(), mask.data_ptr(), st), 30)
            e = ev_ms(torch, lambda: L.cswap_zvc_expand(values.data_ptr(), mask.data_ptr(), begin.data_ptr(), n,
                                                        process, o.data_ptr(), st), 30)
            row[label] = {"process": process, "compress_ms": round(c, 4), "expand_ms": round(e, 4)}
        ex[f"zvc_geometry_{mib}MiB"] = row

    if not only_256:
        for mib in (1, 4, 16, 32, 128):
            geometry_case(mib)
    g = torch.Generator(device=dev); g.manual_seed(1)
    if only_mib and only_mib != 256:
        zvc_case(f"relu_{only_mib}MiB", torch.relu(torch.randn(only_mib << 18, generator=g, device=dev)))
        return ex
    t256 = torch.relu(torch.randn(64 * 1024 * 1024, generator=g, device=dev))
    zvc_case("relu_256MiB", t256)
    if cpu:
        ex["zvc_relu_256MiB"]["cpu_baseline"] = zvc_cpu_baseline(t256, api.PROCESS)
    del t256
    # twice the size: mask and values (286 MB) no longer stay in the 256 MB memory-side cache
    # between the launches of a timing loop, as the 143 MB of the case above do
    if not only_256:
        zvc_case("relu_512MiB", torch.relu(torch.randn(128 * 1024 * 1024, generator=g, device=dev)))
    return ex


def extras(torch, api, dev, zvc_only=0, cpu=False):
    import numpy as np

    from cswap_amd.workloads import config1_field, config2_tensor, field_dims

    ex = {}
    if zvc_only:
        return zvc_extras(torch, api, dev, ex, config2_tensor, only_mib=zvc_only)
    # ---- ZFP at other rates and on configuration 1
    g = torch.Generator(device=dev); g.manual_seed(0)
    big = torch.softmax(torch.randn((32, 12, 512, 512), generator=g, device=dev), dim=-1).contiguous()
    c1 = torch.from_numpy(config1_field()).to(dev)
    for label, t in (("attn_402MB", big), ("config1_16MB", c1)):
        n = t.numel()
        nx, ny, nz = field_dims(t.shape)
        for rate in (4, 8, 16):
            mb = 64 * rate
            s = torch.empty(api.zfp_stream_capacity(nx, ny, nz, mb), dtype=torch.uint8, device=dev)
            o = torch.empty_like(t)
            api.cuda_compress(t, mb, out=s); api.cuda_decompress(s, t.shape, mb, out=o)
            reps = 40 if n > 1 << 24 else 200
            e = ev_ms(torch, lambda: api.cuda_compress(t, mb, out=s), reps)
            d = ev_ms(torch, lambda: api.cuda_decompress(s, t.shape, mb, out=o), reps)
            bpv = 4 + rate / 8
            ex[f"zfp_{label}_r{rate}"] = {
                "compress_ms": round(e, 4), "decompress_ms": round(d, 4),
                "compress_GBs_fp32": round(4 * n / e / 1e6, 1), "decompress_GBs_fp32": round(4 * n / d / 1e6, 1),
                "compress_hbm_frac": round(bpv * n / e / 1e6 / HBM_PEAK_GBS, 4),
                "decompress_hbm_frac": round(bpv * n / d / 1e6 / HBM_PEAK_GBS, 4)}
            if label == "attn_402MB" and rate == 8:
                ce, cd = zfp_cold_pair(torch, api, t, rate, 3, 30)     # 3 x (403 + 101) MB between two uses of a buffer
                ex[f"zfp_{label}_r{rate}"].update({
                    "compress_ms_cold": round(ce, 4), "decompress_ms_cold": round(cd, 4),
                    "compress_hbm_frac_cold": round(bpv * n / ce / 1e6 / HBM_PEAK_GBS, 4),
                    "decompress_hbm_frac_cold": round(bpv * n / cd / 1e6 / HBM_PEAK_GBS, 4)})
    # ---- what this box's memory gives plain kernels on the same 402.7 MB buffer (bytes moved per second):
    # torch's device copy (reads and writes it), fill (writes it), and this library's read-only counting pass
    other = torch.empty_like(big)
    cnt = torch.zeros(1, dtype=torch.int64, device=dev)
    nb = 4 * big.numel()
    ex["box_memory_GBs"] = {
        "copy_read_plus_write": round(2 * nb / ev_ms(torch, lambda: other.copy_(big), 40) / 1e6, 1),
        "fill_write": round(nb / ev_ms(torch, lambda: other.fill_(1.0), 40) / 1e6, 1),
        "count_nonzero_read": round(nb / ev_ms(torch, lambda: api.probe_nnz(big, out=cnt), 40) / 1e6, 1)}
    del big, other

    # ---- configuration 5's other tensors (rates 8 and 16) and configuration 3's stack (rates 4/8/16)
    from cswap_amd.workloads import config3_fields, config5_tensor_torch

    def zfp_case(key, t, rate, cold=0):
        n = t.numel()
        nx, ny, nz = field_dims(t.shape)
        mb = 64 * rate
        s = torch.empty(api.zfp_stream_capacity(nx, ny, nz, mb), dtype=torch.uint8, device=dev)
        o = torch.empty_like(t)
        api.cuda_compress(t, mb, out=s); api.cuda_decompress(s, t.shape, mb, out=o)
        reps = 40 if n > 1 << 24 else 200
        e = ev_ms(torch, lambda: api.cuda_compress(t, mb, out=s), reps)
        d = ev_ms(torch, lambda: api.cuda_decompress(s, t.shape, mb, out=o), reps)
        bpv = 4 + rate / 8
        ex[key] = {"MB": round(4 * n / 1e6, 1), "compress_ms": round(e, 4), "decompress_ms": round(d, 4),
                   "pair_GBs_fp32": round(4 * n / (e + d) / 1e6, 1),
                   "compress_hbm_frac": round(bpv * n / e / 1e6 / HBM_PEAK_GBS, 4),
                   "decompress_hbm_frac": round(bpv * n / d / 1e6 / HBM_PEAK_GBS, 4),
                   "stream_over_input": round(s.numel() / (4 * n), 4)}
        if cold:
            ce, cd = zfp_cold_pair(torch, api, t, rate, cold, reps)
            ex[key].update({"compress_ms_cold": round(ce, 4), "decompress_ms_cold": round(cd, 4),
                            "compress_hbm_frac_cold": round(bpv * n / ce / 1e6 / HBM_PEAK_GBS, 4),
                            "decompress_hbm_frac_cold": round(bpv * n / cd / 1e6 / HBM_PEAK_GBS, 4)})

    for name in ("hidden_gelu", "ffn_gelu"):
        t = config5_tensor_torch(name, dev, seed=0)
        for rate in (8, 16):
            # cold figures at 8 bits per value: 8 rotating copies (8 x 63 MB and 8 x 252 MB between two uses)
            zfp_case(f"zfp_config5_{name}_r{rate}", t, rate, cold=8 if rate == 8 else 0)
        del t
    for name, f in config3_fields(batch=128).items():
        t = torch.from_numpy(f).to(dev)
        for rate in (4, 8, 16):
            zfp_case(f"zfp_config3_{name}_r{rate}", t, rate)
        del t

    # ---- the other scalar types cuda_compress dispatches on: same field shape (64, 64, 4096), 16 Mi values
    g2 = torch.Generator(device=dev); g2.manual_seed(1)
    base = torch.randn((4096, 64, 64), generator=g2, device=dev)
    for label, t, rate in (("i32_r8", (base * 1e6).to(torch.int32), 8), ("f64_r16", base.double(), 16),
                           ("i64_r16", (base.double() * 1e12).to(torch.int64), 16)):
        n, esz = t.numel(), t.element_size()
        mb = 64 * rate
        s = torch.empty(api.zfp_stream_capacity(64, 64, 4096, mb), dtype=torch.uint8, device=dev)
        o = torch.empty_like(t)
        api.cuda_compress(t, mb, out=s); api.cuda_decompress(s, t.shape, mb, out=o)
        e = ev_ms(torch, lambda: api.cuda_compress(t, mb, out=s), 20)
        d = ev_ms(torch, lambda: api.cuda_decompress(s, t.shape, mb, out=o), 20)
        bpv = esz + rate / 8
        ex[f"zfp_{label}_{esz * n >> 20}MiB"] = {
            "compress_ms": round(e, 4), "decompress_ms": round(d, 4),
            "pair_GBs_in": round(esz * n / (e + d) / 1e6, 1),
            "compress_hbm_frac": round(bpv * n / e / 1e6 / HBM_PEAK_GBS, 4),
            "decompress_hbm_frac": round(bpv * n / d / 1e6 / HBM_PEAK_GBS, 4)}
    del base

    zvc_extras(torch, api, dev, ex, config2_tensor, cpu=cpu)

    import bench_parts
    ex["swap"] = bench_parts.bench_schedule(dev)
    ex["swap_backward"] = bench_parts.bench_backward(dev)
    ex["planner"] = bench_parts.bench_planner(dev)
    ex["train_step"] = bench_parts.bench_training_step(dev)
    ex["train_step_transformer"] = bench_parts.bench_transformer_step(dev)
    return ex


if __name__ == "__main__":
    main()
