#!/usr/bin/env python3
"""Benchmark of the int8 inference hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" = the prefill workload (cfg3): the four Llama-8B-style rotated W8A8
linears at M = 2048 tokens (4096->6144, 4096->14336 twice, 14336->4096), each
= block-128 Hadamard rotation + per-token int8 quantization of the fp32
activations, int8 MFMA GEMM against pre-rotated pre-quantized weights, fp32
dequant.  Inputs are resident in HBM before the timed region.  `value` is
int8 TOPS over the whole step (rotate/quant prologue included).

The same run also reports, under "sub_metrics": the GEMM kernels alone, the
decode GEMV sweep (cfg1), decode attention (cfg2), the MoE layer (cfg4) and
the small linear (cfg0), each against its own roofline, with weight / KV
buffers rotated through more than 256 MB so that the Infinity Cache cannot
stand in for HBM; and "cpu_baseline": the CPU oracle timed on the host cores
(a reported baseline, not a target).  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "mojo-linuxperiments_amd"))

PEAK_INT8_TOPS = 5000.0     # dense int8 MFMA, MI355X
PEAK_HBM_GBS = 8000.0
MALL_BYTES = 256 << 20


NO_GRAPH = False    # --no-graph: every timing loop launches eagerly


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def host_topology():
    """Core and NUMA node counts from the sysfs files the upstream NumaInfo reads
    (numa/numa.mojo:107-115)."""
    nodes = 1
    try:
        txt = open("/sys/devices/system/node/online").read().strip()
        nodes = 0
        for part in txt.split(","):
            lo, _, hi = part.partition("-")
            nodes += int(hi or lo) - int(lo) + 1
    except OSError:
        pass
    return {"cores": len(os.sched_getaffinity(0)), "numa_nodes": nodes}


class Timer:
    def __init__(self, mi, stream):
        self.mi, self.stream = mi, stream
        self.e0, self.e1 = mi.Event(), mi.Event()

    def run(self, fn, reps):
        """ms per call of fn(), timed with HIP events on the launch stream."""
        self.mi.check(self.mi.lib.mi_stream_synchronize(self.stream))
        self.e0.record(self.stream)
        for _ in range(reps):
            fn()
        self.e1.record(self.stream)
        self.e1.synchronize()
        return self.e0.elapsed_ms(self.e1) / reps

    def samples(self, fn, n):
        """n per-call durations (ms): an event before and after every call, all recorded back to back on the
        launch stream and read only after the last one, so that the chip never idles between the calls."""
        ev = [self.mi.Event() for _ in range(n + 1)]
        ev[0].record(self.stream)
        for i in range(n):
            fn()
            ev[i + 1].record(self.stream)
        ev[n].synchronize()
        out = [ev[i].elapsed_ms(ev[i + 1]) for i in range(n)]
        for e in ev:
            e.destroy()
        return out

    def settle(self, fn, ms=60.0):
        """Untimed: keep fn() running back to back for about `ms` of GPU time.  After any idle spell the
        chip's power control first throttles the matrix pipe hard and then converges, over about 30 ms of
        continuous load, on the clock it sustains; timing starts from that sustained state."""
        per = max(self.run(fn, 3), 1e-3)
        for _ in range(int(ms / per) + 1):
            fn()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-sub", action="store_true", help="only the headline workload")
    ap.add_argument("--decode-layer-only", action="store_true",
                    help="only the decode-layer chain sub-metric (for a kernel trace of that chain alone)")
    ap.add_argument("--decode-stack", type=int, default=0, metavar="L",
                    help="only a decode step through a stack of L decoder layers (e.g. 32: 11.4 GB of weights and "
                         "caches), each with its own weights and KV cache, as one graph")
    ap.add_argument("--skip-stack", action="store_true", help="no 32-layer decode stack leg (it takes 15 GB more)")
    ap.add_argument("--skip-cpu", action="store_true", help="no CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch everything eagerly: for runs under rocprofv3's kernel trace, whose tool library "
                         "ended in a segmentation fault inside hipGraphLaunch; the line then says method: eager")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="context only: the vendor library's int8 GEMM (torch._int_mm, int32 out) beside this "
                         "library's on the cfg3 shapes, same codes, same sustained clock state; one JSON line")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="context only: what a loop of v_mfma_i32_16x16x64_i8 alone sustains on this machine "
                         "(operands in registers, with and without the GEMM's LDS fragment reads, zeros and "
                         "activation-like codes); one JSON line")
    ap.add_argument("--grid-wait-probe", action="store_true",
                    help="time a grid-wide wait as a cooperative and as a plain launch (its own executable), then exit")
    ap.add_argument("--gemm-timeline", action="store_true",
                    help="context only: where the eight-wave GEMM's time goes (prologue / stage loop / stores, in "
                         "clock ticks read inside the kernel), from the instrumented build of the library; one JSON line")
    ap.add_argument("--gemm-timeline-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--pmc-probe", action="store_true",
                    help="a few launches of the dominant kernels plus a copy-like kernel of known size, "
                         "for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs")
    args = ap.parse_args()
    global NO_GRAPH
    NO_GRAPH = args.no_graph
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no sharding, no collectives); use --gpus 1")

    if args.gemm_timeline:
        # the instrumented library is another build of the same sources: a child process loads it in place of the
        # product library (nothing has touched the GPU in this process yet)
        import subprocess
        tl = os.path.join(ROOT, "mojo-linuxperiments_amd", "libmi355_int8_timeline.so")
        if not os.path.exists(tl):
            sys.exit("bench.py: %s is not built (make -C mojo-linuxperiments_amd/csrc)" % tl)
        env = dict(os.environ, MI355_INT8_LIB=tl)
        sys.exit(subprocess.run([sys.executable, os.path.abspath(__file__), "--gemm-timeline-child"], env=env).returncode)

    import mi355_int8 as mi     # fails loudly when the HIP library is not built
    import workload as wl

    if args.mfma_probe:
        print(json.dumps(mfma_probe()), flush=True)
        return
    if args.grid_wait_probe:
        print(json.dumps(run_probe("grid_wait_probe", "grid_wide_wait")), flush=True)
        return
    if args.gemm_timeline_child:
        return gemm_timeline(mi, wl)
    if args.pmc_probe:
        return pmc_probe(mi, wl)
    if args.vendor_gemm:
        return vendor_gemm(mi, wl)
    if args.decode_stack:
        dev = mi.Device(arena_bytes=(2 << 30) + args.decode_stack * (400 << 20))
        pool = mi.StreamPool(dev, 1)
        s = pool.stream(0)
        for b in (None, 1):
            print(json.dumps(decode_layer_chain(mi, wl, dev, s, Timer(mi, s), reps=5, batch=b,
                                                nlayers=args.decode_stack)), flush=True)
        pool.destroy()
        dev.close()
        return
    if args.decode_layer_only:
        dev = mi.Device(arena_bytes=12 << 30)
        pool = mi.StreamPool(dev, 1)
        s = pool.stream(0)
        print(json.dumps(decode_layer_chain(mi, wl, dev, s, Timer(mi, s), reps=20)), flush=True)
        print(json.dumps(decode_layer_chain(mi, wl, dev, s, Timer(mi, s), reps=20, batch=1)), flush=True)
        pool.destroy()
        dev.close()
        return

    log("matrix-pipe probe ...")
    probe = mfma_probe()   # a child process, finished before this process takes the device

    dev = mi.Device(arena_bytes=12 << 30)
    pool = mi.StreamPool(dev, 1)
    s = pool.stream(0)
    timer = Timer(mi, s)
    lib = mi.lib
    M = wl.PREFILL_M

    # ---- weights: one fp32 matrix per shape from the seed, prepared on the GPU,
    # then replicated to distinct addresses so that reuse across calls misses the cache
    log("preparing weights ...")
    shapes = {}
    for name, K, N in wl.PROJECTIONS:
        if (K, N) in shapes:
            continue
        w = wl.weights(2025, N, K, stream=K + N)
        mark = dev.mark()
        dw = dev.upload(w)
        q0, s0 = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
        mi.fwht_quant(dw, q0, s0, wl.HADAMARD_BLOCK)
        dev.sync()
        qh, sh = dev.download(q0), dev.download(s0)
        dev.reset_to(mark)
        copies = MALL_BYTES // (N * K) + 2
        bufs = []
        for _ in range(copies):
            bufs.append((dev.upload(qh), dev.upload(sh)))
        shapes[(K, N)] = bufs
        del w
    acts = {K: dev.upload(wl.activations(2025, M, K, stream=K)) for K in (4096, 14336)}
    acts_qkv = dev.upload(wl.activations(2025, M, 4096, stream=1))   # the attention block's input: a matrix of its own
    # every projection writes an output of its own (318 MB in all: more than the memory-side cache holds)
    ybufs = {name: dev.empty((M, N), np.float32) for name, K, N in wl.PROJECTIONS}
    ybuf = ybufs["gate"]
    lin_ws = dev.empty(lib.mi_w8a8_linear_workspace_bytes(M, 14336, 14336), np.uint8)
    dev.sync()

    counters = {k: 0 for k in shapes}

    def next_w(K, N):
        bufs = shapes[(K, N)]
        counters[(K, N)] = (counters[(K, N)] + 1) % len(bufs)
        return bufs[counters[(K, N)]]

    # One cfg3 step = the four projections of a decoder layer's prefill.  gate and up read the same activation
    # matrix (as they do in the layer), so its rotate + quantize prologue runs once and both contractions take the
    # codes; qkv and down each quantize their own input.  ONE launch for the three prologues, then ONE launch for the four
    # contractions (mi_gemm_batch_*: a workgroup per compute unit walks a balanced list of 256 x 256 tiles drawn from
    # all four problems).  The same step with four launches (one per projection, the single-problem kernels) and as
    # four whole linears (a prologue each) is timed beside it.
    qx_ws = {K: (dev.empty((M, K), np.int8), dev.empty(M, np.float32)) for K in (4096, 14336)}
    qx_qkv = (dev.empty((M, 4096), np.int8), dev.empty(M, np.float32))
    batch = mi.GemmBatch(dev, [(M, N, K) for _, K, N in wl.PROJECTIONS])

    def batch_ops(codes_of):
        ops = []
        for name, K, N in wl.PROJECTIONS:
            qw, sw = next_w(K, N)
            cx, cs = codes_of(name, K)
            ops.append((cx, cs, qw, sw, ybufs[name]))
        return ops

    def prefill_step():
        # the three inputs (qkv's, gate's and up's, down's) are rotated and quantized by ONE launch
        mi.fwht_quant_batch([(acts_qkv,) + qx_qkv, (acts[4096],) + qx_ws[4096], (acts[14336],) + qx_ws[14336]],
                            wl.HADAMARD_BLOCK, stream=s)
        batch.run_f32(batch_ops(lambda name, K: qx_qkv if name == "qkv" else qx_ws[K]), stream=s)

    def prefill_step_four_launches():
        last_quantized = None
        for name, K, N in wl.PROJECTIONS:
            qw, sw = next_w(K, N)
            cx, cs = qx_ws[K]
            if not (name == "up" and last_quantized == "gate"):
                mi.fwht_quant(acts[K], cx, cs, wl.HADAMARD_BLOCK, stream=s)
            last_quantized = name
            mi.check(lib.mi_w8a8_gemm_dequant_f32(cx.ptr, cs.ptr, qw.ptr, sw.ptr, ybufs[name].ptr, M, N, K, s))

    def prefill_step_four_linears():
        for name, K, N in wl.PROJECTIONS:
            qw, sw = next_w(K, N)
            mi.check(lib.mi_w8a8_linear_f32(acts[K].ptr, qw.ptr, sw.ptr, ybufs[name].ptr, M, N, K, wl.HADAMARD_BLOCK,
                                            lin_ws.ptr, lin_ws.nbytes, s))

    log("headline: prefill step x%d (+%d warm-up)" % (args.steps, args.warmup))
    timer.settle(prefill_step)
    for _ in range(args.warmup):
        prefill_step()
    dev.sync(s)
    t0 = time.perf_counter()
    ms_eager = timer.run(prefill_step, args.steps)
    dev.sync(s)
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    # The declared method: the same K steps recorded once into a graph (the weight rotation is baked in) and
    # replayed as one launch, exactly K steps inside the timed region and no host work between kernels.  The eager
    # figure is reported beside it and never picked.
    def graph_ms(step):
        with mi.Graph.capture(s) as g:
            for _ in range(args.steps):
                step()
        timer.settle(lambda: g.launch())
        ms = timer.run(lambda: g.launch(), 1) / args.steps
        g.destroy()
        return ms

    if NO_GRAPH:
        ms_graph = None
        ms_step = ms_eager
        timer.settle(prefill_step_four_launches)
        ms_four_launches = timer.run(prefill_step_four_launches, args.steps)
        timer.settle(prefill_step_four_linears)
        ms_four_linears = timer.run(prefill_step_four_linears, args.steps)
    else:
        ms_graph = graph_ms(prefill_step)
        ms_step = ms_graph
        ms_four_launches = graph_ms(prefill_step_four_launches)
        ms_four_linears = graph_ms(prefill_step_four_linears)
    step_ops = sum(wl.gemm_ops(M, N, K) for _, K, N in wl.PROJECTIONS)
    value = step_ops / (ms_step * 1e-3) / 1e12

    # ---- the dominant kernel alone: the batched GEMM (one launch, four problems) on already-quantized activations,
    # and, for comparison, each projection as a launch of its own (the single-problem kernels)
    gemm_ms, gemm_samples = {}, {}
    qx = {K: dev.empty((M, K), np.int8) for K in (4096, 14336)}
    sx = {K: dev.empty(M, np.float32) for K in (4096, 14336)}
    for K in qx:
        mi.fwht_quant(acts[K], qx[K], sx[K], wl.HADAMARD_BLOCK, stream=s)
    quant_ms = {K: timer.run(lambda K=K: mi.fwht_quant(acts[K], qx[K], sx[K], wl.HADAMARD_BLOCK, stream=s), 20)
                for K in qx}

    def batch_only():
        batch.run_f32(batch_ops(lambda name, K: (qx[K], sx[K])), stream=s)
    timer.settle(batch_only)
    batch_ms = timer.run(batch_only, max(10, args.steps))
    batch_samples = sorted(timer.samples(batch_only, max(10, args.steps)))
    # the same launch with the SAME weights every time (they then stay in the 256 MB memory-side cache): context
    # for the figure above, which is the one the timed step sees (weights from HBM)
    fixed_ops = batch_ops(lambda name, K: (qx[K], sx[K]))
    resident_only = lambda: batch.run_f32(fixed_ops, stream=s)
    timer.settle(resident_only)
    batch_resident_ms = timer.run(resident_only, max(10, args.steps))
    for name, K, N in wl.PROJECTIONS:
        def one(name=name, K=K, N=N):
            qw, sw = next_w(K, N)
            mi.check(lib.mi_w8a8_gemm_dequant_f32(qx[K].ptr, sx[K].ptr, qw.ptr, sw.ptr, ybufs[name].ptr, M, N, K, s))
        timer.settle(one)
        gemm_ms[name] = timer.run(one, max(10, args.steps))
        gemm_samples[name] = sorted(timer.samples(one, max(10, args.steps)))
    gemm_total_ms = sum(gemm_ms.values())
    gemm_tops = step_ops / (batch_ms * 1e-3) / 1e12
    single_tops = step_ops / (gemm_total_ms * 1e-3) / 1e12
    # HBM-side bytes per launch of the tiled GEMM, measured with hardware counters in a separate run
    traffic, traffic_total = None, None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as fh:
            rec = json.load(fh)
        if "batched_gemm_bytes_per_launch" in rec:
            traffic = rec["batched_gemm_bytes_per_launch"]
            traffic_total = traffic["fetch"] + traffic["write"]
    roofline = {
        "kernel": "k_w8a8_list, v_mfma_i32_16x16x64_i8: ONE launch for the four cfg3 contractions (1,216 tiles of "
                  "256 x 256 on a balanced work list), dequantization fused",
        "bound": "mfma", "achieved": round(gemm_tops, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
        "frac": round(gemm_tops / PEAK_INT8_TOPS, 4), "traffic": traffic_total,
        "traffic_unit": "bytes per launch (fetched + written), rocprofv3 PMC, calibrated",
        "traffic_source": "profiles/hbm_traffic_pmc.md (a separate rocprofv3 --pmc run of bench.py --pmc-probe, "
                          "not this run)",
        "traffic_fetch_write": traffic,
        "launch_us": round(batch_ms * 1e3, 2),
        "with_resident_weights": {
            "what": "the same launch with the same weights every time (resident in the memory-side cache); frac above "
                    "is the launch as the timed step runs it, with weights from HBM",
            "launch_us": round(batch_resident_ms * 1e3, 2),
            "frac": round(step_ops / (batch_resident_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)},
        "launch_us_median": round(batch_samples[len(batch_samples) // 2] * 1e3, 2),
        "launch_us_min": round(batch_samples[0] * 1e3, 2),
        "launch_samples": "median / min over single launches, each between two event records; launch_us is one pair "
                          "of events around back-to-back launches",
        "algorithmic_ops_per_launch": step_ops,
        "single_problem_launches": {
            "what": "the same four contractions as four launches of the single-problem kernels (k_w8a8_pair for qkv "
                    "and down, k_w8a8_tiled for gate and up)",
            "tops": round(single_tops, 1), "frac": round(single_tops / PEAK_INT8_TOPS, 4),
            "per_shape_us": {k: round(v * 1e3, 2) for k, v in gemm_ms.items()},
            "per_shape_us_median": {k: round(v[len(v) // 2] * 1e3, 2) for k, v in gemm_samples.items()},
            "per_shape_us_min": {k: round(v[0] * 1e3, 2) for k, v in gemm_samples.items()},
            "per_shape_frac": {name: round(wl.gemm_ops(M, N, K) / (gemm_ms[name] * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)
                               for name, K, N in wl.PROJECTIONS},
        },
    }
    # what the matrix pipe sustains here with nothing else in the way (power-limited clock): context for `frac`,
    # which stays against the published peak
    runs = (probe.get("mfma_power_limited_peak") or {}).get("runs") if probe else None
    if runs:
        like = [r for r in runs if r["operands"] != "zeros" and r["lds_fragment_reads"]]
        best = max(r["tops"] for r in like)
        roofline["sustained_mfma_measured"] = {
            "tops": best, "frac_of_it": round(gemm_tops / best, 4),
            "what": "a loop of the same MFMA alone with the 8 x 6 wave tile's LDS fragment reads, activation-like "
                    "codes, best of one and two waves per SIMD, ~3 ms per run (mojo-linuxperiments_amd/mfma_peak_probe)",
            "zeros_no_reads_tops": max(r["tops"] for r in runs if r["operands"] == "zeros" and not r["lds_fragment_reads"]),
        }
    else:
        roofline["sustained_mfma_measured"] = None

    out = {
        "metric": "W8A8 GEMM int8 TOPS & decode GB/s (% roofline) @1 GPU; vs CPU host cores",
        "value": round(value, 2), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "cfg3 prefill: the 4 rotated W8A8 projections of a layer (4096->6144, 4096->14336 x2, "
                               "14336->4096) at M=2048, Hadamard block 128, rotate+quant prologues included; gate and up share "
                               "one input, which is rotated and quantized once (3 prologues per step, run as ONE launch: mi_fwht_quant_batch_f32_i8), and the four "
                               "contractions run as ONE launch (mi_gemm_batch_run_f32); every projection writes an output of "
                               "its own (318 MB per step; weights rotate through >256 MB of copies); the K steps are recorded "
                               "into one HIP graph and replayed - the timed method; eager launches from Python are reported "
                               "beside it; about 60 ms of the same steps run untimed before the W warm-up steps so that "
                               "timing starts at the sustained clock",
                   "tokens": M, "ops_per_step": step_ops, "tokens_per_s": round(M / (ms_step * 1e-3), 1),
                   "wall_ms_per_step": round(wall_ms, 4),
                   "ms_per_step_eager": round(ms_eager, 4), "ms_per_step_graph": None if ms_graph is None else round(ms_graph, 4),
                   "method": "eager (--no-graph)" if NO_GRAPH else "graph replay",
                   "ms_per_step_four_launches": round(ms_four_launches, 4),
                   "ms_per_step_four_linears": round(ms_four_linears, 4),
                   "other_forms": "ms_per_step_four_launches: the same step with one launch per projection (3 prologues "
                                  "+ 4 single-problem GEMM launches); ms_per_step_four_linears: four whole linears, a "
                                  "prologue each (4 + 4 launches)"},
        "roofline": roofline,
        "host": host_topology(),
    }

    sub = {"prefill_quant_prologue_us": {str(K): round(v * 1e3, 2) for K, v in quant_ms.items()}}
    prologue_sets = [(acts_qkv,) + qx_qkv, (acts[4096],) + qx_ws[4096], (acts[14336],) + qx_ws[14336]]
    sub["prefill_quant_prologue_us"]["the_step_s_three_inputs_as_one_launch"] = round(
        timer.run(lambda: mi.fwht_quant_batch(prologue_sets, wl.HADAMARD_BLOCK, stream=s), 20) * 1e3, 2)
    if not args.skip_sub:
        sub.update(decode_gemv(mi, wl, dev, pool, s, timer, shapes, next_w))
        sub.update(decode_attention(mi, wl, dev, s, timer))
        sub.update(moe_layer(mi, wl, dev, s, timer))
        sub.update(cfg0_linear(mi, wl, dev, s, timer, shapes))
        sub.update(decode_layer_chain(mi, wl, dev, s, timer))
        sub.update(decode_layer_chain(mi, wl, dev, s, timer, batch=1))
        sub.update(moe_decode_layer_chain(mi, wl, dev, s, timer))
        if not args.skip_stack:
            # the whole stack as one graph: 32 layers, each with its own weights and cache (11.4 GB), in an arena
            # of its own that lives only for this measurement
            sdev = mi.Device(arena_bytes=15 << 30)
            spool = mi.StreamPool(sdev, 1)
            ss = spool.stream(0)
            stimer = Timer(mi, ss)
            sub.update(decode_layer_chain(mi, wl, sdev, ss, stimer, reps=5, nlayers=32))
            sub.update(decode_layer_chain(mi, wl, sdev, ss, stimer, reps=5, batch=1, nlayers=32))
            spool.destroy()
            sdev.close()
        sub.update(host_staging(mi, wl, dev, s, timer))
    out["sub_metrics"] = sub
    if not args.skip_cpu:
        out["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(out), flush=True)
    pool.destroy()
    dev.close()


def pmc_probe(mi, wl):
    """Three launches each of: the rotation-only kernel on fp32 [2048,14336] (reads and writes exactly
    117,440,512 B: the calibration for the FETCH_SIZE / WRITE_SIZE counters), the single-problem GEMMs on the cfg3
    shapes and the batched GEMM over all four (k_w8a8_list), the decode GEMV (M=1, 4096->14336), decode attention (cfg2) and the MoE layer (cfg4)."""
    lib = mi.lib
    dev = mi.Device(arena_bytes=8 << 30)
    M = wl.PREFILL_M
    g = np.random.default_rng(0)
    a = dev.upload(g.standard_normal((M, 14336), dtype=np.float32))
    b = dev.empty((M, 14336), np.float32)
    for _ in range(3):
        mi.fwht(a, b, 128)
    dev.sync()
    y = dev.empty((M, 14336), np.float32)
    bops = []
    for name, K, N in wl.PROJECTIONS:
        qx = dev.upload(g.integers(-127, 128, (M, K)).astype(np.int8))
        qw = dev.upload(g.integers(-127, 128, (N, K)).astype(np.int8))
        sx, sw = dev.upload(np.ones(M, np.float32)), dev.upload(np.ones(N, np.float32))
        bops.append((qx, sx, qw, sw, dev.empty((M, N), np.float32)))
        if name == "up":
            continue
        for _ in range(3):
            mi.check(lib.mi_w8a8_gemm_dequant_f32(qx.ptr, sx.ptr, qw.ptr, sw.ptr, y.ptr, M, N, K, None))
        if name == "gate":
            for _ in range(3):
                mi.check(lib.mi_w8a8_gemm_dequant_f32(qx.ptr, sx.ptr, qw.ptr, sw.ptr, y.ptr, 1, N, K, None))
        dev.sync()
    batch = mi.GemmBatch(dev, [(M, N, K) for _, K, N in wl.PROJECTIONS])   # the four contractions as one launch
    for _ in range(3):
        batch.run_f32(bops)
    dev.sync()
    timer = Timer(mi, None)
    print(json.dumps({"probe": "done", "attention": decode_attention(mi, wl, dev, None, timer, reps=1, graph=False),
                      "moe": moe_layer(mi, wl, dev, None, timer, reps=1, graph=False)}), flush=True)
    dev.close()


def graph_time(mi, dev, s, timer, calls, reps):
    """Per-call ms of a list of closures recorded once into a graph and replayed
    (decode kernels are a few microseconds: eager launches from Python would
    measure the interpreter)."""
    if NO_GRAPH:
        return eager_time(dev, s, timer, calls, max(1, reps // 2))
    for c in calls:
        c()
    dev.sync(s)
    # a graph launch itself costs a pause of several microseconds on the stream (8.8 us between two launches in the
    # kernel trace): the list is recorded as many times over as it takes to put 60 calls or more into one graph, so
    # that the pause is spread over them instead of over three or six
    rounds = max(1, -(-60 // len(calls)))
    with mi.Graph.capture(s) as g:
        for _ in range(rounds):
            for c in calls:
                c()
    g.launch()
    dev.sync(s)
    ms = timer.run(lambda: g.launch(), max(2, reps // rounds + 1)) / (len(calls) * rounds)
    g.destroy()
    return ms


def decode_gemv(mi, wl, dev, pool, s, timer, shapes, next_w):
    """cfg1: M in {1,4,16} x the four projections; weights rotate through > 256 MB."""
    lib = mi.lib
    res = {}
    layer_ms = {}
    for Mb in wl.DECODE_BATCHES:
        mark = dev.mark()
        per = {}
        for name, K, N in wl.PROJECTIONS:
            x = wl.activations(77, Mb, K)
            dx = dev.upload(x)
            qx, sx = dev.empty((Mb, K), np.int8), dev.empty(Mb, np.float32)
            y = dev.empty((Mb, N), np.float32)
            mi.fwht_quant(dx, qx, sx, wl.HADAMARD_BLOCK, stream=s)
            bufs = shapes[(K, N)]
            calls = [(lambda b=b: mi.check(lib.mi_w8a8_gemm_dequant_f32(qx.ptr, sx.ptr, b[0].ptr, b[1].ptr, y.ptr,
                                                                       Mb, N, K, s))) for b in bufs]
            ms = graph_time(mi, dev, s, timer, calls, 20)
            ws = dev.empty(lib.mi_w8a8_linear_workspace_bytes(Mb, N, K), np.uint8)
            calls2 = [(lambda b=b: mi.check(lib.mi_w8a8_linear_f32(dx.ptr, b[0].ptr, b[1].ptr, y.ptr, Mb, N, K,
                                                                  wl.HADAMARD_BLOCK, ws.ptr, ws.nbytes, s)))
                      for b in bufs]
            ms2 = graph_time(mi, dev, s, timer, calls2, 20)
            nbytes = wl.linear_algorithmic_bytes(Mb, N, K)
            per[name] = {"gemv_us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                         "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                         "TOPS": round(wl.gemm_ops(Mb, N, K) / (ms * 1e-3) / 1e12, 2),
                         "linear_with_quant_us": round(ms2 * 1e3, 2)}
        total_ms = sum(v["linear_with_quant_us"] for v in per.values()) * 1e-3
        per["tokens_per_s_four_projections"] = round(Mb / (total_ms * 1e-3), 1)
        res["M%d" % Mb] = per
        dev.reset_to(mark)
    return {"cfg1_decode_gemv": res}


def decode_attention(mi, wl, dev, s, timer, reps=20, graph=True):
    """cfg2: B=16, 32/8 heads, D=128, T=4096; three KV sets in rotation (402 MB per layout).  The headline is the
    cache in the matrix-pipe layouts (keys in 16-token tiles, values in transposed 64-token blocks: the layouts the
    decode chain keeps its cache in); the row-major cache [T, 128] is timed beside it, dense, with the append in
    front, and paged."""
    lib = mi.lib
    c = wl.ATTN
    B, Hq, Hkv, D, T = c["B"], c["Hq"], c["Hkv"], c["D"], c["T"]
    mark = dev.mark()
    rows = B * Hkv * T
    sets = []
    src = dev.upload(wl.normal(88, (rows, D), 0))
    for i in range(3):
        kq, ks = dev.empty((B, Hkv, T, D), np.int8), dev.empty((B, Hkv, T), np.float32)
        vq, vs = dev.empty((B, Hkv, T, D), np.int8), dev.empty((B, Hkv, T), np.float32)
        kt, vt = dev.empty((B, Hkv, T, D), np.int8), dev.empty((B, Hkv, T, D), np.int8)
        mi.check(lib.mi_fwht_quant_f32_i8(src.ptr, kq.ptr, ks.ptr, rows, D, D, s))
        mi.check(lib.mi_fwht_quant_f32_i8(src.ptr, vq.ptr, vs.ptr, rows, D, D, s))
        mi.check(lib.mi_kv_tiled_from_rows_i8(kq.ptr, vq.ptr, kt.ptr, vt.ptr, B * Hkv, T, T, T, s))
        sets.append((kq, ks, vq, vs, kt, vt))
    dq = dev.upload(wl.normal(88, (B, Hq, D), 1))
    do = dev.empty((B, Hq, D), np.float32)
    ws = dev.empty(lib.mi_gqa_decode_workspace_bytes(B, Hq, Hkv, D, T), np.uint8)
    run = (lambda calls: graph_time(mi, dev, s, timer, calls, reps)) if graph else (lambda calls: eager_time(dev, s, timer, calls))
    nbytes = wl.attention_algorithmic_bytes(B, Hq, Hkv, D, T)
    knew = dev.upload(wl.normal(88, (B, Hkv, D), 2))
    vnew = dev.upload(wl.normal(88, (B, Hkv, D), 3))
    dpos = dev.upload(np.full(B, T - 1, np.int32))
    dlen = dev.upload(np.full(B, T, np.int32))

    def tiled(k, append):
        # as a decode loop runs it: the new token's K and V heads are appended (rotate + quantize + write at
        # position T-1 of every sequence), then attention reads the cache through per-sequence lengths
        if append:
            mi.check(lib.mi_kv_append_tiled_f32_i8(knew.ptr, vnew.ptr, Hkv * D, k[4].ptr, k[1].ptr, k[5].ptr, k[3].ptr,
                                                   dpos.ptr, B, Hkv, D, T, s))
        mi.check(lib.mi_gqa_decode_attn_tiled(dq.ptr, k[4].ptr, k[1].ptr, k[5].ptr, k[3].ptr, do.ptr, B, Hq, Hkv, D, T,
                                              dlen.ptr if append else None, T, 0, ws.ptr, ws.nbytes, s))
    ms = run([(lambda k=k: tiled(k, False)) for k in sets])
    ms_app = run([(lambda k=k: tiled(k, True)) for k in sets])
    ms_rows = run([(lambda k=k: mi.gqa_decode(dq, k[0], k[1], k[2], k[3], do, False, ws, stream=s)) for k in sets])

    def cached(k):
        mi.check(lib.mi_kv_append_f32_i8(knew.ptr, vnew.ptr, Hkv * D, k[0].ptr, k[1].ptr, k[2].ptr, k[3].ptr,
                                         dpos.ptr, B, Hkv, D, T, s))
        mi.check(lib.mi_gqa_decode_attn_cache(dq.ptr, k[0].ptr, k[1].ptr, k[2].ptr, k[3].ptr, do.ptr, B, Hq, Hkv, D,
                                              T, dlen.ptr, T, 0, ws.ptr, ws.nbytes, s))
    ms_rows_app = run([(lambda k=k: cached(k)) for k in sets])
    # the row-major caches read as pools of 16-token pages under a shuffled block table (the rows a pool holds are
    # the same bytes; which token sits where does not change the time)
    P = 16
    max_pages = T // P
    table = np.random.default_rng(3).permutation(B * max_pages).astype(np.int32).reshape(B, max_pages)
    dtab = dev.upload(table)

    def paged(k):
        mi.check(lib.mi_gqa_decode_attn_paged(dq.ptr, k[0].ptr, k[1].ptr, k[2].ptr, k[3].ptr, do.ptr, dtab.ptr,
                                              max_pages, P, B, Hq, Hkv, D, dlen.ptr, T, 0, ws.ptr, ws.nbytes, s))
    ms_paged = run([(lambda k=k: paged(k)) for k in sets])
    # the tiled caches read as pools of 64-token pages (one key block and one value block per kv head) under a
    # shuffled block table: the same kernel, one table look-up per block
    pages64 = T // 64
    dtab64 = dev.upload(np.random.default_rng(4).permutation(B * pages64).astype(np.int32).reshape(B, pages64))

    def paged_tiled(k, append):
        if append:
            mi.check(lib.mi_kv_append_tiled_paged_f32_i8(knew.ptr, vnew.ptr, Hkv * D, k[4].ptr, k[1].ptr, k[5].ptr, k[3].ptr,
                                                         dtab64.ptr, pages64, dpos.ptr, B, Hkv, D, s))
        mi.check(lib.mi_gqa_decode_attn_tiled_paged(dq.ptr, k[4].ptr, k[1].ptr, k[5].ptr, k[3].ptr, do.ptr, dtab64.ptr,
                                                    pages64, B, Hq, Hkv, D, dlen.ptr, T, 0, ws.ptr, ws.nbytes, s))
    ms_paged64 = run([(lambda k=k: paged_tiled(k, False)) for k in sets])
    ms_paged64_app = run([(lambda k=k: paged_tiled(k, True)) for k in sets])
    dev.reset_to(mark)
    return {"cfg2_decode_attention": {"us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                      "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                      "tokens_per_s": round(B / (ms * 1e-3), 1), "algorithmic_bytes": nbytes,
                                      "cache_layout": "keys in 16-token tiles, values in transposed 64-token blocks",
                                      "with_kv_append_us": round(ms_app * 1e3, 2),
                                      "paged_64_token_pages_shuffled_table_us": round(ms_paged64 * 1e3, 2),
                                      "paged_64_token_pages_with_kv_append_us": round(ms_paged64_app * 1e3, 2),
                                      "row_major_cache_us": round(ms_rows * 1e3, 2),
                                      "row_major_with_kv_append_us": round(ms_rows_app * 1e3, 2),
                                      "row_major_paged_16_token_pages_us": round(ms_paged * 1e3, 2)}}


def eager_time(dev, s, timer, calls, reps=1):
    for c in calls:
        c()
    dev.sync(s)
    return timer.run(lambda: [c() for c in calls], reps) / len(calls)


def moe_layer(mi, wl, dev, s, timer, reps=20, graph=True):
    """cfg4: 512 tokens, hidden 2048, 128 experts top-8, inner 768 (604 MB of expert weights)."""
    lib = mi.lib
    c = wl.MOE
    T, H, E, topk, I = c["T"], c["H"], c["E"], c["topk"], c["I"]
    mark = dev.mark()
    x = dev.upload(wl.activations(99, T, H))
    wr = dev.upload(wl.weights(99, E, H, 1))

    def prep(n, k, b, stream):
        w = dev.upload(wl.weights(99, E * n, k, stream))
        q, sc = dev.empty((E, n, k), np.int8), dev.empty((E, n), np.float32)
        mi.check(lib.mi_fwht_quant_f32_i8(w.ptr, q.ptr, sc.ptr, E * n, k, b, s))
        return q, sc
    wg, sg = prep(I, H, wl.HADAMARD_BLOCK, 2)
    wu, su = prep(I, H, wl.HADAMARD_BLOCK, 3)
    wd, sd = prep(H, I, wl.MOE_INNER_BLOCK, 4)
    y = dev.empty((T, H), np.float32)
    ws = dev.empty(lib.mi_moe_layer_workspace_bytes(T, H, I, E, topk), np.uint8)
    call = lambda: mi.moe_layer(x, wr, wg, sg, wu, su, wd, sd, y, topk, ws, stream=s)
    ms = graph_time(mi, dev, s, timer, [call], reps) if graph else eager_time(dev, s, timer, [call])
    wbytes = wl.moe_weight_bytes(E, H, I)
    ops = wl.moe_ops(T, topk, H, I)
    dev.reset_to(mark)
    return {"cfg4_moe_layer": {"us": round(ms * 1e3, 2), "GBps": round(wbytes / (ms * 1e-3) / 1e9, 1),
                               "hbm_frac": round(wbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                               "TOPS": round(ops / (ms * 1e-3) / 1e12, 2),
                               "tokens_per_s": round(T / (ms * 1e-3), 1), "weight_bytes": wbytes}}


def gemm_timeline(mi, wl):
    """The eight-wave GEMM on its two cfg3 shapes, 400 launches each on the benchmark's codes (sustained clock), then
    the ticks the last launch left: per workgroup and K half, first instruction -> first stage ready, the stage
    loop, exchange + stores until the last store is issued, until the stores are acknowledged."""
    import ctypes as C
    lib = mi.lib
    if not hasattr(lib, "mi_debug_gemm_timeline"):
        sys.exit("bench.py --gemm-timeline-child needs the instrumented library (run bench.py --gemm-timeline)")
    dev = mi.Device(arena_bytes=6 << 30)
    pool = mi.StreamPool(dev, 1)
    s = pool.stream(0)
    M = wl.PREFILL_M
    out = {}
    for name, K, N, tile in (("qkv", 4096, 6144, (256, 192)), ("down", 14336, 4096, (128, 256))):
        mark = dev.mark()
        m2 = dev.mark()
        qx, sx = dev.empty((M, K), np.int8), dev.empty(M, np.float32)
        mi.fwht_quant(dev.upload(wl.activations(2025, M, K, stream=K)), qx, sx, wl.HADAMARD_BLOCK)
        qw0, sw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
        mi.fwht_quant(dev.upload(wl.weights(2025, N, K, stream=K + N)), qw0, sw, wl.HADAMARD_BLOCK)
        dev.sync()
        xh, sxh, wh, swh = dev.download(qx), dev.download(sx), dev.download(qw0), dev.download(sw)
        dev.reset_to(m2)
        qx, sx, sw = dev.upload(xh), dev.upload(sxh), dev.upload(swh)
        copies = MALL_BYTES // (N * K) + 2
        qws = [dev.upload(wh) for _ in range(copies)]
        y = dev.empty((M, N), np.float32)
        e0, e1 = mi.Event(), mi.Event()
        reps = 400
        for it in range(reps + 40):
            if it == reps:
                e0.record(s)
            mi.check(lib.mi_w8a8_gemm_dequant_f32(qx.ptr, sx.ptr, qws[it % copies].ptr, sw.ptr, y.ptr, M, N, K, s))
        e1.record(s)
        e1.synchronize()
        us = e0.elapsed_ms(e1) / 40 * 1e3
        ntile = (M // tile[0]) * (N // tile[1])
        buf = np.zeros(ntile * 2 * 8, np.uint64)
        lib.mi_debug_gemm_timeline.restype = C.c_int32
        mi.check(lib.mi_debug_gemm_timeline(buf.ctypes.data_as(C.c_void_p), C.c_int32(buf.size)))
        t = buf.reshape(ntile, 2, 8).astype(np.float64)
        nk = K // 128
        mhz = float((t[:, :, 4] / t[:, :, 5]).mean() * 100.0)
        out[name] = {
            "kernel_us_event": round(us, 2), "workgroups": ntile, "stages": nk, "clock_mhz": round(mhz),
            "ticks": {"prologue": round(float(t[:, :, 0].mean())), "stage_loop": round(float(t[:, :, 1].mean())),
                      "exchange_and_stores_issued": [round(float(t[:, h, 2].mean())) for h in (0, 1)],
                      "stores_acknowledged": round(float(t[:, :, 3].mean())), "whole_kernel": round(float(t[:, :, 4].mean()))},
            "ticks_per_stage": round(float(t[:, :, 1].mean()) / nk),
            "mfma_per_simd_and_stage": (tile[0] // 32) * (tile[1] // 32) * 2,
            "us": {"prologue": round(float(t[:, :, 0].mean()) / mhz, 2), "stage_loop": round(float(t[:, :, 1].mean()) / mhz, 2),
                   "exchange_and_stores": round(float((t[:, :, 2] + t[:, :, 3]).mean()) / mhz, 2)},
            "first_entry_to_last_end_us": round(float(t[:, :, 7].max() - t[:, :, 6].min()) / 100.0, 2),
            "entry_skew_us": round(float(t[:, :, 6].max() - t[:, :, 6].min()) / 100.0, 2),
            "end_skew_us": round(float(t[:, :, 7].max() - t[:, :, 7].min()) / 100.0, 2),
        }
        dev.reset_to(mark)
    out["batch"] = list_timeline(mi, wl, dev, s)
    print(json.dumps({"gemm_timeline": out, "M": M,
                      "note": "k_w8a8_pair, clock ticks = s_memtime read by waves 0 and 4 of every workgroup in the "
                              "last of 440 launches; real time = s_memrealtime (100 MHz); instrumented build "
                              "(libmi355_int8_timeline.so), five clock reads a wave outside the stage loop"}), flush=True)
    pool.destroy()
    dev.close()


def list_timeline(mi, wl, dev, s):
    """The batched GEMM (k_w8a8_list) on the four cfg3 projections as one launch: 240 launches on the benchmark's
    codes, then the clock reads one more launch left for every tile of every workgroup: first stage begins, last
    stage issued, last store of the tile issued.  Measured twice: with the same weights every launch (they stay in
    the memory-side cache) and, under "with_weights_from_hbm", with four copies of the weights taken in turn (as the
    timed step of the bench does)."""
    import ctypes as C
    lib = mi.lib
    M = wl.PREFILL_M
    shapes = [(M, 6144, 4096), (M, 14336, 4096), (M, 14336, 4096), (M, 4096, 14336)]
    mark = dev.mark()
    ops, copies = [], []
    for i, (_, N, K) in enumerate(shapes):
        m2 = dev.mark()
        qx, sx = dev.empty((M, K), np.int8), dev.empty(M, np.float32)
        mi.fwht_quant(dev.upload(wl.activations(2025, M, K, stream=K)), qx, sx, wl.HADAMARD_BLOCK)
        qw, sw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
        mi.fwht_quant(dev.upload(wl.weights(2025, N, K, stream=K + N + i)), qw, sw, wl.HADAMARD_BLOCK)
        dev.sync()
        host = [dev.download(b) for b in (qx, sx, qw, sw)]
        dev.reset_to(m2)
        ops.append(tuple(dev.upload(h) for h in host) + (dev.empty((M, N), np.float32),))
        copies.append([(ops[-1][2], ops[-1][3])] + [(dev.upload(host[2]), dev.upload(host[3])) for _ in range(3)])
    batch = mi.GemmBatch(dev, shapes)
    f = lib.mi_debug_gemm_list_timeline
    f.restype, f.argtypes = C.c_int32, [C.c_void_p, C.c_int32, C.c_int32]
    turn = [0]

    def launch_ops(rotate):
        if not rotate:
            return ops
        turn[0] += 1
        return [(o[0], o[1]) + c[turn[0] % 4] + (o[4],) for o, c in zip(ops, copies)]

    res = measure_list_timeline(mi, dev, s, batch, f, lambda: launch_ops(False))
    res["with_weights_from_hbm"] = measure_list_timeline(mi, dev, s, batch, f, lambda: launch_ops(True))
    batch.destroy()
    dev.reset_to(mark)
    return res


def measure_list_timeline(mi, dev, s, batch, f, next_ops):
    for _ in range(200):
        batch.run_f32(next_ops(), stream=s)
    e0, e1 = mi.Event(), mi.Event()
    e0.record(s)
    for _ in range(40):
        batch.run_f32(next_ops(), stream=s)
    e1.record(s)
    e1.synchronize()
    us = e0.elapsed_ms(e1) / 40 * 1e3
    WGS, TILES = 512, 16
    mi.check(f(None, 0, 1))
    batch.run_f32(next_ops(), stream=s)
    dev.sync(s)
    buf = np.zeros(WGS * TILES * 8, np.uint64)
    mi.check(f(buf.ctypes.data, buf.size, 0))
    t = buf.reshape(WGS, TILES, 8).astype(np.int64)
    valid = (t[:, :, 6] & 1) == 1
    wgs = int(valid.any(axis=1).sum())
    nk = t[:, :, 5][valid]
    loop = (t[:, :, 1] - t[:, :, 0])[valid]
    fin = (t[:, :, 2] - t[:, :, 1])[valid]
    real_us = (t[:, :, 4] - t[:, :, 3])[valid] / 100.0
    wait = (t[:, :, 7] & 0xffffffff)[valid]      # wave 0: ticks in the wait for its own loads in front of the stage's barrier
    bar = (t[:, :, 7] >> 32)[valid]              # ... and in the barrier itself (each includes one clock read)
    wait1 = (t[:, :, 6] >> 8)[valid]             # ... the wait of a tile's second stage alone: the first that must see
                                                 # the stores of the tile before acknowledged (loads complete in order)
    first = np.broadcast_to(np.arange(TILES)[None, :] == 0, valid.shape)[valid]
    per_k = {}
    for k in np.unique(nk):
        sel = nk == k
        rec = {"tiles": int(sel.sum()), "loop_ticks_per_stage": round(float(loop[sel].mean() / k)),
               "tile_us": round(float(real_us[sel].mean()), 2),
               "of_a_stage_wave0_waits_for_its_loads_ticks": round(float(wait[sel].mean() / k)),
               "of_a_stage_wave0_waits_in_the_barrier_ticks": round(float(bar[sel].mean() / k))}
        for name, which in (("first_tile_of_a_workgroup", first), ("later_tiles", ~first)):
            if (sel & which).any():
                rec["loop_ticks_per_stage_" + name] = round(float(loop[sel & which].mean() / k))
        per_k["stages_%d" % k] = rec
    start = t[:, :, 3][valid].min()
    ends = np.array([t[w, np.where(valid[w])[0][-1], 4] for w in range(WGS) if valid[w].any()])
    res = {"kernel_us_event": round(us, 2), "workgroups": wgs, "tiles": int(valid.sum()),
           "clock_mhz": round(float(((t[:, :, 2] - t[:, :, 0])[valid] / real_us).mean())),
           "per_tile_depth": per_k, "mfma_per_simd_and_stage": 4 * 8 * 2 * 2,
           "convert_and_store_ticks_per_tile": round(float(fin.mean())),
           "second_stage_wait_ticks_of_later_tiles": {"mean": round(float(wait1[~first].mean())),
                                                      "p90": round(float(np.percentile(wait1[~first], 90)))},
           "loop_ticks_all_tiles": int(loop.sum()), "convert_and_store_ticks_all_tiles": int(fin.sum()),
           "first_tile_start_to_last_store_us": round(float(ends.max() - start) / 100.0, 2),
           "workgroup_end_before_the_last_one_us": {"mean": round(float(ends.max() - ends.mean()) / 100.0, 2),
                                                    "p10": round(float(ends.max() - np.percentile(ends, 10)) / 100.0, 2)},
           "note": "k_w8a8_list, one launch over the four cfg3 projections; clock ticks = s_memtime read by wave 0 of "
                   "every workgroup at three points of every tile and around the wait and the barrier of every stage "
                   "(three reads a stage, about 100 ticks); instrumented build"}
    return res


def run_probe(exe_name, key):
    """Runs one of the measurement executables built by `make bench` (its own process) and returns its JSON line,
    or {key: None, reason} when it is not built or fails."""
    import subprocess
    exe = os.path.join(ROOT, "mojo-linuxperiments_amd", exe_name)
    if not os.path.exists(exe):
        return {key: None, "reason": "%s is not built (make -C mojo-linuxperiments_amd/csrc bench)" % exe_name}
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    if r.returncode != 0:
        return {key: None, "reason": "probe failed: " + r.stderr.strip()[-200:]}
    return json.loads(r.stdout.strip().splitlines()[-1])


def mfma_probe():
    """The matrix-pipe probe (csrc/probe_mfma_peak.hip).  Context for the roofline, never part of `value`."""
    return run_probe("mfma_peak_probe", "mfma_power_limited_peak")


VENDOR_CHILD = r"""
import json, os, sys
import numpy as np, torch
tmp, ncopy, warm = sys.argv[1], int(sys.argv[2]), int(sys.argv[3])
a = torch.from_numpy(np.load(os.path.join(tmp, "x.npy"))).cuda()
wh = np.load(os.path.join(tmp, "w.npy"))
ws = [torch.from_numpy(wh).cuda().t() for _ in range(ncopy)]   # [K, N] views of row-major [N, K]: A . B^T
for i in range(warm):
    torch._int_mm(a, ws[i % ncopy])
torch.cuda.synchronize()
e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
e0.record()
for i in range(40):
    torch._int_mm(a, ws[i % ncopy])
e1.record()
torch.cuda.synchronize()
np.save(os.path.join(tmp, "acc.npy"), torch._int_mm(a, ws[0]).cpu().numpy())
print(json.dumps({"us": round(e0.elapsed_time(e1) / 40 * 1e3, 2)}))
"""


def vendor_gemm(mi, wl):
    """Context, not a target: torch._int_mm (hipBLASLt underneath) on the cfg3 shapes with the codes this library's
    own quantizer produces from the benchmark's activations and weights, timed like the headline (HIP events on the
    launch stream, about 60 ms of the same launches first, weights rotated through more than 256 MB)."""
    import subprocess
    import tempfile
    lib = mi.lib
    dev = mi.Device(arena_bytes=6 << 30)
    pool = mi.StreamPool(dev, 1)
    s = pool.stream(0)
    timer = Timer(mi, s)
    M = wl.PREFILL_M
    out = {}
    for name, K, N in (("qkv", 4096, 6144), ("gate_up", 4096, 14336), ("down", 14336, 4096)):
        mark = dev.mark()
        a = dev.upload(wl.activations(2025, M, K, stream=K))
        qx, sx = dev.empty((M, K), np.int8), dev.empty(M, np.float32)
        mi.fwht_quant(a, qx, sx, wl.HADAMARD_BLOCK)
        w = dev.upload(wl.weights(2025, N, K, stream=K + N))
        qw, sw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
        mi.fwht_quant(w, qw, sw, wl.HADAMARD_BLOCK)
        dev.sync()
        xh, wh = dev.download(qx), dev.download(qw)
        ncopy = MALL_BYTES // (N * K) + 2
        qws = [dev.upload(wh) for _ in range(ncopy)]
        acc = dev.empty((M, N), np.int32)
        y = dev.empty((M, N), np.float32)
        state = {"i": 0}

        def ours_i32():
            state["i"] = (state["i"] + 1) % ncopy
            mi.check(lib.mi_w8a8_gemm_i32(qx.ptr, qws[state["i"]].ptr, acc.ptr, M, N, K, s))

        def ours_f32():
            state["i"] = (state["i"] + 1) % ncopy
            mi.check(lib.mi_w8a8_gemm_dequant_f32(qx.ptr, sx.ptr, qws[state["i"]].ptr, sw.ptr, y.ptr, M, N, K, s))
        res = {}
        for tag, fn in (("this_library_dequant_f32_us", ours_f32), ("this_library_i32_us", ours_i32)):
            timer.settle(fn, 150.0)
            res[tag] = round(timer.run(fn, 40) * 1e3, 2)
        # torch brings its own HIP runtime, which finds no device once this library's runtime holds it: a child
        # process times the vendor GEMM on the same codes and hands back its accumulators' checksum
        mi.check(lib.mi_w8a8_gemm_i32(qx.ptr, qws[0].ptr, acc.ptr, M, N, K, s))
        dev.sync(s)
        ours = dev.download(acc)
        with tempfile.TemporaryDirectory() as tmp:
            np.save(os.path.join(tmp, "x.npy"), xh)
            np.save(os.path.join(tmp, "w.npy"), wh)
            warm = max(3, int(150e3 / max(res["this_library_i32_us"], 1.0)))
            child = subprocess.run([sys.executable, "-c", VENDOR_CHILD, tmp, str(ncopy), str(warm)],
                                   capture_output=True, text=True, timeout=600)
            if child.returncode != 0:
                raise SystemExit("vendor GEMM child failed:\n" + child.stderr[-2000:])
            got = json.loads(child.stdout.strip().splitlines()[-1])
            ref = np.load(os.path.join(tmp, "acc.npy"))
        res["torch_int_mm_i32_us"] = got["us"]
        res["accumulators_equal"] = bool(np.array_equal(ref, ours))
        ops = 2.0 * M * N * K
        res["this_library_i32_frac_of_peak"] = round(ops / res["this_library_i32_us"] / 1e6 / PEAK_INT8_TOPS, 4)
        res["torch_int_mm_frac_of_peak"] = round(ops / res["torch_int_mm_i32_us"] / 1e6 / PEAK_INT8_TOPS, 4)
        out[name] = res
        dev.reset_to(mark)
    pool.destroy()
    dev.close()
    print(json.dumps({"vendor_gemm_context": out, "M": M, "note": "torch._int_mm writes int32; this library's "
                      "dequantizing form writes fp32 (the same number of bytes)"}), flush=True)


def cfg0_linear(mi, wl, dev, s, timer, shapes):
    lib = mi.lib
    c = wl.CFG0
    M, K, N = c["M"], c["K"], c["N"]
    mark = dev.mark()
    w = dev.upload(wl.weights(5, N, K))
    q0, s0 = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
    mi.fwht_quant(w, q0, s0, wl.HADAMARD_BLOCK, stream=s)
    dev.sync(s)
    qh, sh = dev.download(q0, s), dev.download(s0, s)
    bufs = [(dev.upload(qh), dev.upload(sh)) for _ in range(MALL_BYTES // (N * K) + 2)]
    dx = dev.upload(wl.activations(5, M, K))
    y = dev.empty((M, N), np.float32)
    ws = dev.empty(lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    calls = [(lambda b=b: mi.check(lib.mi_w8a8_linear_f32(dx.ptr, b[0].ptr, b[1].ptr, y.ptr, M, N, K,
                                                         wl.HADAMARD_BLOCK, ws.ptr, ws.nbytes, s))) for b in bufs]
    ms = graph_time(mi, dev, s, timer, calls, 20)
    nbytes = wl.linear_algorithmic_bytes(M, N, K)
    dev.reset_to(mark)
    return {"cfg0_linear_m32": {"us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                "TOPS": round(wl.gemm_ops(M, N, K) / (ms * 1e-3) / 1e12, 2)}}


def decode_layer_chain(mi, wl, dev, s, timer, reps=10, batch=None, nlayers=3):
    """A decode step through decoder layers of the cfg1 / cfg2 shapes (hidden 4096, 32/8 heads of 128, FFN 14336,
    16 sequences with 4095 cached tokens each): three layers with their own weights (654 MB) and KV caches
    (417 MB) run one after the other, so that nothing a layer reads is left in the memory-side cache from its
    last turn; the three-layer step is recorded into a graph and replayed.  With nlayers > 3 (a whole stack: 32
    layers hold 7 GB of weights and 4.4 GB of caches) every layer still has its own weights and cache at its own
    address; the fp32 sources of the weights repeat with period three."""
    c = wl.ATTN
    B, Hq, Hkv, D, T = c["B"], c["Hq"], c["Hkv"], c["D"], c["T"]
    if batch is not None:
        B = batch
    H, I = 4096, 14336
    mark = dev.mark()
    inv = 10000.0 ** (-np.arange(D // 2, dtype=np.float64) * 2.0 / D)
    ang = np.arange(T, dtype=np.float64)[:, None] * inv[None, :]
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    g1 = np.ones(H, np.float32)
    layers = []
    wsrc, csrc = {}, {}
    for li in range(nlayers):
        if li % 3 not in wsrc:
            wsrc[li % 3] = [wl.weights(500 + li, n, k, i) for i, (n, k) in
                            enumerate((((Hq + 2 * Hkv) * D, H), (H, Hq * D), (2 * I, H), (H, I)))]
            csrc[li % 3] = wl.normal(600 + li, (B * Hkv * T, D), 0)
        w = wsrc[li % 3]
        L = mi.DecoderLayer(dev, B, H, Hq, Hkv, I, T, w[0], w[1], w[2], w[3], g1, g1, cos, sin, tiled=True)
        if li + 3 >= nlayers:
            wsrc[li % 3] = None
        # a cache of real rows: rotate + quantize N(0,1) keys and values
        m2 = dev.mark()
        src = dev.upload(csrc[li % 3])
        L.fill_cache_from_rows(src, T, s)
        dev.sync(s)
        dev.reset_to(m2)
        layers.append(L)
    x = dev.upload(wl.activations(700, B, H))
    out = dev.empty((B, H), np.float32)
    dpos, dlen = dev.upload(np.full(B, T - 1, np.int32)), dev.upload(np.full(B, T, np.int32))

    def step():
        # inside the stack a layer's closing residual add is done by the next layer's first kernel
        layers[0].step(x, dpos, dlen, T, None, s)
        for li in range(1, nlayers):
            layers[li].step(layers[li - 1].dn, dpos, dlen, T, out if li == nlayers - 1 else None, s,
                            residual=layers[li - 1].h1)
    ms = graph_time(mi, dev, s, timer, [step], reps) / len(layers)
    wbytes = ((Hq + 2 * Hkv) * D * H + H * Hq * D + 2 * I * H + H * I)
    nbytes = wbytes + wl.attention_algorithmic_bytes(B, Hq, Hkv, D, T)
    dev.reset_to(mark)
    res = {"us_per_layer": round(ms * 1e3, 2), "kernels_per_layer": 10 if B > 1 else 8, "layers_in_graph": nlayers,
           "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
           "tokens_per_s_per_layer": round(B / (ms * 1e-3), 1), "algorithmic_bytes": nbytes}
    if nlayers == 3:
        res["tokens_per_s_32_layers"] = round(B / (32 * ms * 1e-3), 1)        # extrapolated from three layers
        return {"decode_layer_b%d_t4096" % B: res}
    res["us_per_step"] = round(ms * 1e3 * nlayers, 1)                           # measured: the stack is one graph
    res["tokens_per_s"] = round(B / (nlayers * ms * 1e-3), 1)
    return {"decode_stack_%d_layers_b%d_t4096" % (nlayers, B): res}


def moe_decode_layer_chain(mi, wl, dev, s, timer, reps=10, nlayers=3):
    """A decode step through decoder layers whose FFN is the cfg4 MoE (hidden 2048, 16/4 heads of 128, 128 experts
    top-8, inner 768), 16 sequences with 4095 cached tokens each: three layers with their own weights (1.8 GB of
    experts) and caches, one graph.  With 16 tokens x 8 picks about two thirds of the experts are hit per layer."""
    c, m = wl.ATTN, wl.MOE
    B, D, T = c["B"], c["D"], c["T"]
    H, E, topk, I = m["H"], m["E"], m["topk"], m["I"]
    Hq, Hkv = H // D, max(1, H // D // 4)
    mark = dev.mark()
    inv = 10000.0 ** (-np.arange(D // 2, dtype=np.float64) * 2.0 / D)
    ang = np.arange(T, dtype=np.float64)[:, None] * inv[None, :]
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    g1 = np.ones(H, np.float32)
    lib = mi.lib
    layers = []
    for li in range(nlayers):
        wq = wl.weights(800 + li, (Hq + 2 * Hkv) * D, H, 0)
        wo = wl.weights(800 + li, H, Hq * D, 1)
        moe = {"wr": wl.weights(800 + li, E, H, 2), "topk": topk}
        for name, n, k, b, st in (("g", I, H, wl.HADAMARD_BLOCK, 3), ("u", I, H, wl.HADAMARD_BLOCK, 4),
                                  ("d", H, I, wl.MOE_INNER_BLOCK, 5)):
            m2 = dev.mark()
            q, sc = dev.empty((E, n, k), np.int8), dev.empty((E, n), np.float32)
            keep = dev.mark()
            w = dev.upload(wl.weights(800 + li, E * n, k, st))
            mi.check(lib.mi_fwht_quant_f32_i8(w.ptr, q.ptr, sc.ptr, E * n, k, b, s))
            dev.sync(s)
            dev.reset_to(keep)
            moe["w" + name], moe["s" + name] = q, sc
        L = mi.DecoderLayer(dev, B, H, Hq, Hkv, I, T, wq, wo, None, None, g1, g1, cos, sin, tiled=True, moe=moe)
        m2 = dev.mark()
        src = dev.upload(wl.normal(900 + li, (B * Hkv * T, D), 0))
        L.fill_cache_from_rows(src, T, s)
        dev.sync(s)
        dev.reset_to(m2)
        layers.append(L)
    x = dev.upload(wl.activations(701, B, H))
    out = dev.empty((B, H), np.float32)
    dpos, dlen = dev.upload(np.full(B, T - 1, np.int32)), dev.upload(np.full(B, T, np.int32))

    def step():
        layers[0].step(x, dpos, dlen, T, None, s)
        for li in range(1, nlayers):
            layers[li].step(layers[li - 1].dn, dpos, dlen, T, out if li == nlayers - 1 else None, s,
                            residual=layers[li - 1].h1)
    ms = graph_time(mi, dev, s, timer, [step], reps) / nlayers
    dev.reset_to(mark)
    return {"decode_layer_moe_b%d_t4096" % B: {
        "us_per_layer": round(ms * 1e3, 2), "layers_in_graph": nlayers, "tokens_per_s_per_layer": round(B / (ms * 1e-3), 1),
        "shape": "hidden %d, %d/%d heads, %d experts top-%d, inner %d" % (H, Hq, Hkv, E, topk, I),
        "expert_weight_bytes_per_layer": wl.moe_weight_bytes(E, H, I)}}


def host_staging(mi, wl, dev, s, timer):
    """The host-buffer variant of the boundary for the cfg3 QKV linear: activations fp32 [2048,4096] in from a
    pinned staging slab and the fp32 [2048,6144] result back out, over the host link.  Never part of `value`."""
    import ctypes as C
    lib = mi.lib
    M, K, N = wl.PREFILL_M, 4096, 6144
    nin, nout = 4 * M * K, 4 * M * N
    h = C.c_void_p()
    mi.check(lib.mi_host_arena_create(dev.ctx, nin + nout + 4096, 256, 0, C.byref(h)), "mi_host_arena_create")
    hin, hout = lib.mi_arena_alloc(h, nin), lib.mi_arena_alloc(h, nout)
    mark = dev.mark()
    din, dout = dev.empty((M, K), np.float32), dev.empty((M, N), np.float32)
    ms_in = timer.run(lambda: mi.check(lib.mi_memcpy_h2d(din.ptr, hin, nin, s)), 10)
    ms_out = timer.run(lambda: mi.check(lib.mi_memcpy_d2h(hout, dout.ptr, nout, s)), 10)
    dev.reset_to(mark)
    mi.check(lib.mi_arena_destroy(h))
    return {"host_staging_cfg3_qkv": {"h2d_us": round(ms_in * 1e3, 1), "h2d_GBps": round(nin / (ms_in * 1e-3) / 1e9, 1),
                                      "d2h_us": round(ms_out * 1e3, 1), "d2h_GBps": round(nout / (ms_out * 1e-3) / 1e9, 1)}}


def node_cpu_lists():
    """{node: [cpus]} from /sys/devices/system/node/node*/cpulist, the files the upstream NumaInfo parses
    (numa/numa.mojo:107-115), restricted to the CPUs this process may run on."""
    allowed = os.sched_getaffinity(0)
    nodes = {}
    base = "/sys/devices/system/node"
    try:
        names = sorted(n for n in os.listdir(base) if n.startswith("node") and n[4:].isdigit())
    except OSError:
        names = []
    for n in names:
        try:
            txt = open(os.path.join(base, n, "cpulist")).read().strip()
        except OSError:
            continue
        cpus = []
        for part in filter(None, txt.split(",")):
            lo, _, hi = part.partition("-")
            cpus.extend(range(int(lo), int(hi or lo) + 1))
        cpus = [c for c in cpus if c in allowed]
        if cpus:
            nodes[int(n[4:])] = cpus
    if not nodes:
        nodes[0] = sorted(allowed)
    return nodes


def cpu_baseline(wl):
    """The CPU oracle (a builder-written port; upstream has no CPU kernels for this path) on the host cores, one
    OpenMP thread per core, each pinned to a CPU of its NUMA node as the upstream pool pins its workers
    (threading/linux_threading.mojo:89-91).  The headline workload (the four cfg3 linears at M = 2048: rotate +
    quantize, int8 GEMM, dequant) runs for about 6 s; cfg0, cfg1, cfg2 and cfg4 follow on bounded samples (a few
    calls each), about 20 s in all."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import ctypes as C
    import cpu_oracle as orc
    nodes = node_cpu_lists()
    nth = orc.num_threads()
    # threads are dealt to the nodes in turn, inside a node to its CPUs in turn
    order, depth = [], 0
    while len(order) < nth:
        took = False
        for n in sorted(nodes):
            if depth < len(nodes[n]) and len(order) < nth:
                order.append(nodes[n][depth])
                took = True
        depth += 1
        if not took:
            depth = 0
            if not any(nodes.values()):
                break
    pinned = orc.pin_threads(order) if order else 0
    M = wl.PREFILL_M
    g = np.random.default_rng(3)
    ptr = lambda a: a.ctypes.data_as(C.c_void_p)
    lib = orc.lib()

    def linear_call(x, qw, sw, bufs):
        Mx, K = x.shape
        N = qw.shape[0]
        y, qx, sx, acc = bufs
        rc = lib.orc_w8a8_linear(ptr(x), ptr(qw), ptr(sw), ptr(y), C.c_int64(Mx), C.c_int64(N), C.c_int64(K),
                                 C.c_int(128), ptr(qx), ptr(sx), ptr(acc))
        assert rc == 0

    def bufs_for(Mx, N, K):   # outputs allocated and touched once, as a resident caller's are
        return (np.zeros((Mx, N), np.float32), np.zeros((Mx, K), np.int8), np.zeros(Mx, np.float32),
                np.zeros((Mx, N), np.int32))

    def timed(fn, budget_s, max_calls=10000):
        fn()   # first touch
        n, dt = 0, 0.0
        while dt < budget_s and n < max_calls:
            t0 = time.perf_counter()
            fn()
            dt += time.perf_counter() - t0
            n += 1
        return dt / n, n

    xs = {K: wl.activations(1, M, K, stream=K) for K in (4096, 14336)}
    ws = {}
    for name, K, N in wl.PROJECTIONS:
        if (K, N) not in ws:
            ws[(K, N)] = (g.integers(-127, 128, (N, K), dtype=np.int8), np.full(N, 0.001, np.float32))
    orc.rotate_quant_rows(xs[4096][:64], 128)          # load the library, spin up the OpenMP team
    outs = {(K, N): bufs_for(M, N, K) for _, K, N in wl.PROJECTIONS}

    def cfg3_step():
        for name, K, N in wl.PROJECTIONS:
            linear_call(xs[K], ws[(K, N)][0], ws[(K, N)][1], outs[(K, N)])
    per_step, passes = timed(cfg3_step, 6.0, 400)
    step_ops = sum(wl.gemm_ops(M, N, K) for _, K, N in wl.PROJECTIONS)
    per = {}
    # cfg1: decode GEMV sweep (rotate + quantize + contraction + dequant per call; bytes = the GPU leg's)
    cfg1 = {}
    for Mx in wl.DECODE_BATCHES:
        row = {}
        for name, K, N in wl.PROJECTIONS:
            x = np.ascontiguousarray(xs[K][:Mx])
            b = bufs_for(Mx, N, K)
            sec, n = timed(lambda: linear_call(x, ws[(K, N)][0], ws[(K, N)][1], b), 0.25, 50)
            row[name] = {"us": round(sec * 1e6, 1), "GBps": round(wl.linear_algorithmic_bytes(Mx, N, K) / sec / 1e9, 1)}
        cfg1["M%d" % Mx] = row
    per["cfg1_decode_gemv"] = cfg1
    outs = None
    # cfg0: the single rotated linear at M = 32
    K0 = N0 = 4096
    x0, b0 = np.ascontiguousarray(xs[4096][:32]), bufs_for(32, N0, K0)
    w0 = (g.integers(-127, 128, (N0, K0), dtype=np.int8), np.full(N0, 0.001, np.float32))
    sec, n = timed(lambda: linear_call(x0, w0[0], w0[1], b0), 1.0, 200)
    per["cfg0_linear_m32"] = {"us": round(sec * 1e6, 1),
                              "GBps": round(wl.linear_algorithmic_bytes(32, N0, K0) / sec / 1e9, 1),
                              "TOPS": round(wl.gemm_ops(32, N0, K0) / sec / 1e12, 3)}
    # cfg2: decode attention over an int8 cache (codes straight from the generator: the time does not depend on them)
    c = wl.ATTN
    B, Hq, Hkv, D, T = c["B"], c["Hq"], c["Hkv"], c["D"], c["T"]
    kq = g.integers(-127, 128, (B, Hkv, T, D), dtype=np.int8)
    vq = g.integers(-127, 128, (B, Hkv, T, D), dtype=np.int8)
    ks = np.full((B, Hkv, T), 0.03, np.float32)
    q = wl.normal(88, (B, Hq, D), 1)
    sec, n = timed(lambda: orc.gqa_decode(q, kq, ks, vq, ks), 1.5, 50)
    nbytes = wl.attention_algorithmic_bytes(B, Hq, Hkv, D, T)
    per["cfg2_decode_attention"] = {"us": round(sec * 1e6, 1), "GBps": round(nbytes / sec / 1e9, 1),
                                    "tokens_per_s": round(B / sec, 1)}
    kq = vq = None
    # cfg4: the MoE layer (router + dispatch + grouped expert FFN)
    mc = wl.MOE
    Tm, H, E, topk, I = mc["T"], mc["H"], mc["E"], mc["topk"], mc["I"]
    xm = wl.activations(5, Tm, H)
    wr = (0.02 * g.standard_normal((E, H))).astype(np.float32)
    wg, wu = g.integers(-127, 128, (E, I, H), dtype=np.int8), g.integers(-127, 128, (E, I, H), dtype=np.int8)
    wd = g.integers(-127, 128, (E, H, I), dtype=np.int8)
    sg, sd = np.full((E, I), 0.001, np.float32), np.full((E, H), 0.001, np.float32)

    def moe_call():
        idx, w = orc.moe_route(xm, wr, topk)
        orc.moe_ffn(xm, idx, w, wg, sg, wu, sg, wd, sd, 128, 256)
    sec, n = timed(moe_call, 2.0, 20)
    wbytes = wl.moe_weight_bytes(E, H, I)
    per["cfg4_moe_layer"] = {"us": round(sec * 1e6, 1), "GBps": round(wbytes / sec / 1e9, 1),
                             "TOPS": round(wl.moe_ops(Tm, topk, H, I) / sec / 1e12, 3),
                             "tokens_per_s": round(Tm / sec, 1)}
    topo = host_topology()
    return {"value": round(step_ops / per_step / 1e12, 4), "unit": "TOPS", "cores": nth, "kind": "port",
            "numa_nodes": topo["numa_nodes"], "threads_pinned": pinned,
            "pinning": "one OpenMP thread per core, dealt to the NUMA nodes in turn and pinned to a CPU of its node "
                       "(node CPU lists from /sys/devices/system/node/node*/cpulist)",
            "sample": "the cfg3 step (four rotated W8A8 linears at M=2048: rotate+quant, int8 GEMM, dequant) x %d, "
                      "%.1f s, OpenMP C, int8 GEMM %s; per_config: a few calls of each other config (0.25 - 2 s each)" % (
                          passes, per_step * passes,
                          "blocked AVX-512 VNNI (4x6 register tiles)" if lib.orc_gemm_uses_vnni()
                          else "auto-vectorized dot products"),
            "per_config": per}


if __name__ == "__main__":
    main()
