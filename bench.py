#!/usr/bin/env python3
"""Benchmark of the arbitrary-bit quantized GEMM hot path on one MI355X.

Workload (BASELINE.json configs[1]): W2A8 signed decode GEMMs on the LLaMA-7B linears,
M in {1, 4, 8} x (N, K) in {(4096, 4096), (11008, 4096), (4096, 11008)} = 9 GEMMs per step,
int32 output, operands packed and resident in HBM.  Synthetic data: activations N(0, 32) clipped
to int8, weights uniform 2-bit, packed into bit planes (the reference's wire format) and from
there into the library's K-tiled layout: the same bits in another order, weights converted once
as a model loader does, activations in the order the quantising kernel writes them.  The same
GEMMs on the plane operands themselves are timed beside it (extra.decode_plane_operands).

The 256 MB Infinity Cache is defeated by rotation: every shape owns >= 512 MiB of distinct
weight buffers and consecutive launches walk through them, so a buffer is revisited only after
more than the cache's capacity of other weights has streamed through.

Timed region: exactly K steps, a step being one launch of each of the 9 GEMMs in turn, replayed from one HIP
graph so the host launch rate does not bound the measurement, bracketed by one pair of HIP events on the launch
stream: the average launch duration of the roofline is that interval over 9 K launches.  The per-GEMM rows on
stderr come from one graph per GEMM (K launches of it), replayed after the timed region.

Prints ONE short JSON line on stdout.  Progress and the side measurements go to stderr, the side measurements also
as JSON into the file --extra-out names (default: bench_extra.json in the output folder beside this script).
"""
import argparse
import importlib.util
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X dense int8
SHAPES = [(4096, 4096), (11008, 4096), (4096, 11008)]
MS = [1, 4, 8]
Q_BITS, P_BITS, SIGNED = 8, 2, True
ROTATE_BYTES = 512 << 20


# HBM bytes per launch of the dominant kernel come from the rocprofv3 --pmc summary kept under profiles/ (two counter
# runs of this script scaled by a plain copy of known size): the summary carries one line
# `bench.py reads: kernel=<family> traffic_bytes_per_launch=<n>` (the kernel trace: `avg_dispatch_ns=<n>`) per measured
# kernel family, and the figure is reported only for the family it was taken on.
PROFILE_SUMMARIES = ("decode_w2a8_prepared_bench_hbm_traffic.md", "decode_w2a8_prepared_bench_kernel_trace.md")
LINE_LIMIT = 4096  # the one stdout line must stay far below what a log tail keeps


def profile_figures(family, directory=None):
    """{'traffic_bytes_per_launch': n, 'avg_dispatch_ns': n, 'source': [...]} for a kernel family, from profiles/*.md."""
    directory = directory or os.path.join(ROOT, "profiles")
    out = {}
    for name in PROFILE_SUMMARIES:
        try:
            text = open(os.path.join(directory, name)).read()
        except OSError:
            continue
        for line in text.splitlines():
            if "bench.py reads:" not in line:
                continue
            fields = dict(f.split("=", 1) for f in line.split("bench.py reads:", 1)[1].replace("`", " ").split() if "=" in f)
            if fields.get("kernel") != family:
                continue
            for key in ("traffic_bytes_per_launch", "avg_dispatch_ns"):
                if key in fields:
                    out[key] = int(fields[key])
                    out.setdefault("source", []).append("profiles/" + name)
    return out


def headline(value, steps, warmup, total_s, n_gemms, clock_settle_s, dominant, tuples, launches, bytes_per_launch,
             avg_launch_us, cpu_tops, cpu_threads, cpu_sample, plane_operand_tops=None, extra_file=None, figures=None):
    """The one JSON object bench.py prints on stdout.  Side measurements never go in here: they are written to a file
    of their own (and logged on stderr), so that this line stays a few hundred bytes."""
    figures = profile_figures(dominant) if figures is None else figures
    achieved = bytes_per_launch / (avg_launch_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": figures.get("traffic_bytes_per_launch"),
                "kernel": dominant + ":" + ",".join(sorted(set(t.split(":")[1] for t in tuples))),
                "launches_per_step": launches,
                "algorithmic_bytes_per_launch_avg": round(bytes_per_launch),
                "avg_launch_us": round(avg_launch_us, 3)}
    if "avg_dispatch_ns" in figures:
        # an isolated dispatch under the profiler (no overlap with the next launch's ramp): the conservative figure
        iso = bytes_per_launch / (figures["avg_dispatch_ns"] * 1e-9) / 1e9
        roofline["kernel_trace_avg_us"] = round(figures["avg_dispatch_ns"] / 1e3, 3)
        roofline["frac_kernel_trace"] = round(iso / HBM_PEAK_GBS, 4)
    result = {
        "metric": "effective int TOPS (2*M*N*K / t) over the LLaMA-7B W2A8 decode GEMMs, M in {1,4,8}",
        "value": round(value, 4),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(total_s * 1e3 / steps, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",  # packed fields unpacked to int8, int8 MFMA with int32 accumulation
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: W2A8 signed decode GEMM, M in {1,4,8} x (N,K) in "
                               "{(4096,4096),(11008,4096),(4096,11008)}, int32 out, packed operands resident in HBM "
                               "(K-tiled layout: weights prepared once, activations as the quantising kernel writes them)",
                   "gemms_per_step": n_gemms, "x_bits": Q_BITS, "w_bits": P_BITS, "signed": SIGNED,
                   "clock_settle_s": clock_settle_s},
        "roofline": roofline,
        "cpu_baseline": {"value": round(cpu_tops, 5), "unit": "TOPS", "cores": int(cpu_threads), "kind": "port",
                         "sample": cpu_sample},
    }
    if plane_operand_tops is not None:  # the same GEMMs on the reference's plane layout (what this line measured at first)
        result["plane_operands_value"] = round(plane_operand_tops, 4)
    if extra_file:
        result["extra_file"] = extra_file
    line = json.dumps(result)
    assert len(line) < LINE_LIMIT, "headline line grew to %d bytes" % len(line)
    return line


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def load_binding():
    spec = importlib.util.spec_from_file_location("abq_gemm", os.path.join(ROOT, "abq-llm_amd", "abq_gemm.py"))
    mod = importlib.util.module_from_spec(spec)
    sys.modules["abq_gemm"] = mod
    spec.loader.exec_module(mod)
    return mod


def random_planes(torch, shape):
    """Bit planes of uniformly random values are uniformly random words."""
    lo = torch.randint(0, 1 << 16, shape, dtype=torch.int32, device="cuda")
    hi = torch.randint(0, 1 << 16, shape, dtype=torch.int32, device="cuda")
    return lo | (hi << 16)


CLOCK_SETTLE_S = 0.3  # untimed load in front of the headline's warm-up steps


def settle(replay, seconds=0.05):
    """Untimed calls of `replay` until the chip has been under that load for `seconds`.  The first launch of a graph
    uploads it, and a chip that has idled (behind host work) takes tens of milliseconds of load to reach the clock it
    sustains: a GEMM timed right after one untimed replay measured up to 17 % slower than the same GEMM timed later."""
    import torch
    t0 = time.perf_counter()
    while True:
        replay()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 >= seconds:
            return


def algorithmic_bytes(M, N, K, q, p, out_bytes=4):
    return p * N * K // 8 + q * M * K // 8 + out_bytes * M * N


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--clock-settle-s", type=float, default=CLOCK_SETTLE_S,
                    help="untimed passes over the headline's launches in front of the warm-up steps, in seconds (0: none)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="plain stream launches instead of HIP graphs")
    ap.add_argument("--no-extra", action="store_true", help="skip the side measurements")
    ap.add_argument("--extras", default=None,
                    help="comma-separated side measurements to run (default all): decode_plane_operands, prefill, prefill_fp6, library_int8_gemm, "
                         "decode_fused_linears, decode_group_scales, small_batch, decoder_layer_w2a8_group128")
    ap.add_argument("--extra-out", default=os.path.join(ROOT, "gpurun_out", "bench_extra.json"),
                    help="file the side measurements are written to as JSON ('' for none); they never go on stdout")
    ap.add_argument("--pmc-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (the known-size kernel that "
                         "calibrates FETCH_SIZE / WRITE_SIZE in a counter run)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build measures one GPU; --gpus %d is not supported (the path would shard by "
            "splitting N, or K with an integer all-reduce, across GPUs; nothing here uses a second GPU)." % args.gpus)
        sys.exit(2)
    K_STEPS, W_STEPS = args.steps, args.warmup

    import numpy as np
    import torch
    abq = load_binding()
    abq.lib()  # fails loudly if the HIP library is not built
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    torch.manual_seed(0)
    dev_name = torch.cuda.get_device_name(0)
    log("device:", dev_name)

    # ---------------------------------------------------------------- synthetic operands
    weights, weights_tiled, xs, xs_tiled = {}, {}, {}, {}
    for (N, K) in SHAPES:
        wbytes = P_BITS * N * K // 8
        R = max(2, math.ceil(ROTATE_BYTES / wbytes))
        weights[(N, K)] = random_planes(torch, (R, P_BITS, N, K // 32))
        wt = torch.empty((R, K // 128, N, P_BITS, 4), dtype=torch.int32, device="cuda")
        for r in range(R):
            abq.relayout_planes(weights[(N, K)][r], out=wt[r])
        weights_tiled[(N, K)] = wt
    for K in sorted(set(k for _, k in SHAPES)):
        for M in MS:
            x = torch.clamp(torch.round(torch.randn(M, K, device="cuda") * 32.0), -128, 127).to(torch.int32)
            xs[(M, K)] = abq.pack_i32(x, Q_BITS)
            xs_tiled[(M, K)] = abq.relayout_planes(xs[(M, K)])
    torch.cuda.synchronize()

    cases = []
    for (N, K) in SHAPES:
        Wt = weights_tiled[(N, K)]
        for M in MS:
            out = torch.empty((M, N), dtype=torch.int32, device="cuda")
            gemms = [abq.Gemm(xs_tiled[(M, K)], Wt[r], SIGNED, out=out, x_tiled=True, w_tiled=True) for r in range(Wt.shape[0])]
            cases.append(dict(M=M, N=N, K=K, gemms=gemms, out=out, ops=2.0 * M * N * K,
                              bytes=algorithmic_bytes(M, N, K, Q_BITS, P_BITS),
                              kernel="%s:%s" % (gemms[0].strategy, gemms[0].config_name),
                              planes=(xs[(M, K)], weights[(N, K)][0])))

    def launch_group(case, count, offset=0):
        g = case["gemms"]
        for s in range(count):
            g[(offset + s) % len(g)].run()

    # ---------------------------------------------------------------- HIP graphs
    # The timed region is ONE graph that holds the K steps as they run in a model (GEMM 1 .. 9, then again), so a
    # replay's own launch cost is spread over 9 K launches; one graph per GEMM (K launches of it) gives the per-GEMM
    # rows afterwards, outside the timed region.
    use_graph = not args.no_graph
    graphs, step_graph = [], None

    def launch_steps(count, offset=0):
        for s in range(count):
            for case in cases:
                g = case["gemms"]
                g[(offset + s) % len(g)].run()

    if use_graph:
        try:
            launch_steps(2)
            torch.cuda.synchronize()
            step_graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(step_graph):
                launch_steps(K_STEPS)
            for case in cases:
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr):
                    launch_group(case, K_STEPS)
                graphs.append(gr)
        except Exception as e:  # noqa: BLE001
            log("HIP graph capture failed (%r); falling back to plain stream launches" % (e,))
            use_graph, graphs, step_graph = False, [], None
            torch.cuda.synchronize()

    if args.pmc_copy_mib:
        src = torch.empty(args.pmc_copy_mib << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------------------------------------------------------- warmup
    # First the chip is brought to the clock it sustains under this load (a chip that has idled takes tens of
    # milliseconds of work to get there; the first launch of a graph also uploads it): untimed passes over the same
    # launches for CLOCK_SETTLE_S, then the W warm-up steps of the contract.
    def one_pass():
        if use_graph:
            step_graph.replay()
        else:
            launch_steps(K_STEPS)
    if args.clock_settle_s > 0:
        settle(one_pass, args.clock_settle_s)
    launch_steps(W_STEPS, offset=7)
    torch.cuda.synchronize()

    # ---------------------------------------------------------------- timed region: exactly K steps
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    one_pass()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    total_s = t1 - t0
    timed_us_per_launch = e0.elapsed_time(e1) * 1e3 / (K_STEPS * len(cases))

    # ---------------------------------------------------------------- per-GEMM rows (outside the timed region)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in cases]
    if use_graph:
        settle(lambda: [gr.replay() for gr in graphs], 0.05)
    for i, case in enumerate(cases):
        ev[i][0].record()
        if use_graph:
            graphs[i].replay()
        else:
            launch_group(case, K_STEPS)
        ev[i][1].record()
    torch.cuda.synchronize()

    per_gemm = []
    groups = {}
    for i, case in enumerate(cases):
        us = ev[i][0].elapsed_time(ev[i][1]) * 1e3 / K_STEPS
        gbs = case["bytes"] / (us * 1e-6) / 1e9
        per_gemm.append(dict(M=case["M"], N=case["N"], K=case["K"], us=round(us, 3),
                             tops=round(case["ops"] / (us * 1e-6) / 1e12, 3), hbm_gbs=round(gbs, 1),
                             hbm_frac=round(gbs / HBM_PEAK_GBS, 4), kernel=case["kernel"]))
        g = groups.setdefault(case["kernel"], dict(us=0.0, bytes=0.0, launches=0))
        g["us"] += us
        g["bytes"] += case["bytes"]
        g["launches"] += 1
    # the headline GEMMs all run one kernel family (the tile tuple differs with the shape): one group
    families = {}
    for name, g in groups.items():
        f = families.setdefault(name.split(":")[0], dict(us=0.0, bytes=0.0, launches=0, tuples=[]))
        f["us"] += g["us"]
        f["bytes"] += g["bytes"]
        f["launches"] += g["launches"]
        f["tuples"].append(name)
    dominant = max(families, key=lambda k: families[k]["us"])
    dg = families[dominant]
    # launch duration of the dominant kernel: the timed region's own events when every GEMM of a step runs that kernel
    # family (the case), else the family's share of the per-GEMM rows
    avg_launch_us = timed_us_per_launch if len(families) == 1 else dg["us"] / dg["launches"]
    total_ops = sum(c["ops"] for c in cases) * K_STEPS
    value = total_ops / total_s / 1e12
    log("headline: %.2f TOPS over %d GEMMs x %d steps, %.3f us per launch in the timed region, %.3f as K launches per GEMM "
        "(rows are logged at the end)" % (value, len(cases), K_STEPS, avg_launch_us, dg["us"] / dg["launches"]))

    # ---------------------------------------------------------------- CPU baseline (bounded sample) + parity
    sys.path.insert(0, ROOT)
    from oracle import abq_oracle
    abq_oracle.build()
    host = []
    for case in cases:
        gm = case["gemms"][0]
        gm.run()
        torch.cuda.synchronize()
        host.append((case["planes"][0].cpu().numpy().view(np.uint32), case["planes"][1].cpu().numpy().view(np.uint32),
                     case["out"].cpu().numpy().copy()))
    cpu_ops, cpu_s, cpu_threads, reps = 0.0, 0.0, 1, 0
    while cpu_s < args.cpu_seconds and reps < 1000:
        for case, (xp, wp, gpu_out) in zip(cases, host):
            c0 = time.perf_counter()
            d, cpu_threads = abq_oracle.gemm_popc(xp, wp, SIGNED)
            cpu_s += time.perf_counter() - c0
            cpu_ops += case["ops"]
            if reps == 0:
                assert np.array_equal(d, gpu_out), "GPU result differs from the CPU oracle: %s" % case["kernel"]
        reps += 1
    xp, wp, gpu_out = host[0]  # M=1, 4096x4096: the reference's own single-threaded bit-serial loop
    c0 = time.perf_counter()
    d = abq_oracle.gemm_bitserial(xp, wp, SIGNED)
    bitserial_s = time.perf_counter() - c0
    assert np.array_equal(d, gpu_out)

    extra = {"per_gemm": per_gemm, "launch_mode": "hipgraph" if use_graph else "stream",
             "device": dev_name, "cache_defeat": "rotation over >=512 MiB of distinct weight buffers per shape",
             "cpu_bitserial_1core": {"tops": round(cases[0]["ops"] / bitserial_s / 1e12, 6),
                                     "sample": "M=1 N=4096 K=4096 once, engine/test_any_mma.cu compute_ref restated"}}

    # ---------------------------------------------------------------- side measurement: prefill shapes
    def want(name):
        return not args.no_extra and (args.extras is None or name in args.extras.split(","))

    if want("decode_plane_operands"):
        # the headline GEMMs with both operands in the reference's plane layout (what the engine API's callers hand
        # over): the decode kernel that expands planes in registers / LDS
        rows = []
        for case in cases:
            M, N, K = case["M"], case["N"], case["K"]
            Wr = weights[(N, K)]
            gs = [abq.Gemm(xs[(M, K)], Wr[r], SIGNED, out=case["out"]) for r in range(Wr.shape[0])]
            for r in range(4):
                gs[r % len(gs)].run()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                for r in range(100):
                    gs[r % len(gs)].run()
            settle(gr.replay)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            gr.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 100
            gbs = case["bytes"] / (us * 1e-6) / 1e9
            rows.append(dict(M=M, N=N, K=K, us=round(us, 3), hbm_gbs=round(gbs, 1), hbm_frac=round(gbs / HBM_PEAK_GBS, 4),
                             kernel="%s:%s" % (gs[0].strategy, gs[0].config_name)))
            log("plane operands M=%d N=%d K=%d  %.2f us  %.0f GB/s (%.1f%% of HBM peak)" % (M, N, K, us, gbs, 100 * gbs / HBM_PEAK_GBS))
            del gr, gs
        extra["decode_plane_operands"] = rows

    if want("prefill"):
        prefill = []
        for (q, p, signed) in [(8, 2, True), (4, 4, True), (4, 4, False), (8, 8, True), (8, 8, False)]:
            for (N, K) in SHAPES:
                wpl = random_planes(torch, (p, N, K // 32))
                wtl = abq.relayout_planes(wpl)  # weights prepared once in the K-tiled layout
                # (pairs with an unsigned 8-bit operand: the weights' row sums are prepared with them; the activations'
                # are taken inside the timed call when they arrive as planes, and come with them when they arrive tiled)
                u8 = not signed and 8 in (q, p)
                wrs = abq.row_sums(wpl) if u8 else None
                # unsigned W8A8: the weights as biased records (code - 128 written at preparation), which the signed
                # pair's kernel runs without flipping anything after its LDS reads
                biased = u8 and (q, p) == (8, 8)
                if biased:
                    wtl = abq.relayout_planes_biased(wpl)
                for M in (512, 2048):
                    xpl = random_planes(torch, (q, M, K // 32))
                    ws = torch.empty(xpl.numel() * 4 + 4 * M + 512, dtype=torch.uint8, device="cuda")
                    gm = abq.Gemm(xpl, wtl, signed, w_tiled=True, workspace=ws, w_row_sums=wrs,
                                  biased=(False, True) if biased else None)  # activations converted per call
                    gm.run()
                    torch.cuda.synchronize()
                    reps = 20  # (a replay's own launch cost is spread over the steps of the graph)
                    gr = torch.cuda.CUDAGraph()  # replayed like the decode GEMMs: no host launch cost in the figure
                    with torch.cuda.graph(gr):
                        for _ in range(reps):
                            gm.run()
                    settle(gr.replay)
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    gr.replay()
                    e1.record()
                    torch.cuda.synchronize()
                    us = e0.elapsed_time(e1) * 1e3 / reps
                    del gr
                    tops = 2.0 * M * N * K / (us * 1e-6) / 1e12
                    # the same GEMM with the activations already in the K-tiled layout, which is how the fused
                    # quantise + pack kernel hands them over: no conversion launch in the timed call
                    xtl = abq.relayout_planes_biased(xpl) if biased else abq.relayout_planes(xpl)
                    gt = abq.Gemm(xtl, wtl, signed, x_tiled=True, w_tiled=True, w_row_sums=wrs,
                                  x_row_sums=abq.row_sums(xpl) if u8 else None, biased=(True, True) if biased else None)
                    gt.run()
                    torch.cuda.synchronize()
                    gr = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(gr):
                        for _ in range(reps):
                            gt.run()
                    settle(gr.replay)
                    e0.record()
                    gr.replay()
                    e1.record()
                    torch.cuda.synchronize()
                    us_t = e0.elapsed_time(e1) * 1e3 / reps
                    del gr
                    tops_t = 2.0 * M * N * K / (us_t * 1e-6) / 1e12
                    prefill.append(dict(w_bits=p, x_bits=q, signed=signed, M=M, N=N, K=K, us=round(us, 1),
                                        tops=round(tops, 2), mfma_frac=round(tops / INT8_MFMA_PEAK_TOPS, 4),
                                        tiled_in=dict(us=round(us_t, 1), tops=round(tops_t, 2),
                                                      mfma_frac=round(tops_t / INT8_MFMA_PEAK_TOPS, 4)),
                                        kernel="%s:%s" % (gm.strategy, gm.config_name)))
                    del gm, gt, xpl, xtl, ws
                del wpl, wtl
        extra["prefill"] = prefill
        for r in prefill:
            log("prefill W%dA%d %s M=%d N=%d K=%d  %.1f us  %.1f TOPS (%.1f%% of int8 MFMA peak); tiled in %.1f us %.1f TOPS"
                % (r["w_bits"], r["x_bits"], "int" if r["signed"] else "uint", r["M"], r["N"], r["K"], r["us"],
                   r["tops"], 100 * r["mfma_frac"], r["tiled_in"]["us"], r["tiled_in"]["tops"]))

    if want("prefill_fp6"):
        # The same W4A4 GEMMs on the FP6 matrix-core route (exact for operands of at most 4 bits unsigned /
        # 5 bits signed): weights prepared once as FP6 records; activations either converted from planes inside
        # the timed call, as above, or already FP6 (what the fused quantise-and-pack kernel hands over).
        prefill_fp6 = []
        for signed in (True, False):
            for (N, K) in SHAPES:
                wf6 = abq.relayout_planes_fp6(random_planes(torch, (4, N, K // 32)), signed)
                for M in (512, 2048):
                    xpl = random_planes(torch, (4, M, K // 32))
                    xf6 = abq.relayout_planes_fp6(xpl, signed)
                    ws = torch.empty((K // 128) * M * 96, dtype=torch.uint8, device="cuda")
                    row = dict(w_bits=4, x_bits=4, signed=signed, M=M, N=N, K=K)
                    xsc = torch.rand(M, device="cuda") * 0.01 + 0.001
                    wsc = torch.rand(N, device="cuda") * 0.01 + 0.001
                    for tag, gm in (("planes_in", abq.Gemm(xpl, wf6, signed, w_fp6=4, workspace=ws)),
                                    ("fp6_in", abq.Gemm(xf6, wf6, signed, x_fp6=4, w_fp6=4)),
                                    # per-token x per-channel scales, fp16 out: the epilogue the model's linears use
                                    ("fp6_in_f16_scaled", abq.Gemm(xf6, wf6, signed, x_fp6=4, w_fp6=4, out_kind=abq.OUT_F16_SCALED,
                                                                   x_scale=xsc, w_scale=wsc))):
                        gm.run()
                        torch.cuda.synchronize()
                        reps = 20
                        gr = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(gr):
                            for _ in range(reps):
                                gm.run()
                        settle(gr.replay)
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record()
                        gr.replay()
                        e1.record()
                        torch.cuda.synchronize()
                        us = e0.elapsed_time(e1) * 1e3 / reps
                        del gr
                        tops = 2.0 * M * N * K / (us * 1e-6) / 1e12
                        row[tag] = dict(us=round(us, 1), tops=round(tops, 2), mfma_int8_frac=round(tops / INT8_MFMA_PEAK_TOPS, 4))
                        row["kernel"] = "%s:%s" % (gm.strategy, gm.config_name)
                        del gm
                    prefill_fp6.append(row)
                    log("prefill FP6 W4A4 %s M=%d N=%d K=%d  planes in %.0f  FP6 in %.0f  FP6 in, scaled fp16 out %.0f TOPS"
                        % ("int" if signed else "uint", M, N, K, row["planes_in"]["tops"], row["fp6_in"]["tops"],
                           row["fp6_in_f16_scaled"]["tops"]))
                    del xpl, xf6, ws, xsc, wsc
                del wf6
        extra["prefill_fp6"] = prefill_fp6

    if want("library_int8_gemm"):
        # Yardstick for the prefill figures: the vendor library's plain int8 GEMM (torch._int_mm, operands
        # already int8 and K-major, nothing to unpack) on the same shapes, timed the same way.
        vendor = []
        try:
            for (N, K) in SHAPES:
                for M in (512, 2048):
                    a8 = torch.randint(-128, 128, (M, K), dtype=torch.int8, device="cuda")
                    b8 = torch.randint(-128, 128, (N, K), dtype=torch.int8, device="cuda").t()
                    # timed like our own GEMMs: a graph of reps launches (eager launches of so short a kernel would
                    # measure the host), replayed until the chip is at its sustained clock, then once more with events;
                    # eager launches if the library cannot be captured
                    reps = 20
                    out8 = torch._int_mm(a8, b8)
                    torch.cuda.synchronize()
                    try:
                        gr = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(gr):
                            for _ in range(reps):
                                torch._int_mm(a8, b8, out=out8)
                        run = gr.replay
                    except Exception:  # noqa: BLE001
                        torch.cuda.synchronize()

                        def run():
                            for _ in range(reps):
                                torch._int_mm(a8, b8, out=out8)
                    settle(run)
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    run()
                    e1.record()
                    torch.cuda.synchronize()
                    us = e0.elapsed_time(e1) * 1e3 / reps
                    tops = 2.0 * M * N * K / (us * 1e-6) / 1e12
                    vendor.append(dict(M=M, N=N, K=K, us=round(us, 1), tops=round(tops, 2),
                                       mfma_frac=round(tops / INT8_MFMA_PEAK_TOPS, 4)))
                    del a8, b8, out8
        except Exception as exc:  # the yardstick is optional: a torch build without int8 matmul only loses this entry
            vendor = {"unavailable": repr(exc)[:120]}
        extra["library_int8_gemm"] = vendor

    def time_rotating(gs, reps=100):
        """us per launch of the GEMMs in gs run round robin, HIP-graph replay"""
        for r in range(4):
            gs[r % len(gs)].run()
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for r in range(reps):
                gs[r % len(gs)].run()
        settle(gr.replay)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        gr.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    def tiled_copies(Wr):
        wt = torch.empty((Wr.shape[0], Wr.shape[3] // 4, Wr.shape[2], Wr.shape[1], 4), dtype=torch.int32, device="cuda")
        for r in range(Wr.shape[0]):
            abq.relayout_planes(Wr[r], out=wt[r])
        return wt

    if want("decode_fused_linears"):
        # ------------------------------------------------------------ side measurement: several linears per launch
        # QKV (N = 3 * 4096) and gate + up (N = 2 * 11008) share their activations, so each is one GEMM
        # over concatenated weight planes: the launch + ramp cost is paid once for 12 or 22 MB.
        fused = []
        for name, N, K in (("qkv", 3 * 4096, 4096), ("gate_up", 2 * 11008, 4096)):
            wbytes = P_BITS * N * K // 8
            Wr = random_planes(torch, (max(2, math.ceil(ROTATE_BYTES / wbytes)), P_BITS, N, K // 32))
            Wt = tiled_copies(Wr)
            for M in MS:
                out = torch.empty((M, N), dtype=torch.int32, device="cuda")
                gs = [abq.Gemm(xs_tiled[(M, K)], Wt[r], SIGNED, out=out, x_tiled=True, w_tiled=True) for r in range(Wt.shape[0])]
                us = time_rotating(gs)
                us_planes = time_rotating([abq.Gemm(xs[(M, K)], Wr[r], SIGNED, out=out) for r in range(Wr.shape[0])])
                gbs = algorithmic_bytes(M, N, K, Q_BITS, P_BITS) / (us * 1e-6) / 1e9
                fused.append(dict(linears=name, M=M, N=N, K=K, us=round(us, 3), hbm_gbs=round(gbs, 1),
                                  hbm_frac=round(gbs / HBM_PEAK_GBS, 4), kernel="%s:%s" % (gs[0].strategy, gs[0].config_name),
                                  plane_operands_us=round(us_planes, 3)))
                log("fused %s M=%d N=%d K=%d  %.2f us  %.0f GB/s (%.1f%% of HBM peak); plane operands %.2f us"
                    % (name, M, N, K, us, gbs, 100 * gbs / HBM_PEAK_GBS, us_planes))
                del gs, out
            del Wr, Wt
        extra["decode_fused_linears"] = fused

    if want("decode_group_scales"):
        # ------------------------------------------------------------ side measurement: decode with the dequantising epilogue
        # group-128 weight scales and zero points, per-token scales, fp16 output, on prepared operands (the
        # group-scale variant of the decode kernel on K-tiled operands) and on plane operands beside it; bytes add
        # the scale and zero-point arrays to the packed weights
        deq = []
        for (N, K) in SHAPES:
            G = K // 128
            wbytes = P_BITS * N * K // 8
            Wr = weights[(N, K)]
            wsc = torch.rand((N, G), device="cuda") * 0.01 + 0.001
            wz = torch.randint(-2, 2, (N, G), device="cuda").float()
            for M in (1, 8):
                xsc = torch.rand(M, device="cuda") * 0.05 + 0.01
                sums = torch.randint(-1000, 1000, (M, G), dtype=torch.int32, device="cuda")
                out = torch.empty((M, N), dtype=torch.float16, device="cuda")
                kw = dict(out=out, out_kind=abq.OUT_F16_SCALED, x_scale=xsc, w_scale=wsc, group_size=128, w_zero=wz, x_group_sums=sums)
                Wt = weights_tiled[(N, K)]
                gs = [abq.Gemm(xs_tiled[(M, K)], Wt[r], SIGNED, x_tiled=True, w_tiled=True, **kw) for r in range(Wt.shape[0])]
                us = time_rotating(gs)
                us_planes = time_rotating([abq.Gemm(xs[(M, K)], Wr[r], SIGNED, **kw) for r in range(Wr.shape[0])])
                nbytes = algorithmic_bytes(M, N, K, Q_BITS, P_BITS, out_bytes=2) + 2 * N * G * 4
                gbs = nbytes / (us * 1e-6) / 1e9
                deq.append(dict(M=M, N=N, K=K, group_size=128, us=round(us, 3), hbm_gbs=round(gbs, 1),
                                hbm_frac=round(gbs / HBM_PEAK_GBS, 4), kernel="%s:%s" % (gs[0].strategy, gs[0].config_name),
                                plane_operands_us=round(us_planes, 3)))
                log("dequant decode M=%d N=%d K=%d  %.2f us  %.0f GB/s (%.1f%% of HBM peak)  %s; plane operands %.2f us"
                    % (M, N, K, us, gbs, 100 * gbs / HBM_PEAK_GBS, gs[0].strategy, us_planes))
                del gs, out
        # the same with 3-bit weights (what the reference's default 2-bit quantiser, bit balance, writes): as padded
        # 4-bit records on the prepared-operand kernel, and on plane operands
        deq3 = []
        for (N, K) in SHAPES:
            G = K // 128
            R3 = max(2, math.ceil(ROTATE_BYTES / (4 * N * K // 8)))
            w3 = random_planes(torch, (3, N, K // 32))
            w3p = abq.relayout_planes_padded(w3, SIGNED)
            Wp3 = w3p.unsqueeze(0).repeat(R3, 1, 1, 1, 1)
            W3 = w3.unsqueeze(0).repeat(R3, 1, 1, 1)
            wsc = torch.rand((N, G), device="cuda") * 0.01 + 0.001
            wz = torch.randint(-4, 4, (N, G), device="cuda").float()
            # (records of code - zero point, as wide as the padded ones: no zero points left to read)
            Wf3 = abq.relayout_planes_folded(w3, wz, 128, SIGNED).unsqueeze(0).repeat(R3, 1, 1, 1, 1)
            for M in (1, 8):
                xsc = torch.rand(M, device="cuda") * 0.05 + 0.01
                sums = torch.randint(-1000, 1000, (M, G), dtype=torch.int32, device="cuda")
                out = torch.empty((M, N), dtype=torch.float16, device="cuda")
                kw = dict(out=out, out_kind=abq.OUT_F16_SCALED, x_scale=xsc, w_scale=wsc, group_size=128, w_zero=wz, x_group_sums=sums)
                gs = [abq.Gemm(xs_tiled[(M, K)], Wp3[r], SIGNED, x_tiled=True, w_tiled=True, value_bits=(Q_BITS, 3), **kw) for r in range(R3)]
                us = time_rotating(gs)
                us_planes = time_rotating([abq.Gemm(xs[(M, K)], W3[r], SIGNED, **kw) for r in range(R3)])
                kwf = dict(kw, w_zero=None, x_group_sums=None)
                us_folded = time_rotating([abq.Gemm(xs_tiled[(M, K)], Wf3[r], SIGNED, x_tiled=True, w_tiled=True, **kwf) for r in range(R3)])
                deq3.append(dict(M=M, N=N, K=K, w_bits=3, group_size=128, us=round(us, 3), kernel="%s:%s" % (gs[0].strategy, gs[0].config_name),
                                 plane_operands_us=round(us_planes, 3), folded_zero_points_us=round(us_folded, 3)))
                log("dequant decode W3A8 M=%d N=%d K=%d  %.2f us (%s, padded records); plane operands %.2f us; zero points folded in %.2f us"
                    % (M, N, K, us, gs[0].strategy, us_planes, us_folded))
                del gs, out
            del Wp3, W3, Wf3
        # ... and a prefill of 1024 tokens on the same 3-bit weights: padded 4-bit records (the 4-bit pair's LDS-staged
        # kernel) against the 3-bit records (the register-staged kernel of the odd widths)
        pre3 = []
        for (N, K) in SHAPES:
            G = K // 128
            w3 = random_planes(torch, (3, N, K // 32))
            w3p, w3t = abq.relayout_planes_padded(w3, SIGNED), abq.relayout_planes(w3)
            wsc = torch.rand((N, G), device="cuda") * 0.01 + 0.001
            wz = torch.randint(-4, 4, (N, G), device="cuda").float()
            x = torch.randn((1024, K), device="cuda", dtype=torch.float16)
            xt, xsc, _, sums = abq.quant_pack_f16(x, Q_BITS, symmetric=True, tiled=True, group_size=128)
            out = torch.empty((1024, N), dtype=torch.float16, device="cuda")
            kw = dict(out=out, out_kind=abq.OUT_F16_SCALED, x_scale=xsc, w_scale=wsc, group_size=128, w_zero=wz, x_group_sums=sums,
                      x_tiled=True, w_tiled=True)
            gp = abq.Gemm(xt, w3p, SIGNED, value_bits=(Q_BITS, 3), **kw)
            us = time_rotating([gp])
            us_own = time_rotating([abq.Gemm(xt, w3t, SIGNED, **kw)])
            tops = 2.0 * 1024 * N * K / (us * 1e-6) / 1e12
            pre3.append(dict(M=1024, N=N, K=K, w_bits=3, group_size=128, us=round(us, 2), tops=round(tops, 1),
                             kernel="%s:%s" % (gp.strategy, gp.config_name), own_width_records_us=round(us_own, 2)))
            log("dequant prefill W3A8 M=1024 N=%d K=%d  %.1f us  %.0f TOPS (padded records); 3-bit records %.1f us" % (N, K, us, tops, us_own))
            del w3, w3p, w3t, out, xt
        extra["decode_group_scales"] = deq
        extra["decode_group_scales_w3a8"] = deq3
        extra["prefill_group_scales_w3a8"] = pre3

    if want("small_batch"):
        # ------------------------------------------------------------ side measurement: 32 and 64 rows on prepared operands
        # Between 17 and 128 rows the library weighs the decode kernel over blocks of 16 rows against the prefill
        # kernel's smallest tile; the kernel it picks and its time, int32 output and the group-128 dequantising epilogue.
        small = []
        for (N, K) in SHAPES:
            G = K // 128
            Wt = weights_tiled[(N, K)]
            wsc = torch.rand((N, G), device="cuda") * 0.01 + 0.001
            wz = torch.randint(-2, 2, (N, G), device="cuda").float()
            for M in (32, 64):
                xt = abq.relayout_planes(random_planes(torch, (Q_BITS, M, K // 32)))
                gs = [abq.Gemm(xt, Wt[r], SIGNED, x_tiled=True, w_tiled=True) for r in range(Wt.shape[0])]
                us = time_rotating(gs)
                xsc = torch.rand(M, device="cuda") * 0.05 + 0.01
                sums = torch.randint(-1000, 1000, (M, G), dtype=torch.int32, device="cuda")
                out = torch.empty((M, N), dtype=torch.float16, device="cuda")
                gg = [abq.Gemm(xt, Wt[r], SIGNED, x_tiled=True, w_tiled=True, out=out, out_kind=abq.OUT_F16_SCALED, x_scale=xsc,
                               w_scale=wsc, group_size=128, w_zero=wz, x_group_sums=sums) for r in range(Wt.shape[0])]
                us_g = time_rotating(gg)
                small.append(dict(M=M, N=N, K=K, us=round(us, 2), kernel="%s:%s" % (gs[0].strategy, gs[0].config_name),
                                  group128=dict(us=round(us_g, 2), kernel=gg[0].strategy)))
                log("small batch M=%d N=%d K=%d  int32 %.2f us (%s)  group scales %.2f us (%s)"
                    % (M, N, K, us, gs[0].strategy, us_g, gg[0].strategy))
                del gs, gg, out, xt
        # the reference's own test shape (BASELINE configs[0]): W4A4 unsigned, 64 x 4096 x 4096, plane operands through
        # init + exec, nothing prepared
        x4, w4 = random_planes(torch, (4, 64, 4096 // 32)), random_planes(torch, (4, 4096, 4096 // 32))
        g4 = abq.Gemm(x4, w4, False)
        us4 = time_rotating([g4])
        small.append(dict(M=64, N=4096, K=4096, x_bits=4, w_bits=4, signed=False, operands="planes", us=round(us4, 2),
                          tops=round(2.0 * 64 * 4096 * 4096 / (us4 * 1e-6) / 1e12, 2), kernel="%s:%s" % (g4.strategy, g4.config_name)))
        log("reference test shape W4A4 uint 64x4096x4096 on plane operands  %.2f us (%s)" % (us4, g4.config_name))
        extra["small_batch"] = small

    if want("decoder_layer_w2a8_group128"):
        # ------------------------------------------------------------ side measurement: one decoder layer's linears
        # BASELINE configs[4]: W2A8, 2-bit weights with group-128 scales and zero points (prepared layout),
        # activations quantised per token on the device inside the timed call, fp16 output; gate and up run
        # as one GEMM with the fused SiLU-gate epilogue.  Time = quantise+pack kernel + GEMM, graph replay.
        layer = []
        for tokens in (1, 16, 1024, 16384):  # a decode step of batch 1 and 16 (weights rotating, like every decode row), two prefills
            for name, N, K, act in (("qkv", 12288, 4096, 0), ("o", 4096, 4096, 0), ("gate_up_silu", 22016, 4096, 1),
                                    ("down", 4096, 11008, 0)):
                G = K // 128
                wpl = random_planes(torch, (P_BITS, N, K // 32))
                wt = abq.relayout_planes(wpl)
                wsc = torch.rand((N, G), device="cuda") * 0.01 + 0.001
                wz = torch.randint(-2, 2, (N, G), device="cuda").float()
                x = torch.randn((tokens, K), device="cuda", dtype=torch.float16)
                xt, xsc, _, sums = abq.quant_pack_f16(x, Q_BITS, symmetric=True, tiled=True, group_size=128)
                out = torch.empty((tokens, N // 2 if act else N), dtype=torch.float16, device="cuda")
                kwl = dict(out=out, out_kind=abq.OUT_F16_SCALED, x_scale=xsc, w_scale=wsc, group_size=128,
                           w_zero=wz, x_group_sums=sums, x_tiled=True, w_tiled=True, act=act)
                gm = abq.Gemm(xt, wt, SIGNED, **kwl)
                # decode steps: the weights rotate over >= 512 MiB of copies, so that the Infinity Cache does not serve them
                # (a prefill streams its activations and outputs through the cache anyway)
                copies = [wt]
                if tokens <= 16:
                    wbytes = wt.numel() * 4
                    wrot = wt.unsqueeze(0).repeat(max(2, math.ceil(ROTATE_BYTES / wbytes)), 1, 1, 1, 1)
                    copies = [wrot[r] for r in range(wrot.shape[0])]
                gms = [gm] if len(copies) == 1 else [abq.Gemm(xt, c, SIGNED, **kwl) for c in copies]

                def quantise_and_run(gemms):
                    """us per step of: quantise + pack the fp16 rows, then the GEMM (the next of `gemms`), graph replay"""
                    calls = [0]

                    def step():
                        abq._check(abq.lib().abq_quant_pack_f16(x.data_ptr(), tokens, K, Q_BITS, 1, 1, xt.data_ptr(), xsc.data_ptr(),
                                                                None, sums.data_ptr(), 128, abq._stream_ptr(None)), "quant_pack")
                        gemms[calls[0] % len(gemms)].run()
                        calls[0] += 1
                    step()
                    torch.cuda.synchronize()
                    # (a replay's own launch cost is spread over its steps; a decode graph walks through all weight copies)
                    reps = max(20, len(gemms)) if tokens < 1024 else 10 if tokens < 8192 else 3
                    gr = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(gr):
                        for _ in range(reps):
                            step()
                    settle(gr.replay)
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    gr.replay()
                    e1.record()
                    torch.cuda.synchronize()
                    del gr
                    return e0.elapsed_time(e1) * 1e3 / reps

                us = quantise_and_run(gms)
                tops = 2.0 * tokens * N * K / (us * 1e-6) / 1e12
                entry = dict(linear=name, tokens=tokens, N=N, K=K, us=round(us, 1), tops=round(tops, 1),
                             mfma_frac=round(tops / INT8_MFMA_PEAK_TOPS, 4), kernel="%s:%s" % (gm.strategy, gm.config_name))
                log("layer %s tokens=%d N=%d K=%d  %.1f us  %.0f TOPS (%.1f%% of int8 MFMA peak)"
                    % (name, tokens, N, K, us, tops, 100 * tops / INT8_MFMA_PEAK_TOPS))
                if tokens <= 16 and tokens * K <= 16384 and gm.strategy == "decode_tiled":
                    # the smallest calls: the decode kernel quantises the rows itself, one launch, same output bit for bit
                    out1 = torch.empty_like(out)
                    g1s = []
                    for c in copies:
                        g1 = abq.Gemm(xt, c, SIGNED, out=out1, out_kind=abq.OUT_F16_SCALED, x_scale=xsc, w_scale=wsc, group_size=128,
                                      x_tiled=True, w_tiled=True, act=act)
                        g1.set_dynamic_f16_activations(x, True, w_zero=wz)
                        g1s.append(g1)
                    g1s[0].run()
                    torch.cuda.synchronize()
                    if not torch.equal(out1, out):
                        raise RuntimeError("one-launch dynamic GEMM differs from quantise + GEMM (%s, tokens=%d)" % (name, tokens))
                    us1 = time_rotating(g1s, reps=max(20, len(g1s)))
                    entry["one_launch_us"] = round(us1, 1)
                    log("layer %s tokens=%d: one launch (kernel quantises the rows) %.1f us" % (name, tokens, us1))
                    del g1, g1s, out1
                if tokens >= 1024:
                    # the same prefill on a second copy of the weights with the zero points folded into 4-bit records
                    # (abq_relayout_planes_folded): no zero-point term in the epilogue
                    wf = abq.relayout_planes_folded(wpl, wz, 128, SIGNED)
                    outf = torch.empty_like(out)
                    gf = abq.Gemm(xt, wf, SIGNED, out=outf, out_kind=abq.OUT_F16_SCALED, x_scale=xsc, w_scale=wsc, group_size=128,
                                  x_tiled=True, w_tiled=True, act=act)
                    usf = quantise_and_run([gf])
                    torch.cuda.synchronize()
                    worst = float((outf.float() - out.float()).abs().max() / out.float().abs().max().clamp_min(1e-6))
                    if worst > 5e-3:
                        raise RuntimeError("GEMM on folded zero points differs from the zero-point term (%s, tokens=%d): %g" % (name, tokens, worst))
                    entry["folded_zero_points"] = dict(us=round(usf, 1), tops=round(2.0 * tokens * N * K / (usf * 1e-6) / 1e12, 1),
                                                       kernel="%s:%s" % (gf.strategy, gf.config_name))
                    log("layer %s tokens=%d: zero points folded into 4-bit records %.1f us  %.0f TOPS" % (name, tokens, usf, entry["folded_zero_points"]["tops"]))
                    del gf, wf, outf
                layer.append(entry)
                del gm, gms, copies, out, x, xt, wt, wpl
        extra["decoder_layer_w2a8_group128"] = layer


    # ---------------------------------------------------------------- output
    # side measurements: a file of their own (stderr already carries them line by line); the headline rows are logged
    # last so that they are what a tail of stderr keeps
    extra_file = None
    if args.extra_out:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.extra_out)), exist_ok=True)
            with open(args.extra_out, "w") as f:
                json.dump(extra, f, indent=1)
            extra_file = os.path.relpath(os.path.abspath(args.extra_out), ROOT)
        except OSError as exc:
            log("side measurements not written (%r)" % (exc,))
    for r in per_gemm:
        log("M=%d N=%d K=%d  %.2f us  %.2f TOPS  %.0f GB/s (%.1f%% of HBM peak)  %s"
            % (r["M"], r["N"], r["K"], r["us"], r["tops"], r["hbm_gbs"], 100 * r["hbm_frac"], r["kernel"]))
    plane_tops = None
    if "decode_plane_operands" in extra:
        plane_tops = sum(c["ops"] for c in cases) / sum(r["us"] * 1e-6 for r in extra["decode_plane_operands"]) / 1e12
    print(headline(value, K_STEPS, W_STEPS, total_s, len(cases), args.clock_settle_s, dominant, dg["tuples"],
                   dg["launches"], dg["bytes"] / dg["launches"], avg_launch_us, cpu_ops / cpu_s / 1e12, cpu_threads,
                   "%d passes over the same 9 GEMMs (%.1f s), oracle popcount GEMM with OpenMP" % (reps, cpu_s),
                   plane_operand_tops=plane_tops, extra_file=extra_file), flush=True)


if __name__ == "__main__":
    main()
