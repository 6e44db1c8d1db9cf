#!/usr/bin/env python3
"""Benchmark of the decode+matmul hot path on one MI355X.

Headline (the JSON line's `value`): batch-1 decode-GEMV at the Llama-2-70B projection
shapes.  One step = the four GEMVs (8192->10240, 8192->8192, 8192->28672, 28672->8192), each
on the next of several distinct code buffers so that the 256 MB Infinity Cache cannot serve
the weights; `value` is code bytes (N*K/4 per GEMV) per second over the timed region, inputs
resident in HBM.  The region of exactly --steps steps is timed --repeats times (one HIP graph
replay of up to 60 steps, bracketed by synchronisation) and the median region counts.
`dtype` says what the arithmetic is: halves in and out, fp8 x bf8 operands on the matrix unit
(exact for the grid and every finite x), fp32 sums; `config.value_f16_only` is the same step with
the 8-bit kernels switched off, timed after the headline.  Before the --warmup steps the step is
replayed for --preheat-ms (200 ms): the device needs some 15 ms of work to leave its idle clocks.

`roofline` is the GEMV kernel that carries most of the step's bytes, alone: code bytes per
launch over the kernel's launch duration - HIP events on the stream around replays of a graph of
that kernel's launches of the step, region / launches - against 8 TB/s; `roofline.f16_only` is the
same for the 16-bit-only step's kernel, and `roofline.read_only_step` what a reader of the same
rotating buffers gets per step: this library's read probe (same launch shape and access pattern
as the batch-1 kernels, no decode) and, owing nothing to this library, torch's row sums and
torch's device copy (from `hbm_read_probe`, which also has the probe per shape and per launch with
nothing to read: the memory system's and the launch path's share of the step).  `gemv_shapes` and
`all_gemv_launches` hold every launch of the step, per shape and per kernel, from HIP events
placed around each eager launch by the library's timing hook.  `gemv_7b_step` is a
Llama-2-7B layer's four projections as one graph, gate and up as one call on concatenated code
rows.  `prefill`, `small_batch` and `integer_operator` carry the M=2048, M=4..32 and int8
figures; `dispatch_check` times the operator's choice of kernel against the alternatives around
every threshold of the choice and lists the rows where it is more than 10 % slower;
`cpu_baseline` is the torch CPU path on the host cores on the four calls of one step.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16, published
MFMA_I8_PEAK_TOPS = 5000.0     # MI355X dense int8, published
# HBM bytes one GEMV launch moves, per kernel, averaged over the four shapes of the step (the 8-bit kernel
# serves all of them in the headline, the 16-bit kernel with resident sums in the 16-bit-only leg; the
# streaming kernel's figure is from the build in which it served that leg): rocprofv3 FETCH_SIZE and
# WRITE_SIZE per dispatch, each scaled by what the same counter reads for a plain 256 MiB device copy
# (x2.000 and x1.000).  39.19 MB per launch against 38,855,680 algorithmic bytes (codes, x, grid, y): 1.009.
# The many-tile 8-bit kernel (more than eight row tiles per compute unit) runs in no leg of this file.
GEMV_TRAFFIC_BYTES_PER_LAUNCH = {"dmm::gemv_q8d_kernel": 39186492, "dmm::gemv_f16d_kernel": 39173941,
                                 "dmm::gemv_stream_kernel": 39189916}
GEMV_TRAFFIC_SOURCE = {k: "constant from an earlier rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command, summarised in "
                          "profiles/gemv_kernels_llama70b_batch1.md; not measured by this run (a counter run cannot share a "
                          "process with the timed one)" for k in GEMV_TRAFFIC_BYTES_PER_LAUNCH}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--repeats", type=int, default=5,
                    help="how many times the region of exactly --steps steps is timed; the median region is reported")
    ap.add_argument("--preheat-ms", type=float, default=200.0,
                    help="untimed replays of the step for this long before the warmup steps: the device takes some "
                         "15 ms of work to leave its idle clocks, more than a short --warmup covers")
    ap.add_argument("--quick", action="store_true", help="skip prefill / small-batch / CPU legs")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of HIP graph replays")
    ap.add_argument("--graph-steps", type=int, default=60,
                    help="steps per HIP graph replay (rounded down to whole turns of the code-buffer sets)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the M = 2048 leg and print its object (for profiling the matrix-matrix kernel)")
    ap.add_argument("--integer-only", action="store_true",
                    help="run only the integer-operator leg and print its object (for profiling that kernel)")
    ap.add_argument("--small-batch-only", action="store_true",
                    help="run only the two small-batch legs and print their objects (for profiling the small-batch kernel)")
    ap.add_argument("--dispatch-check-only", action="store_true",
                    help="run only the check of the operator's kernel choices against the alternatives and print its object")
    ap.add_argument("--rotate-mb", type=int, default=400, help="distinct code bytes to rotate through, at least")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch 8 plain device copies of 256 MiB first (a known-size reference for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); "
              "use --gpus 1.  The path shards by rows of the code matrix (column-parallel) or by K "
              "(row-parallel, one all-reduce of the output).", file=sys.stderr)
        sys.exit(2)

    import torch
    import decode_matmul_amd as dmm
    from decode_matmul_amd import capi, workload

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; this benchmark measures the GPU kernels", file=sys.stderr)
        sys.exit(3)
    dev = "cuda:0"
    torch.cuda.set_device(0)
    lib = capi.lib()
    stream = torch.cuda.current_stream().cuda_stream

    def call(x, codes, grid, scale, y):
        M, K = x.shape
        st = lib.dmm_decode_matmul_f16(x.data_ptr(), codes.data_ptr(), grid.data_ptr(), scale, y.data_ptr(),
                                       M, codes.shape[0], K, stream)
        if st != 0:
            raise capi.DmmError("dmm_decode_matmul_f16", st)

    def rand_codes(N, K, copies, seed):
        # device RNG: uniform over all 65536 code values, `copies` distinct matrices
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        return [torch.randint(-32768, 32768, (N, K // 8), generator=g, dtype=torch.int16, device=dev)
                for _ in range(copies)]

    if args.copy_calibration:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(8):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.prefill_only:
        print(json.dumps({"prefill": prefill(torch, dmm, lib, capi, workload, dev, stream, rand_codes)}))
        return

    if args.integer_only:
        print(json.dumps({"integer_operator": integer_operator(torch, lib, capi, workload, dev, stream, rand_codes)}))
        return

    if args.dispatch_check_only:
        print(json.dumps({"dispatch_check": dispatch_check(torch, lib, capi, workload, dev)}))
        return

    if args.small_batch_only:
        print(json.dumps({"small_batch": small_batch(torch, lib, capi, workload, dev, stream, rand_codes),
                          "small_batch_70b": small_batch(torch, lib, capi, workload, dev, stream, rand_codes,
                                                         shapes=workload.LLAMA2_70B, batches=(2, 4, 8, 16))}))
        return

    # ---------------------------------------------------------------- headline: 70B GEMV
    shapes = workload.LLAMA2_70B
    step_bytes = sum(workload.code_bytes(N, K) for K, N in shapes)
    copies = max(2, -(-args.rotate_mb * 1000000 // step_bytes))
    probs = []
    for i, (K, N) in enumerate(shapes):
        x, _, grid, scale = workload.make_inputs(1, 8, K, seed=0)
        probs.append(dict(K=K, N=N, x=x.to(dev), grid=grid.to(dev), scale=scale,
                          codes=rand_codes(N, K, copies, 100 + i),
                          y=torch.empty(1, N, dtype=torch.float16, device=dev)))
    st = lib.dmm_init(-1)                # the once-per-device host work, before anything is captured
    if st != 0:
        raise capi.DmmError("dmm_init", st)

    def step(i):
        for p in probs:
            call(p["x"], p["codes"][i % copies], p["grid"], p["scale"], p["y"])

    # HIP graphs of several consecutive steps each (a step = its four launches, on the next set
    # of code buffers), so that the timed loop costs the host one graph launch per
    # `--graph-steps` steps.  A decode step of a model is one graph of hundreds of launches (80
    # layers of these four projections at this size), not one of four: with a graph per step the
    # GPU sat idle for about 15 us between replays, a fifth of the step, and with four ctypes
    # calls per 56 us step the eager loop sits close to being bound by the host.
    def prepare_steps():
        """A function that runs exactly n steps with the kernel choice as it stands now (the choice
        is made when a launch is captured), and how it launches them."""
        def run_steps(n):
            for i in range(n):
                step(i)
        mode = "eager"
        if not args.no_graph:
            try:
                chunk = max(copies, args.graph_steps // copies * copies)   # whole turns of the buffer sets
                graphs = {}

                def graph_of(n):                 # n consecutive steps, starting on buffer set 0
                    if n not in graphs:
                        g = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(g):
                            cap = torch.cuda.current_stream().cuda_stream
                            for i in range(n):
                                for p in probs:
                                    st = lib.dmm_decode_matmul_f16(p["x"].data_ptr(), p["codes"][i % copies].data_ptr(),
                                                                   p["grid"].data_ptr(), p["scale"], p["y"].data_ptr(),
                                                                   1, p["N"], p["K"], cap)
                                    if st != 0:
                                        raise capi.DmmError("dmm_decode_matmul_f16", st)
                        graphs[n] = g
                    return graphs[n]

                for n in {min(chunk, args.steps), args.steps % chunk, args.warmup % chunk, 12} - {0}:
                    graph_of(n)              # captured ahead of the timed regions

                def run_steps(n):                # exactly n steps: whole chunks, then the rest
                    for _ in range(n // chunk):
                        graph_of(chunk).replay()
                    if n % chunk:
                        graph_of(n % chunk).replay()
                per = min(chunk, args.steps)
                mode = "hip graph, %d steps (%d launches) per replay" % (per, per * len(probs))
            except Exception as e:   # capture unavailable: time the eager loop
                print("bench.py: graph capture failed (%s); timing eager launches" % e, file=sys.stderr)
        return run_steps, mode

    def dominant_kernel_timing(f16_only=False):
        """dominant_kernel_timing_now with the 8-bit kernels allowed (the headline) or switched off."""
        if not f16_only:
            return dominant_kernel_timing_now()
        was8 = lib.dmm_set_gemv_8bit(0)
        try:
            return dominant_kernel_timing_now()
        finally:
            lib.dmm_set_gemv_8bit(was8)

    def dominant_kernel_timing_now():
        """The kernel that carries most of the step's bytes (by the operator's choice per shape), and its
        launch duration in the regime the headline runs in: its launches of the step alone (its shapes
        taking turns over the rotating buffers) as a HIP graph, HIP events on the stream around each
        replay, duration = region / launches.  That is how a kernel trace of graph launches reads too (one
        dispatch begins as the one before ends).  Eager, event-bracketed launches start cold after an idle
        gap and read 0.5 - 1 us longer; they are in `gemv_shapes` and `all_gemv_launches`."""
        per_kernel = {}
        for p in probs:
            n = lib.dmm_gemv_kernel_name(1, p["N"], p["K"]).decode()
            per_kernel[n] = per_kernel.get(n, 0) + workload.code_bytes(p["N"], p["K"])
        dom = max(per_kernel, key=per_kernel.get)
        dom_probs = [p for p in probs if lib.dmm_gemv_kernel_name(1, p["N"], p["K"]).decode() == dom]
        if args.no_graph:
            return dom, dom_probs, None, "eager launches, HIP events around each kernel"
        try:
            gsteps = max(copies, args.graph_steps // copies * copies)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                cap = torch.cuda.current_stream().cuda_stream
                for i in range(gsteps):
                    for p in dom_probs:
                        st = lib.dmm_decode_matmul_f16(p["x"].data_ptr(), p["codes"][i % copies].data_ptr(), p["grid"].data_ptr(),
                                                       p["scale"], p["y"].data_ptr(), 1, p["N"], p["K"], cap)
                        if st != 0:
                            raise capi.DmmError("dmm_decode_matmul_f16", st)
            replays = max(1, -(-args.steps // gsteps))
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            regs = []
            for _ in range(max(1, args.repeats)):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(replays):
                    g.replay()
                e1.record()
                torch.cuda.synchronize()
                regs.append(e0.elapsed_time(e1) * 1e-3 / (replays * gsteps * len(dom_probs)))
            mode = ("HIP events around replays of a graph of this kernel's launches of the step (%d launches per replay, "
                    "%d replays per region, median of %d regions)" % (gsteps * len(dom_probs), replays, len(regs)))
            return dom, dom_probs, sorted(regs)[len(regs) // 2], mode
        except Exception as e:
            print("bench.py: roofline graph failed (%s); using the eager event timing" % e, file=sys.stderr)
            return dom, dom_probs, None, "eager launches, HIP events around each kernel"

    def timed_region(run_steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_steps(args.steps)
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    # the operator's own kernel choice, and the same steps with the 8-bit kernels switched off: every
    # launch in 16-bit arithmetic (half x half products, fp32 sums), the arithmetic the operator's
    # definition states.  Each is timed over exactly args.steps steps, `--repeats` times; the median
    # region counts.
    run_auto, launch_mode = prepare_steps()
    was = lib.dmm_set_gemv_8bit(0)
    try:
        run_f16, _ = prepare_steps()
        names16 = sorted({lib.dmm_gemv_kernel_name(1, N, K).decode() for K, N in shapes})
        if args.no_graph:
            run_f16 = None               # eager launches choose as they run: timed below, switched off
    finally:
        lib.dmm_set_gemv_8bit(was)
    t_heat = time.perf_counter()
    while (time.perf_counter() - t_heat) * 1e3 < args.preheat_ms:
        run_auto(12)
        torch.cuda.synchronize()
    run_auto(args.warmup)
    regions = [timed_region(run_auto) for _ in range(max(1, args.repeats))]
    dom, dom_probs, dom_launch_s, dom_mode = dominant_kernel_timing()
    # The 16-bit-only variant afterwards, not in turns with the headline: regions of the two taking turns
    # read 1.5 - 3 % slower than regions of one alone (measured), and a region right after a change of
    # kernels slower still, hence the untimed regions first.
    if run_f16:
        run_f16(args.warmup)
        for _ in range(5):
            timed_region(run_f16)
        regions16 = [timed_region(run_f16) for _ in range(max(1, args.repeats))]
    else:
        was = lib.dmm_set_gemv_8bit(0)
        try:
            run_auto(args.warmup)
            regions16 = [timed_region(run_auto) for _ in range(max(1, args.repeats))]
        finally:
            lib.dmm_set_gemv_8bit(was)
    dom16, dom16_probs, dom16_launch_s, dom16_mode = dominant_kernel_timing(f16_only=True)
    wall = sorted(regions)[len(regions) // 2]
    wall16 = sorted(regions16)[len(regions16) // 2]
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes * args.steps / wall / 1e9
    value_f16_only = step_bytes * args.steps / wall16 / 1e9

    # same region again with the kernel's own begin/end events
    n_launch = args.steps * len(probs)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_launch)]
    for a, b in ev:
        a.record(); b.record()
    torch.cuda.synchronize()
    j = 0
    for i in range(args.steps):
        for p in probs:
            lib.dmm_set_kernel_events(ev[j][0].cuda_event, ev[j][1].cuda_event)
            call(p["x"], p["codes"][i % copies], p["grid"], p["scale"], p["y"])
            j += 1
    lib.dmm_set_kernel_events(None, None)
    torch.cuda.synchronize()
    per_shape = {}
    j = 0
    for i in range(args.steps):
        for p in probs:
            per_shape.setdefault((p["K"], p["N"]), []).append(ev[j][0].elapsed_time(ev[j][1]) * 1e-3)
            j += 1
    kern_s = sum(sum(v) for v in per_shape.values())
    shape_rows = []
    kernels = {}    # kernel name -> launches, seconds, code bytes (the step runs two GEMV kernels)
    for (K, N), v in per_shape.items():
        avg = sum(v) / len(v)
        gbs = workload.code_bytes(N, K) / avg / 1e9
        name = lib.dmm_gemv_kernel_name(1, N, K).decode()
        shape_rows.append({"K": K, "N": N, "code_bytes": workload.code_bytes(N, K), "kernel_us": round(avg * 1e6, 3),
                           "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "kernel": name})
        k = kernels.setdefault(name, {"launches": 0, "seconds": 0.0, "bytes": 0})
        k["launches"] += len(v)
        k["seconds"] += sum(v)
        k["bytes"] += workload.code_bytes(N, K) * len(v)
    # the roofline object covers the kernel that carries most of the step's bytes; all launches
    # together are in `all_gemv_launches`
    kd = kernels[dom]
    eager_launch_us = kd["seconds"] / kd["launches"] * 1e6
    all_gbs = step_bytes * args.steps / kern_s / 1e9
    dom_bytes_per_launch = kd["bytes"] / kd["launches"]
    if dom_launch_s is None:
        dom_launch_s = kd["seconds"] / kd["launches"]
    achieved = dom_bytes_per_launch / dom_launch_s / 1e9
    # the same object for the 16-bit-only step's dominant kernel (its launches of the step as a graph)
    f16_roofline = None
    if dom16_launch_s is not None:
        b16 = sum(workload.code_bytes(p["N"], p["K"]) for p in dom16_probs) / len(dom16_probs)
        f16_roofline = {"kernel": dom16, "avg_launch_us": round(dom16_launch_s * 1e6, 3),
                        "achieved": round(b16 / dom16_launch_s / 1e9, 2), "unit": "GB/s",
                        "frac": round(b16 / dom16_launch_s / 1e9 / HBM_PEAK_GBS, 4),
                        "algorithmic_bytes_per_launch": b16,
                        "shapes": [{"K": p["K"], "N": p["N"]} for p in dom16_probs],
                        "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH.get(dom16), "timing": dom16_mode}

    out = {
        "metric": "batch-1 effective weight GB/s (code bytes N*K/4 per second, Llama-2-70B projection shapes)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 in/out; fp8 x bf8 MFMA operands (exact), fp32 sums",
        "dtype_note": "x, grid, y and the decoded weights are halves, sums fp32; launches of more than one row tile "
                      "per compute unit multiply fp8 weights (exact for this grid) by x split into four bf8 terms "
                      "(exact) on the 8-bit matrix unit; config.value_f16_only is the same step with every launch on "
                      "half x half products, roofline.f16_only that step's dominant kernel",
        "value_f16_only": round(value_f16_only, 2),
        "ms_per_step_f16_only": round(wall16 * 1e3 / args.steps, 5),
        "kernels_f16_only": names16,
        "timed_regions_ms": [round(r * 1e3, 4) for r in regions],
        "timed_regions_ms_f16_only": [round(r * 1e3, 4) for r in regions16],
        "data": "synthetic",
        "config": {"workload": "configs[2]: batch-1 decode-GEMV, 8192->10240, 8192->8192, 8192->28672, 28672->8192",
                   "M": 1, "code_buffers_rotated": copies, "distinct_code_MB": round(copies * step_bytes / 1e6, 1),
                   "step": "4 GEMVs, one per shape", "launch": launch_mode, "preheat_ms": args.preheat_ms,
                   "value_f16_only": round(value_f16_only, 2), "ms_per_step_f16_only": round(wall16 * 1e3 / args.steps, 5),
                   "kernels": sorted({lib.dmm_gemv_kernel_name(1, N, K).decode() for K, N in shapes}),
                   "kernels_f16_only": names16},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH.get(dom),
                     "traffic_source": GEMV_TRAFFIC_SOURCE.get(dom),
                     "kernel": dom, "launches": kd["launches"],
                     "avg_launch_us": round(dom_launch_s * 1e6, 3),
                     "timing": dom_mode,
                     "avg_launch_us_eager_events": round(eager_launch_us, 3),
                     "algorithmic_bytes_per_launch": dom_bytes_per_launch,
                     "f16_only": f16_roofline},
        "all_gemv_launches": {"launches": n_launch, "avg_launch_us": round(kern_s / n_launch * 1e6, 3),
                              "GBps": round(all_gbs, 2), "frac_hbm": round(all_gbs / HBM_PEAK_GBS, 4),
                              "kernels": {n: {"launches": k["launches"],
                                              "avg_launch_us": round(k["seconds"] / k["launches"] * 1e6, 3),
                                              "GBps": round(k["bytes"] / k["seconds"] / 1e9, 2)}
                                          for n, k in kernels.items()}},
        "gemv_shapes": shape_rows,
    }

    if not args.quick:
        out["hbm_read_probe"] = hbm_read_probe(torch, lib, probs, copies, stream, args.steps)
        # what a reader of the same rotating buffers gets, per step of four launches, beside the operator's step:
        # this library's read-only probe and two that owe nothing to it (torch's row sums and device copy)
        hp, li = out["hbm_read_probe"], out["hbm_read_probe"].get("library_independent") or {}
        out["roofline"]["read_only_step"] = {
            "operator_step_us": round(ms_per_step * 1e3, 3),
            "own_probe_step_us": hp.get("step_us"), "own_probe_GBps": hp.get("step_GBps"),
            "torch_row_sums_step_us": (li.get("torch_row_sums") or {}).get("step_us"),
            "torch_row_sums_GBps_read": (li.get("torch_row_sums") or {}).get("GBps_read"),
            "torch_copy_step_us": (li.get("torch_copy") or {}).get("step_us"),
            "torch_copy_GBps_moved": (li.get("torch_copy") or {}).get("GBps_moved")}
        out["gemv_packed"] = gemv_packed(torch, lib, capi, workload, probs, copies, stream, args.steps)
        out["gemv_7b_step"] = gemv_7b_step(torch, lib, capi, workload, dev, rand_codes)
        out["gemv_7b_shapes"] = gemv_7b(torch, lib, capi, workload, dev, stream, rand_codes)
        out["small_batch"] = small_batch(torch, lib, capi, workload, dev, stream, rand_codes)
        out["small_batch_70b"] = small_batch(torch, lib, capi, workload, dev, stream, rand_codes,
                                             shapes=workload.LLAMA2_70B, batches=(2, 4, 8, 16))
        out["integer_operator"] = integer_operator(torch, lib, capi, workload, dev, stream, rand_codes)
        out["prefill"] = prefill(torch, dmm, lib, capi, workload, dev, stream, rand_codes)
        out["dispatch_check"] = dispatch_check(torch, lib, capi, workload, dev)
        out["cpu_baseline"] = cpu_baseline(torch, workload)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


# Untimed launches ahead of the event-timed ones of a small-batch or integer leg: the host work between two
# configurations (new inputs, new code buffers) leaves the GPU idle long enough to drop its clocks, and a
# handful of launches does not bring them back (the same 48 launches read up to 40 % longer after 5 than after 200)
WARM_LAUNCHES = 200


def timed_kernel(torch, lib, fn, reps):
    """Average duration (s) of the library's dominant kernel over `reps` calls of fn(i)."""
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record(); b.record()
    torch.cuda.synchronize()
    for i in range(reps):
        lib.dmm_set_kernel_events(ev[i][0].cuda_event, ev[i][1].cuda_event)
        fn(i)
    lib.dmm_set_kernel_events(None, None)
    torch.cuda.synchronize()
    t = [a.elapsed_time(b) * 1e-3 for a, b in ev]
    return sum(t) / len(t)


GRAPH_LAUNCHES, GRAPH_WARM_REPLAYS, GRAPH_REGIONS, GRAPH_REPLAYS_PER_REGION = 24, 20, 5, 4


def graph_launch_us(torch, launch, copies):
    """us per launch of launch(i, stream) as replays of one HIP graph of 24 dependent launches over the rotating
    code buffers (what a serving loop sees: the time from the end of one kernel to the end of the next, the
    ~1.7 us between dependent launches included).  Events around regions of 4 replays (96 launches: the ~17 us a
    region costs beyond its kernels are 0.2 us per launch), median of 5 regions after 20 replays."""
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        cap = torch.cuda.current_stream().cuda_stream
        for i in range(GRAPH_LAUNCHES):
            launch(i, cap)
    for _ in range(GRAPH_WARM_REPLAYS):
        g.replay()
    torch.cuda.synchronize()
    t = []
    for _ in range(GRAPH_REGIONS):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(GRAPH_REPLAYS_PER_REGION):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        t.append(a.elapsed_time(b) * 1e3 / (GRAPH_REPLAYS_PER_REGION * GRAPH_LAUNCHES))
    return sorted(t)[len(t) // 2]


def hbm_read_probe(torch, lib, probs, copies, stream, steps):
    """What a kernel that only reads gets out of the memory system at the headline shapes: the
    library's read probe (same launch shape and access pattern as the batch-1 kernels, no decode)
    over the same rotating code buffers, the four shapes taking turns.  Per shape the kernel's own
    duration by events; `step_us` is the wall time per step of the four probes replayed as the
    same kind of HIP graph the headline is timed with (so it holds the gaps between dependent
    launches too), and `launch_us_empty` the wall time per launch of that graph when each probe has a
    single row tile to read, i.e. what a launch costs before it moves any data."""
    dev = probs[0]["x"].device
    sink = torch.zeros(16, dtype=torch.int32, device=dev)

    def fn(k, i, s=stream):
        p = probs[k]
        st = lib.dmm_read_probe(p["codes"][i % copies].data_ptr(), sink.data_ptr(), p["N"], p["K"], s)
        assert st == 0, st
    for i in range(3):
        for k in range(len(probs)):
            fn(k, i)
    n = steps * len(probs)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in ev:
        a.record(); b.record()
    torch.cuda.synchronize()
    j = 0
    for i in range(steps):
        for k in range(len(probs)):
            lib.dmm_set_kernel_events(ev[j][0].cuda_event, ev[j][1].cuda_event)
            fn(k, i)
            j += 1
    lib.dmm_set_kernel_events(None, None)
    torch.cuda.synchronize()
    rows = []
    for k, p in enumerate(probs):
        v = [ev[i * len(probs) + k][0].elapsed_time(ev[i * len(probs) + k][1]) * 1e-3 for i in range(steps)]
        t = sum(v) / len(v)
        b = p["N"] * p["K"] // 4
        rows.append({"K": p["K"], "N": p["N"], "code_bytes": b, "kernel_us": round(t * 1e6, 3),
                     "GBps": round(b / t / 1e9, 1), "frac_hbm": round(b / t / 1e9 / HBM_PEAK_GBS, 4)})
    out = {"kernel": "dmm::read_probe_kernel", "shapes": rows}

    graph_steps = max(copies, 12 // copies * copies)

    def graph_us(empty):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            cap = torch.cuda.current_stream().cuda_stream
            for i in range(graph_steps):
                for k, p in enumerate(probs):
                    if empty:
                        st = lib.dmm_read_probe(p["codes"][i % copies].data_ptr(), sink.data_ptr(), 16, p["K"], cap)
                        assert st == 0, st
                    else:
                        fn(k, i, cap)
        for _ in range(10):
            g.replay()
        torch.cuda.synchronize()
        t = []
        for _ in range(5):
            t0 = time.perf_counter()
            for _ in range(8):
                g.replay()
            torch.cuda.synchronize()
            t.append((time.perf_counter() - t0) / (8 * graph_steps))
        return sorted(t)[2] * 1e6
    try:
        step_us = graph_us(False)
        step_bytes = sum(p["N"] * p["K"] // 4 for p in probs)
        out["step_us"] = round(step_us, 3)
        out["step_GBps"] = round(step_bytes / step_us / 1e3, 1)
        out["step_frac_hbm"] = round(step_bytes / step_us / 1e3 / HBM_PEAK_GBS, 4)
        out["launch_us_empty"] = round(graph_us(True) / len(probs), 3)
        out["launch"] = "hip graph, %d steps (%d launches) per replay" % (graph_steps, graph_steps * len(probs))
    except Exception as e:
        print("bench.py: read-probe graph failed (%s)" % e, file=sys.stderr)
    out["library_independent"] = torch_read_figures(torch, probs, copies)
    return out


def torch_read_figures(torch, probs, copies):
    """What the box gives a reader of the same rotating code buffers without any kernel of this library: torch's
    device-to-device copy (reads and writes the bytes) and torch's row sums (reads them, writes next to nothing:
    the buffer as 4096 rows of int32, one sum per row), the four shapes taking turns, each as replays of one
    HIP graph like the headline.  Per step of four launches; `GBps_read` counts the code bytes once."""
    step_bytes = sum(p["N"] * p["K"] // 4 for p in probs)
    graph_steps = max(copies, 12 // copies * copies)
    dst = [torch.empty_like(p["codes"][0]) for p in probs]
    views = [[c.view(torch.int32).view(4096, -1) for c in p["codes"]] for p in probs]
    sums = [torch.empty(4096, dtype=torch.int32, device=dst[0].device) for _ in probs]

    def enqueue_copy(i):
        for k, p in enumerate(probs):
            dst[k].copy_(p["codes"][i % copies])

    def enqueue_sum(i):
        for k in range(len(probs)):
            torch.sum(views[k][i % copies], dim=1, dtype=torch.int32, out=sums[k])

    def graph_step_us(enqueue):
        enqueue(0)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(graph_steps):
                enqueue(i)
        for _ in range(10):
            g.replay()
        torch.cuda.synchronize()
        t = []
        for _ in range(5):
            t0 = time.perf_counter()
            for _ in range(8):
                g.replay()
            torch.cuda.synchronize()
            t.append((time.perf_counter() - t0) / (8 * graph_steps))
        return sorted(t)[2] * 1e6
    out = {"launch": "hip graph, %d steps (%d launches) per replay" % (graph_steps, graph_steps * len(probs))}
    for name, enqueue, moved in (("torch_copy", enqueue_copy, 2), ("torch_row_sums", enqueue_sum, 1)):
        try:
            us = graph_step_us(enqueue)
            out[name] = {"step_us": round(us, 3), "GBps_read": round(step_bytes / us / 1e3, 1),
                         "frac_hbm_read": round(step_bytes / us / 1e3 / HBM_PEAK_GBS, 4),
                         "GBps_moved": round(moved * step_bytes / us / 1e3, 1),
                         "frac_hbm_moved": round(moved * step_bytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        except Exception as e:
            print("bench.py: %s graph failed (%s)" % (name, e), file=sys.stderr)
            out[name] = None
    return out


def gemv_7b_step(torch, lib, capi, workload, dev, rand_codes):
    """One decode step's projections of a Llama-2-7B layer as the caller would issue them: fused QKV
    (4096 -> 12288), o_proj (4096 -> 4096), gate and up as ONE call on their concatenated code rows (4096 ->
    22016), down (11008 -> 4096); 12 layers' worth of distinct code buffers (590 MB) captured as one HIP graph
    of 48 launches.  Wall time per layer step and code bytes per second, beside the eager per-shape figures."""
    layer = ((4096, 12288), (4096, 4096), (4096, 22016), (11008, 4096))
    layers = 12
    probs = []
    for j, (K, N) in enumerate(layer):
        x, _, grid, scale = workload.make_inputs(1, 8, K, seed=0)
        probs.append(dict(K=K, N=N, x=x.to(dev), grid=grid.to(dev), scale=scale, codes=rand_codes(N, K, layers, 300 + j),
                          y=torch.empty(1, N, dtype=torch.float16, device=dev)))
    layer_bytes = sum(workload.code_bytes(N, K) for K, N in layer)

    def enqueue(stream):
        for i in range(layers):
            for p in probs:
                st = lib.dmm_decode_matmul_f16(p["x"].data_ptr(), p["codes"][i].data_ptr(), p["grid"].data_ptr(), p["scale"],
                                               p["y"].data_ptr(), 1, p["N"], p["K"], stream)
                if st != 0:
                    raise capi.DmmError("dmm_decode_matmul_f16", st)
    enqueue(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        enqueue(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        g.replay()
    torch.cuda.synchronize()
    reps, times = 10, []
    for _ in range(5):
        t0 = time.perf_counter()
        for _ in range(reps):
            g.replay()
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) / (reps * layers))
    t = sorted(times)[len(times) // 2]
    return {"launches_per_step": len(layer), "shapes": [{"K": K, "N": N} for K, N in layer],
            "graph": "%d layer steps (%d launches) per replay" % (layers, layers * len(layer)),
            "us_per_step": round(t * 1e6, 3), "code_bytes_per_step": layer_bytes,
            "GBps": round(layer_bytes / t / 1e9, 1), "frac_hbm": round(layer_bytes / t / 1e9 / HBM_PEAK_GBS, 4),
            "kernels": [lib.dmm_gemv_kernel_name(1, N, K).decode() for K, N in layer]}


def gemv_packed(torch, lib, capi, workload, probs, copies, stream, steps):
    """The headline step again with the codes repacked offline (dmm_pack_codes: a wave's load is
    1 KB of consecutive bytes).  Same inputs, bit-identical outputs; kernel durations by events,
    measured like the row-major ones: the four shapes take turns and every launch reads the next
    of `copies` distinct buffers of its shape, so that the Infinity Cache cannot serve the codes
    (a loop over one shape alone would cycle through 50 - 176 MB and be served from it in part)."""
    packed = []
    for p in probs:
        K, N = p["K"], p["N"]
        bufs = []
        for c in p["codes"]:
            buf = torch.empty(lib.dmm_packed_bytes(N, K) // 2, dtype=torch.int16, device=c.device)
            st = lib.dmm_pack_codes(c.data_ptr(), buf.data_ptr(), N, K, stream)
            assert st == 0, st
            bufs.append(buf)
        packed.append(bufs)
    ys = [torch.empty_like(p["y"]) for p in probs]

    def fn(k, i):
        p = probs[k]
        st = lib.dmm_gemv_packed_f16(p["x"].data_ptr(), packed[k][i % copies].data_ptr(), p["grid"].data_ptr(),
                                     p["scale"], ys[k].data_ptr(), 1, p["N"], p["K"], stream)
        assert st == 0, st
    for k, p in enumerate(probs):        # bit-identity against the row-major call on the same codes
        fn(k, 1)
        lib.dmm_decode_matmul_f16(p["x"].data_ptr(), p["codes"][1 % copies].data_ptr(), p["grid"].data_ptr(), p["scale"],
                                  p["y"].data_ptr(), 1, p["N"], p["K"], stream)
        torch.cuda.synchronize()
        assert torch.equal(ys[k], p["y"]), "packed and row-major results differ"
    for i in range(3):
        for k in range(len(probs)):
            fn(k, i)
    n = steps * len(probs)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in ev:
        a.record(); b.record()
    torch.cuda.synchronize()
    j = 0
    for i in range(steps):
        for k in range(len(probs)):
            lib.dmm_set_kernel_events(ev[j][0].cuda_event, ev[j][1].cuda_event)
            fn(k, i)
            j += 1
    lib.dmm_set_kernel_events(None, None)
    torch.cuda.synchronize()
    rows = []
    tot_b = tot_t = 0.0
    for k, p in enumerate(probs):
        v = [ev[i * len(probs) + k][0].elapsed_time(ev[i * len(probs) + k][1]) * 1e-3 for i in range(steps)]
        t = sum(v) / len(v)
        b = workload.code_bytes(p["N"], p["K"])
        tot_b += b
        tot_t += t
        rows.append({"K": p["K"], "N": p["N"], "kernel_us": round(t * 1e6, 3), "GBps": round(b / t / 1e9, 1),
                     "frac_hbm": round(b / t / 1e9 / HBM_PEAK_GBS, 4)})
    return {"shapes": rows, "achieved_GBps": round(tot_b / tot_t / 1e9, 2),
            "frac_hbm": round(tot_b / tot_t / 1e9 / HBM_PEAK_GBS, 4)}


def gemv_7b(torch, lib, capi, workload, dev, stream, rand_codes):
    """configs[1]: batch-1 GEMV at the Llama-2-7B projection shapes, enough code buffers in
    rotation per shape (30 or more, at least 320 MB) that the 256 MB Infinity Cache cannot serve them."""
    rows = []
    for K, N in workload.LLAMA2_7B:
        copies = max(30, -(-320_000_000 // workload.code_bytes(N, K)))
        codes = rand_codes(N, K, copies, 7)
        x, _, grid, scale = workload.make_inputs(1, 8, K, seed=0)
        x, grid = x.to(dev), grid.to(dev)
        y = torch.empty(1, N, dtype=torch.float16, device=dev)

        def fn(i):
            st = lib.dmm_decode_matmul_f16(x.data_ptr(), codes[i % copies].data_ptr(), grid.data_ptr(), scale,
                                           y.data_ptr(), 1, N, K, stream)
            assert st == 0, st
        for i in range(5):
            fn(i)
        # these kernels run 5-7 us, close to the ~4 us floor of an event pair around one kernel,
        # so time 120 back-to-back launches as one region instead (launch gaps included)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(120):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        t = a.elapsed_time(b) * 1e-3 / 120
        gbs = workload.code_bytes(N, K) / t / 1e9
        rows.append({"K": K, "N": N, "code_bytes": workload.code_bytes(N, K), "us_per_launch": round(t * 1e6, 3),
                     "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)})
    return rows


def small_batch(torch, lib, capi, workload, dev, stream, rand_codes, shapes=None, batches=(4, 8, 16, 32)):
    """A few rows of x (the small-batch configuration's shapes by default; the headline's shapes
    as a second leg), every launch on the next of enough code buffers to stay out of the Infinity
    Cache: `kernel_us` is the kernel's duration by events around eager launches (box and launch
    conditions move it by a microsecond or two), `graph_us` the time per launch of the same calls as
    one HIP graph, which the rates are computed from."""
    rows = []
    for K, N in (workload.SMALL_BATCH if shapes is None else shapes):
        copies = max(2, -(-320 * 1000000 // workload.code_bytes(N, K)))
        codes = rand_codes(N, K, copies, 7)
        for M in batches:
            x, _, grid, scale = workload.make_inputs(M, 8, K, seed=0)
            x, grid = x.to(dev), grid.to(dev)
            y = torch.empty(M, N, dtype=torch.float16, device=dev)
            # the operator's workspace (split-K partial sums for short x; 0 bytes = none used)
            ws_bytes = lib.dmm_workspace_bytes(M, N, K)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)

            def fn(i, s=stream):
                st = lib.dmm_decode_matmul_ws_f16(x.data_ptr(), codes[i % copies].data_ptr(), grid.data_ptr(), scale,
                                                  y.data_ptr(), M, N, K, ws.data_ptr(), ws_bytes, s)
                assert st == 0, st
            for i in range(WARM_LAUNCHES):
                fn(i)
            t = timed_kernel(torch, lib, fn, 48)     # spans both kernels when the call splits K
            tg = graph_launch_us(torch, fn, copies) * 1e-6
            rows.append({"M": M, "K": K, "N": N, "kernel_us": round(t * 1e6, 3), "graph_us": round(tg * 1e6, 3),
                         "workspace_MB": round(ws_bytes / 1e6, 1),
                         "GBps_code": round(workload.code_bytes(N, K) / tg / 1e9, 1),
                         "TFLOPs": round(workload.flops(M, N, K) / tg / 1e12, 2)})
    return rows


def integer_operator(torch, lib, capi, workload, dev, stream, rand_codes):
    """The reference's own operator (int8 x, int16 codes in its tile order, int64 table -> int32,
    dmm_decode_matmul_i8) at the headline shapes, M = 1 and M = 8 (the reference asks for M % 8
    == 0).  `kernel_us`: kernel durations by events around eager launches; `graph_us`: per launch of
    the same calls as one HIP graph (the rates are computed from it); every launch reads the next of
    enough code buffers to stay out of the Infinity Cache.  Random 16-bit codes are equally random in either layout."""
    from decode_matmul_amd import codebook
    cb = codebook.build_codebook_abs().to(dev)
    rows = []
    for K, N in workload.LLAMA2_70B:
        copies = max(2, -(-320 * 1000000 // workload.code_bytes(N, K)))
        codes = rand_codes(N, K, copies, 11)
        for M in (1, 8):
            g = torch.Generator(device=dev)
            g.manual_seed(5)
            x = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8, device=dev)
            out = torch.empty(M, N, dtype=torch.int32, device=dev)

            def fn(i, s=stream):
                st = lib.dmm_decode_matmul_i8(x.data_ptr(), codes[i % copies].data_ptr(), cb.data_ptr(), out.data_ptr(),
                                              M, N, K, 1, s)
                assert st == 0, st
            for i in range(WARM_LAUNCHES):
                fn(i)
            t = timed_kernel(torch, lib, fn, 40)
            tg = graph_launch_us(torch, fn, copies) * 1e-6
            rows.append({"M": M, "K": K, "N": N, "kernel_us": round(t * 1e6, 3), "graph_us": round(tg * 1e6, 3),
                         "GBps_code": round(workload.code_bytes(N, K) / tg / 1e9, 1),
                         "frac_hbm": round(workload.code_bytes(N, K) / tg / 1e9 / HBM_PEAK_GBS, 4),
                         "kernel": lib.dmm_integer_kernel_name(M, N, K).decode()})
        del codes
    # M = 2048 at the prefill shapes: the int8 matrix-matrix kernel (2 M N K integer operations)
    M = 2048
    for K, N in workload.PREFILL:
        codes = rand_codes(N, K, 2, 13)
        g = torch.Generator(device=dev)
        g.manual_seed(6)
        x = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8, device=dev)
        out = torch.empty(M, N, dtype=torch.int32, device=dev)

        def fn(i):
            st = lib.dmm_decode_matmul_i8(x.data_ptr(), codes[i % 2].data_ptr(), cb.data_ptr(), out.data_ptr(),
                                          M, N, K, 1, stream)
            assert st == 0, st
        for i in range(3):
            fn(i)
        t = timed_kernel(torch, lib, fn, 20)
        rows.append({"M": M, "K": K, "N": N, "kernel_us": round(t * 1e6, 2),
                     "TOPs": round(workload.flops(M, N, K) / t / 1e12, 1),
                     "frac_mfma_i8": round(workload.flops(M, N, K) / t / 1e12 / MFMA_I8_PEAK_TOPS, 4),
                     "kernel": lib.dmm_integer_kernel_name(M, N, K).decode()})
    return rows


def prefill(torch, dmm, lib, capi, workload, dev, stream, rand_codes):
    rows = []
    M = 2048
    for K, N in workload.PREFILL:
        codes = rand_codes(N, K, 2, 9)
        x, _, grid, scale = workload.make_inputs(M, 8, K, seed=0)
        x, grid = x.to(dev), grid.to(dev)
        y = torch.empty(M, N, dtype=torch.float16, device=dev)

        def fn(i):
            st = lib.dmm_decode_matmul_f16(x.data_ptr(), codes[i % 2].data_ptr(), grid.data_ptr(), scale,
                                           y.data_ptr(), M, N, K, stream)
            assert st == 0, st
        for i in range(3):
            fn(i)
        t = timed_kernel(torch, lib, fn, 20)
        # the same call on codes repacked offline (bit-identical result)
        packed = [dmm.pack_codes(c) for c in codes]
        y_pk = torch.empty_like(y)

        def fn_pk(i):
            st = lib.dmm_decode_matmul_packed_f16(x.data_ptr(), packed[i % 2].data_ptr(), grid.data_ptr(), scale,
                                                  y_pk.data_ptr(), M, N, K, None, 0, stream)
            assert st == 0, st
        for i in range(3):
            fn_pk(i)
        t_pk = timed_kernel(torch, lib, fn_pk, 20)
        fn(1)
        fn_pk(1)
        torch.cuda.synchronize()
        assert torch.equal(y, y_pk), "packed and row-major results differ"
        # comparison: own decode kernel -> dense half W in HBM -> library GEMM (torch.matmul)
        for i in range(3):
            W = dmm.decode(codes[i % 2], grid)
            ref = torch.matmul(x, W.T)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(20):
            W = dmm.decode(codes[i % 2], grid)
            ref = torch.matmul(x, W.T)
        b.record()
        torch.cuda.synchronize()
        t_cmp = a.elapsed_time(b) * 1e-3 / 20
        tf = workload.flops(M, N, K) / t / 1e12
        rows.append({"M": M, "K": K, "N": N, "kernel_us": round(t * 1e6, 2), "TFLOPs": round(tf, 1),
                     "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                     "packed_kernel_us": round(t_pk * 1e6, 2),
                     "packed_TFLOPs": round(workload.flops(M, N, K) / t_pk / 1e12, 1),
                     "decode_then_library_gemm_us": round(t_cmp * 1e6, 2),
                     "decode_then_library_gemm_TFLOPs": round(workload.flops(M, N, K) / t_cmp / 1e12, 1)})
    tot_f = sum(workload.flops(M, N, K) for K, N in workload.PREFILL)
    tot_t = sum(r["kernel_us"] for r in rows) * 1e-6
    return {"shapes": rows,
            "roofline": {"bound": "mfma", "achieved": round(tot_f / tot_t / 1e12, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(tot_f / tot_t / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                         "traffic": None, "kernel": "dmm::gemm_reg_kernel"}}


def dispatch_check(torch, lib, capi, workload, dev):
    """The operator's choice of kernel against the alternatives, around every threshold of the choice: each
    candidate as launches of one HIP graph over the same rotating code buffers (300 MB or more per graph, so the
    codes come from HBM), HIP events around a replay, median of 7.  A row lists the operator's own time
    (`chosen_us`), the alternatives', and `slower_by` = chosen / best - 1; `flagged` are the rows where the
    choice is more than 10 % slower than an alternative."""
    from decode_matmul_amd import codebook
    pool_bytes = 420 * 1000 * 1000
    g = torch.Generator(device=dev)
    g.manual_seed(77)
    pool = torch.randint(-32768, 32768, (pool_bytes // 2,), generator=g, dtype=torch.int16, device=dev)
    cb = codebook.build_codebook_abs().to(dev)

    def graph_us(launch, nbytes):
        """launch(code_ptr, stream) -> status; us per launch"""
        stride = (nbytes + 255) // 256 * 256
        n_buf = max(2, pool_bytes // stride)
        L = min(max(6, -(-300 * 1000 * 1000 // stride)), 72, n_buf)
        cur = torch.cuda.current_stream().cuda_stream
        for i in range(2):
            st = launch(pool.data_ptr() + i * stride, cur)
            if st != 0:
                return None
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            cap = torch.cuda.current_stream().cuda_stream
            for i in range(L):
                st = launch(pool.data_ptr() + i * stride, cap)
                assert st == 0, st
        t_warm = time.perf_counter()          # 25 ms of replays: the clocks a candidate is timed at must not
        while True:                           # depend on how long the host took to set it up
            for _ in range(4):
                gr.replay()
            torch.cuda.synchronize()
            if time.perf_counter() - t_warm > 0.025:
                break
        t = []
        for _ in range(7):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            gr.replay()
            b.record()
            torch.cuda.synchronize()
            t.append(a.elapsed_time(b) * 1e3 / L)
        return sorted(t)[3]

    rows = []

    def add(check, M, K, N, times, extra=None):
        chosen = times.pop("operator")
        alts = {k: round(v, 3) for k, v in times.items() if v is not None}
        best = min(alts.values()) if alts else chosen
        row = {"check": check, "M": M, "K": K, "N": N, "chosen_us": round(chosen, 3), "alternatives_us": alts,
               "slower_by": round(chosen / best - 1.0, 4)}
        if extra:
            row.update(extra)
        rows.append(row)

    def half_inputs(M, K):
        x, _, grid, scale = workload.make_inputs(M, 8, K, seed=0)
        return x.to(dev), grid.to(dev), scale

    # ---- one to four rows of x: 8-bit against 16-bit kernels (pick_gemv)
    mv_shapes = {1: ((4096, 4096), (4096, 4352), (4096, 8192), (8192, 4096), (8192, 4352), (8192, 8192), (8192, 8448),
                     (11008, 4096), (11008, 4352), (11008, 8192), (11008, 8448), (12288, 4352), (28672, 4096),
                     (28672, 4352)),
                 2: ((4096, 8192), (4096, 12288), (4096, 12544), (4096, 16384)),
                 4: ((3072, 12288), (3072, 12544), (3072, 16384))}
    for M, shapes in mv_shapes.items():
        for K, N in shapes:
            x, grid, scale = half_inputs(M, K)
            y = torch.empty(M, N, dtype=torch.float16, device=dev)
            nbytes = workload.code_bytes(N, K)

            def op(fn):
                return lambda c, s: fn(x.data_ptr(), c, grid.data_ptr(), scale, y.data_ptr(), M, N, K, s)
            times = {"operator": graph_us(op(lib.dmm_decode_matmul_f16), nbytes),
                     "8-bit": graph_us(op(lib.dmm_gemv_8bit_f16), nbytes)}
            was = lib.dmm_set_gemv_8bit(0)
            try:
                times["16-bit"] = graph_us(op(lib.dmm_gemv_f16), nbytes)
            finally:
                lib.dmm_set_gemv_8bit(was)
            add("pick_gemv", M, K, N, times, {"kernel": lib.dmm_gemv_kernel_name(M, N, K).decode()})

    # ---- up to 32 rows: the 16-bit kernel with resident sums against the kernels that served before it
    for M in (2, 4, 8, 12, 16, 24, 32):
        for K, N in ((4096, 11008), (4096, 22016), (11008, 4096), (8192, 8192), (8192, 10240), (8192, 28672),
                     (28672, 8192), (1024, 16384), (4096, 4096), (8192, 4096)):
            x, grid, scale = half_inputs(M, K)
            y = torch.empty(M, N, dtype=torch.float16, device=dev)

            def op2(c, s):
                return lib.dmm_decode_matmul_f16(x.data_ptr(), c, grid.data_ptr(), scale, y.data_ptr(), M, N, K, s)
            times = {"operator": graph_us(op2, workload.code_bytes(N, K))}
            for name, value in (("streaming, small-batch or 8-bit", 0), ("resident sums", 1)):
                was = lib.dmm_set_choice(2, value)
                try:
                    times[name] = graph_us(op2, workload.code_bytes(N, K))
                finally:
                    lib.dmm_set_choice(2, was)
            add("pick_gemv, resident sums", M, K, N, times, {"kernel": lib.dmm_gemv_kernel_name(M, N, K).decode()})

    # ---- 17 .. 32 rows with a workspace (passes against split K), more rows (passes against the matrix-matrix
    # kernel, with and without a workspace)
    ws = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
    mm_cases = [("passes_beat_splitk", M, K, N) for M in (17, 32)
                for K, N in ((4096, 11008), (8192, 8192), (8192, 8448), (4096, 17408), (8192, 10240), (4096, 4096),
                             (11008, 4096), (4096, 22016), (8192, 28672), (28672, 8192), (16384, 8192))]
    mm_cases += [("passes_beat_gemm", M, K, N) for M in (48, 64, 128, 256)
                 for K, N in ((4096, 4096), (4096, 11008), (11008, 4096), (8192, 8192))]
    for check, M, K, N in mm_cases:
        x, grid, scale = half_inputs(M, K)
        y = torch.empty(M, N, dtype=torch.float16, device=dev)
        nbytes = workload.code_bytes(N, K)

        def ws_op(c, s):
            nb = min(lib.dmm_workspace_bytes(M, N, K), ws.numel())
            return lib.dmm_decode_matmul_ws_f16(x.data_ptr(), c, grid.data_ptr(), scale, y.data_ptr(), M, N, K,
                                                ws.data_ptr(), nb, s)

        def plain_op(c, s):
            return lib.dmm_decode_matmul_f16(x.data_ptr(), c, grid.data_ptr(), scale, y.data_ptr(), M, N, K, s)
        times = {"operator": graph_us(ws_op, nbytes)}
        if check == "passes_beat_gemm":
            times["operator, no workspace"] = graph_us(plain_op, nbytes)
        for name, value in (("passes", 0), ("matrix-matrix", 1), ("split K", 2)):
            was = lib.dmm_set_choice(0, value)
            try:
                if value != 2 or lib.dmm_workspace_bytes(M, N, K) > 0:
                    times[name] = graph_us(ws_op, nbytes)
            finally:
                lib.dmm_set_choice(0, was)
        extra = None
        if check == "passes_beat_gemm":      # the choice without a workspace: passes or matrix-matrix only
            t0 = times.pop("operator, no workspace")
            best2 = min(times["passes"], times["matrix-matrix"])
            extra = {"chosen_no_workspace_us": round(t0, 3), "slower_by_no_workspace": round(t0 / best2 - 1.0, 4)}
        add(check, M, K, N, times, extra)

    # ---- the integer operator on up to 32 rows: the kernel with resident sums against the row-block kernel
    for M in (1, 4, 8, 12, 16, 32):
        for K, N in ((4096, 11008), (8192, 8192), (8192, 10240), (8192, 28672), (28672, 8192), (512, 16384), (1024, 16384),
                     (2048, 8192)):
            gi = torch.Generator(device=dev)
            gi.manual_seed(5)
            x = torch.randint(-128, 128, (M, K), generator=gi, dtype=torch.int8, device=dev)
            out = torch.empty(M, N, dtype=torch.int32, device=dev)

            def i8_small(c, s):
                return lib.dmm_decode_matmul_i8(x.data_ptr(), c, cb.data_ptr(), out.data_ptr(), M, N, K, 1, s)
            times = {"operator": graph_us(i8_small, workload.code_bytes(N, K))}
            kernel = lib.dmm_integer_kernel_name(M, N, K).decode()
            for name, value in (("row blocks", 0), ("resident sums", 1)):
                was = lib.dmm_set_choice(3, value)
                try:
                    times[name] = graph_us(i8_small, workload.code_bytes(N, K))
                finally:
                    lib.dmm_set_choice(3, was)
            add("int8, up to 32 rows", M, K, N, times, {"kernel": kernel})

    # ---- the integer operator on more than 16 rows: passes against the matrix-matrix kernel (pick_int8)
    for M in (32, 64, 128, 192, 256, 384):
        for K, N in ((4096, 4096), (11008, 4096), (8192, 28672), (28672, 8192)):
            gi = torch.Generator(device=dev)
            gi.manual_seed(5)
            x = torch.randint(-128, 128, (M, K), generator=gi, dtype=torch.int8, device=dev)
            out = torch.empty(M, N, dtype=torch.int32, device=dev)

            def i8_op(c, s):
                return lib.dmm_decode_matmul_i8(x.data_ptr(), c, cb.data_ptr(), out.data_ptr(), M, N, K, 1, s)
            times = {"operator": graph_us(i8_op, workload.code_bytes(N, K))}
            for name, value in (("passes", 1), ("matrix-matrix", 2)):
                was = lib.dmm_set_choice(1, value)
                try:
                    times[name] = graph_us(i8_op, workload.code_bytes(N, K))
                finally:
                    lib.dmm_set_choice(1, was)
            add("pick_int8", M, K, N, times, {"kernel": lib.dmm_integer_kernel_name(M, N, K).decode()})

    def worst(r):
        return max(r["slower_by"], r.get("slower_by_no_workspace", 0.0))
    flagged = [r for r in rows if worst(r) > 0.10]
    return {"rows": rows, "n_rows": len(rows), "flagged": flagged,
            "worst_slower_by": round(max(worst(r) for r in rows), 4),
            "timing": "launches of one HIP graph per candidate over rotating code buffers, HIP events around a replay, "
                      "median of 7; slower_by = operator's time / best candidate's - 1"}


def cpu_baseline(torch, workload):
    """The torch CPU path (decode to dense half, then matmul) on the host cores, on a bounded
    sample: the four batch-1 calls of one step of the workload, one untimed pass and then the
    median of 5 per call (about 10 s of CPU work)."""
    from oracle import cpu_path
    dec = mm = 0.0
    total = 0
    for K, N in workload.LLAMA2_70B:
        x, codes, grid, scale = workload.make_inputs(1, N, K, seed=0)
        cpu_path.time_cpu_path(x, codes, grid, scale, repeats=1)
        d, m, _ = cpu_path.time_cpu_path(x, codes, grid, scale, repeats=5)
        dec, mm, total = dec + d, mm + m, total + workload.code_bytes(N, K)
        del x, codes
    gbs = total / (dec + mm) / 1e9
    return {"value": round(gbs, 4), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "one step of the workload (4 batch-1 calls, %.1f MB of codes), per call one untimed pass and "
                      "the median of 5; decode %.3f s + matmul %.3f s per step" % (total / 1e6, dec, mm),
            "host_cpu_count": os.cpu_count()}


if __name__ == "__main__":
    main()
