#!/usr/bin/env python3
"""Benchmark of the NCE op path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg5] [--no-others] [--no-cpu]

The default workload is cfg5, the INT8 ResNet-50 task graph at batch 32 (53 convolutions, one max pool, 16
residual adds): a step is one pass of the whole graph over its batch, inputs, weights and tables already
resident in HBM, all 70 tasks launched from one task list (one C call per step). The single-task workloads
(cfg2, cfg3_*, cfg4) ride along in "other_workloads", each with its own roofline. The timed steps are bracketed
by torch.cuda.synchronize(); HIP events on the launch stream give the device-side duration used for the
roofline figure. Prints ONE JSON line.

    python bench.py --summarize-pmc DIR1 [DIR2 ...]     (no GPU needed)
turns the counter_collection.csv files that `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of this
script left in those directories into the markdown table kept in profiles/hbm_traffic.md, which is where
"roofline.traffic" comes from.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0  # MI355X dense INT8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0    # MI355X HBM3E, GB/s

TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic.md")


def load_traffic():
    """{workload: HBM bytes per step} from the table rocprofv3 counter runs produced (profiles/hbm_traffic.md); a
    workload without a row has no measured traffic (None in the bench line)."""
    out = {}
    try:
        with open(TRAFFIC_TABLE) as f:
            for line in f:
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 6 and cells[0] not in ("workload", "") and not set(cells[0]) <= set("-: "):
                    try:
                        out[cells[0]] = int(cells[5])
                    except ValueError:
                        pass
    except OSError:
        pass
    return out


def summarize_pmc(dirs):
    """Markdown table of HBM traffic per step from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script.

    Each directory holds one run of ONE workload made with `--traffic-reference --marks DIR/marks.json`: every nce::
    dispatch of the run belongs to that workload, marks.json says how many steps ran, and the plain 256 MiB device
    copies of --traffic-reference give the scale of the counter (what it reads for a copy of known size)."""
    import csv
    import glob
    runs = {}
    for d in dirs:
        marks = json.load(open(os.path.join(d, "marks.json")))
        total, ref, ctr_name = 0.0, [], None
        for path in glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True):
            for r in csv.DictReader(open(path)):
                val = float(r["Counter_Value"])
                ctr_name = r["Counter_Name"]
                if "nce::" in r["Kernel_Name"]:
                    total += val
                elif val > 0.3 * 262144:   # a 256 MiB copy (every other foreign dispatch is far smaller)
                    ref.append(val)
        if ctr_name is None or not ref:
            sys.exit(f"{d}: no counter rows or no reference copy found")
        runs.setdefault(marks["workload"], {})[ctr_name] = (total / marks["steps_total"], 262144.0 / (sum(ref) / len(ref)),
                                                             marks["algorithmic_bytes"])
    print("| workload | FETCH_SIZE per step | WRITE_SIZE per step | fetch scale | write scale | HBM bytes per step | algorithmic bytes | ratio |")
    print("|---|---|---|---|---|---|---|---|")
    for wl, c in sorted(runs.items()):
        if "FETCH_SIZE" not in c or "WRITE_SIZE" not in c:
            continue
        (f, fs, alg), (w, ws, _) = c["FETCH_SIZE"], c["WRITE_SIZE"]
        nbytes = int((f * fs + w * ws) * 1024)
        print(f"| {wl} | {f:.1f} | {w:.1f} | {fs:.3f} | {ws:.3f} | {nbytes} | {alg} | {nbytes / alg:.2f} |")


def make_workloads():
    from npu_plugin_amd import workloads as W
    return {
        "cfg2": (W.cfg2, "mfma"),
        "cfg3_dw": (W.cfg3_dw, "hbm"),
        "cfg3_maxpool": (W.cfg3_maxpool, "hbm"),
        "cfg3_avgpool": (W.cfg3_avgpool, "hbm"),
        "cfg4": (W.cfg4, "hbm"),
    }


def make_scaled_workloads():
    """The same layers at a batch that gives every CU several rounds of work: what the kernels reach once the
    ~2.4 us launch gap and the per-workgroup set-up no longer dominate (the configurations above are 3-10 us long)."""
    from npu_plugin_amd import workloads as W
    return {
        "cfg2_batch512": (lambda: W.cfg2(n=512), "mfma"),
        "conv3x3_32x56x56x256_256": (lambda: W.conv_case(W.SEED + 20, 32, 56, 56, 256, 256, name="conv3x3_32x56x56x256_256"), "mfma"),
        "cfg3_dw_batch128": (lambda: W.cfg3_dw(n=128), "hbm"),
        "cfg3_maxpool_batch512": (lambda: W.cfg3_maxpool(n=512), "hbm"),
        "cfg4_batch512": (lambda: W.cfg4(n=512), "hbm"),
    }


MIN_WARM_S = 0.03  # every measurement is preceded by at least this much GPU work (clocks ramp on an idle device)


STEPS_RUN = [0]  # steps enqueued so far, warm-up and timed (--marks reports the count after the main workload)


def warm_up(run, count, per_run=1):
    """Runs `run()` at least `count` times and for at least MIN_WARM_S of wall time, then waits for the device: the
    timed region that follows sees a device at its working clocks whatever step count the caller chose."""
    import torch
    t0 = time.perf_counter()
    done = 0
    while done < max(1, count) or time.perf_counter() - t0 < MIN_WARM_S:
        run()
        done += 1
        if done % 8 == 0:
            torch.cuda.synchronize()  # (keeps the wall clock honest: enqueues run ahead of the device)
    torch.cuda.synchronize()
    STEPS_RUN[0] += done * per_run
    return done


def time_task(ex, dc, steps, warmup, reps=1):
    """Returns (wall seconds per step, event seconds per step); with reps > 1 the median of that many timed runs of
    `steps` steps each (the side workloads: 3-15 us per step, where one run's figure moves by several per cent with the
    launch jitter of the moment)."""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    warm = ex.task_list()
    for _ in range(max(warmup, 1)):
        warm.append(dc.task)
    timed = ex.task_list()
    for _ in range(steps):
        timed.append(dc.task)
    warm_up(lambda: warm.enqueue(stream), 1, per_run=max(warmup, 1))
    runs = []
    for _ in range(max(1, reps)):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        timed.enqueue(stream)
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        STEPS_RUN[0] += steps
        runs.append(((t1 - t0) / steps, e0.elapsed_time(e1) * 1e-3 / steps))
    warm.destroy()
    timed.destroy()
    runs.sort(key=lambda r: r[1])
    return runs[len(runs) // 2]


def measure(ex, name, maker, bound, steps, warmup, reps=1):
    from npu_plugin_amd import workloads as W
    case = maker()
    dc = W.DeviceCase(case)
    wall, ev = time_task(ex, dc, steps, warmup, reps)
    ops, nbytes = case.ops(), case.algorithmic_bytes()
    if bound == "mfma":
        value, unit = ops / wall / 1e9, "GOPS"
        roof = {"bound": "mfma", "achieved": ops / ev / 1e12, "peak": PEAK_INT8_TOPS / 1.0, "unit": "TOP/s"}
        roof["peak"] = PEAK_INT8_TOPS
        roof["achieved"] = ops / ev / 1e12
    else:
        value, unit = nbytes / wall / 1e9, "GB/s"
        roof = {"bound": "hbm", "achieved": nbytes / ev / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = load_traffic().get(name)
    roof["kernel_us"] = ev * 1e6
    return case, {"workload": case.name, "value": value, "unit": unit, "ms_per_step": wall * 1e3, "ops_per_step": ops,
                  "bytes_per_step": nbytes, "roofline": roof}


def per_layer_table(ex, dg, reps=10):
    """HIP-event time of every task of the graph, run alone `reps` times back to back."""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    g = dg.graph
    rows = []
    for L, task in zip(g.layers, dg.tasks):
        tl = ex.task_list()
        for _ in range(reps):
            tl.append(task)
        warm_up(lambda: tl.enqueue(stream), 1)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        tl.enqueue(stream)
        e1.record()
        torch.cuda.synchronize()
        tl.destroy()
        us = e0.elapsed_time(e1) * 1e3 / reps
        n, oh, ow, oc = g.tensors[L.dst]
        ops = 2 * n * oh * ow * oc * L.kernel[0] * L.kernel[1] * L.real_ic if L.task_type == 0 else 0
        rows.append({"layer": L.name, "task_type": L.task_type, "out": [n, oh, ow, oc], "kernel": L.kernel,
                     "strides": L.strides, "in_ch": g.tensors[L.src][3], "us": us, "tops": ops / us / 1e6,
                     "gbs": g.layer_bytes(L) / us / 1e3})
    return rows


def measure_graph(ex, steps, warmup, batch=32, per_layer=False):
    """cfg5: the whole ResNet-50 task graph (53 convs + max pool + 16 adds) as one step."""
    import torch
    from npu_plugin_amd import workloads as W
    graph = W.ResNet50Graph(batch=batch)
    dg = W.DeviceGraph(graph, ex, graph.make_input())
    stream = torch.cuda.current_stream().cuda_stream
    warm_up(lambda: dg.run(stream), warmup)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        dg.run(stream)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    ev = e0.elapsed_time(e1) * 1e-3 / steps
    STEPS_RUN[0] += steps
    ops = graph.conv_ops()
    conv_bytes = sum(graph.layer_bytes(L) for L in graph.layers if L.task_type == 0)
    other_bytes = sum(graph.layer_bytes(L) for L in graph.layers if L.task_type != 0)
    roof = {"bound": "mfma", "achieved": ops / ev / 1e12, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
            "frac": ops / ev / 1e12 / PEAK_INT8_TOPS, "traffic": load_traffic().get("cfg5"), "kernel_us": ev * 1e6,
            "note": "whole graph per step: 53 conv + 1 max pool + 16 add tasks from one task list, launched back to back; an add that directly follows the convolution producing its input runs inside that convolution's launch"}
    layers = per_layer_table(ex, dg) if per_layer else None
    if layers:
        for r in layers:
            print(f"{r['layer']:22s} type {r['task_type']} in_ch {r['in_ch']:5d} out {r['out']} k {r['kernel']} s {r['strides']} "
                  f"{r['us']:8.1f} us {r['tops']:7.1f} TOP/s {r['gbs']:7.0f} GB/s", file=sys.stderr)
    dg.task_list.destroy()
    return {"workload": f"cfg5_resnet50_b{batch}_224", "tasks": len(graph.layers), "steps": steps, "value": ops / wall / 1e9, "unit": "GOPS",
            "ms_per_step": wall * 1e3, "ops_per_step": ops, "conv_bytes_per_step": conv_bytes,
            "pool_add_bytes_per_step": other_bytes, "roofline": roof}


def cpu_baseline(case, bound, budget_s=12.0):
    """The CPU oracle (a port of the reference's semantics; the reference itself has no executable
    arithmetic for this path) timed on the host cores, on whole passes of the same workload."""
    from oracle import nce_oracle
    from tests.cases import run_oracle
    cores = min(16, nce_oracle.lib().nce_oracle_max_threads())
    run_oracle(case, cores)  # warm
    n, t0 = 0, time.perf_counter()
    while True:
        run_oracle(case, cores)
        n += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or n >= 100:
            break
    per = dt / n
    if bound == "mfma":
        v, unit = case.ops() / per / 1e9, "GOPS"
    else:
        v, unit = case.algorithmic_bytes() / per / 1e9, "GB/s"
    return {"value": v, "unit": unit, "cores": cores, "kind": "port",
            "sample": f"{n} full passes of {case.name} ({per * 1e3:.1f} ms each)"}


def cpu_baseline_graph(batch=2, budget_s=12.0):
    """cfg5 on the CPU oracle: whole passes of the same graph at a small batch (the work per image does not depend on
    the batch: every task is independent per image), reported as conv GOPS like the GPU figure."""
    from npu_plugin_amd import workloads as W
    from oracle import nce_oracle
    from tests.cases import run_graph_oracle
    cores = min(16, nce_oracle.lib().nce_oracle_max_threads())
    graph = W.ResNet50Graph(batch=batch)
    x = graph.make_input()
    run_graph_oracle(graph, x, cores)  # warm
    n, t0 = 0, time.perf_counter()
    while True:
        run_graph_oracle(graph, x, cores)
        n += 1
        dt = time.perf_counter() - t0
        if dt > budget_s or n >= 100:
            break
    per = dt / n
    return {"value": graph.conv_ops() / per / 1e9, "unit": "GOPS", "cores": cores, "kind": "port",
            "sample": f"{n} full passes of the cfg5 graph at batch {batch} instead of 32 ({per * 1e3:.1f} ms each, "
                      f"{per / batch * 32 * 1e3:.0f} ms for a batch-32 step at the same rate)"}


def measure_chain(ex, steps, warmup):
    """cfg3 as the chain it is: depthwise -> max pool -> average pool, each reading the previous task's output, the
    three tasks of a step launched from one task list."""
    import torch
    from npu_plugin_amd import workloads as W
    dw, mp, ap = W.cfg3_dw(), W.cfg3_maxpool(), W.cfg3_avgpool()
    d_dw, d_mp, d_ap = W.DeviceCase(dw), W.DeviceCase(mp), W.DeviceCase(ap)
    tasks = [d_dw.task, W.build_task(mp, d_dw.output, None, None, d_mp.output), W.build_task(ap, d_mp.output, None, None, d_ap.output)]
    stream = torch.cuda.current_stream().cuda_stream
    warm, timed = ex.task_list(), ex.task_list()
    for tl, k in ((warm, max(1, warmup)), (timed, steps)):
        for _ in range(k):
            for t in tasks:
                tl.append(t)
    warm_up(lambda: warm.enqueue(stream), 1, per_run=max(warmup, 1))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    timed.enqueue(stream)
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    ev = e0.elapsed_time(e1) * 1e-3 / steps
    STEPS_RUN[0] += steps
    warm.destroy()
    timed.destroy()
    # algorithmic bytes of the chain: input and weights once, every output once (the intermediates are outputs of the
    # contract and must be written; a consumer re-reading them is not counted)
    nbytes = dw.algorithmic_bytes() + int(np.prod(mp.out_shape)) + int(np.prod(ap.out_shape))
    return {"workload": "cfg3_chain_dw_maxpool_avgpool_16x112x112x96", "value": nbytes / wall / 1e9, "unit": "GB/s",
            "ms_per_step": wall * 1e3, "bytes_per_step": nbytes,
            "roofline": {"bound": "hbm", "achieved": nbytes / ev / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": nbytes / ev / 1e9 / PEAK_HBM_GBS, "traffic": load_traffic().get("cfg3_chain"), "kernel_us": ev * 1e6}}


def main():
    if len(sys.argv) > 1 and sys.argv[1] == "--summarize-pmc":
        return summarize_pmc(sys.argv[2:])
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200, help="timed steps")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg5", help="cfg1..cfg5, cfg3_chain, a large-batch variant, or conv:N,H,W,IC,OC,K,STRIDE,PAD")
    ap.add_argument("--no-others", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-scaled", action="store_true", help="skip the large-batch variants of the workloads")
    ap.add_argument("--batch", type=int, default=32, help="cfg5 only: batch of the graph (profiling; the headline is 32)")
    ap.add_argument("--per-layer", action="store_true", help="cfg5: print a per-task timing table on stderr")
    ap.add_argument("--traffic-reference", action="store_true",
                    help="also run plain 256 MiB device copies, the known-size reference for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--marks", default=None, help="with --traffic-reference: write {workload, steps_total, algorithmic_bytes} here")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported (no collectives, no sharding).")

    import torch  # device memory and streams

    import npu_plugin_amd as nce
    workloads = make_workloads()
    if args.workload in make_scaled_workloads():  # a large-batch variant as the main workload (profiling)
        workloads = dict(workloads, **{args.workload: make_scaled_workloads()[args.workload]})
    if args.workload.startswith("conv:"):  # one convolution layer by shape (profiling): conv:N,H,W,IC,OC,K,STRIDE,PAD
        from npu_plugin_amd import workloads as W
        n, h, w_, ic, oc, k, st, pad = [int(x) for x in args.workload[5:].split(",")]
        workloads = dict(workloads, **{args.workload: (lambda: W.conv_case(W.SEED + 21, n, h, w_, ic, oc, k=(k, k), s=(st, st),
                                                                              pads=(pad, pad, pad, pad)), "mfma")})
    if args.workload not in workloads and args.workload not in ("cfg5", "cfg3_chain"):
        sys.exit(f"unknown workload {args.workload}; choose from {sorted(workloads) + ['cfg3_chain', 'cfg5']}")
    ex = nce.Executor(device_id=0, log_level=1)
    if args.traffic_reference:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").fill_(7)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    graph_steps, graph_warm = args.steps, max(1, args.warmup)
    # The side workloads are 3-15 us per step: they are timed over at least 200 steps whatever --steps says, so that their
    # figures do not depend on the step count chosen for the headline.
    side_steps = max(args.steps, 200)
    if args.workload == "cfg5":
        case, bound = None, "mfma"
        main_res = measure_graph(ex, graph_steps, graph_warm, batch=args.batch, per_layer=args.per_layer)
        main_res["bytes_per_step"] = main_res["conv_bytes_per_step"] + main_res["pool_add_bytes_per_step"]
        workload_name = main_res["workload"]
        steps_total = STEPS_RUN[0]
    elif args.workload == "cfg3_chain":
        case, bound = None, "hbm"
        main_res = measure_chain(ex, args.steps, args.warmup)
        main_res["ops_per_step"] = 0
        workload_name = main_res["workload"]
        steps_total = STEPS_RUN[0]
    else:
        maker, bound = workloads[args.workload]
        case, main_res = measure(ex, args.workload, maker, bound, args.steps, args.warmup)
        workload_name = case.name
        steps_total = STEPS_RUN[0]
    if args.marks:
        with open(args.marks, "w") as f:
            json.dump({"workload": args.workload, "steps_total": steps_total, "algorithmic_bytes": main_res["bytes_per_step"]}, f)
    line = {
        "metric": "INT8 GOPS & % MFMA peak (conv); GB/s & % HBM peak (dw/pool/eltwise)",
        "value": main_res["value"],
        "unit": main_res["unit"],
        "n_gpus": 1,
        "steps": main_res.get("steps", args.steps),
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 (u8 x i8 -> i32 accumulate, integer PPE)",
        "data": "synthetic (seeded uniform u8 activations, i8 weights, random per-channel mult/shift tables)",
        "config": {"workload": workload_name, "ops_per_step": main_res["ops_per_step"], "bytes_per_step": main_res["bytes_per_step"]},
        "roofline": main_res["roofline"],
    }
    if not args.no_others:
        others = {}
        for name, (mk, bd) in workloads.items():
            if name == args.workload:
                continue
            _, r = measure(ex, name, mk, bd, side_steps, args.warmup, reps=5)
            others[name] = r
        if args.workload != "cfg3_chain":
            others["cfg3_chain"] = measure_chain(ex, side_steps, args.warmup)
        if args.workload != "cfg5":
            others["cfg5"] = measure_graph(ex, graph_steps, graph_warm)
        # The same graph with the opt-in persistent segments (an executor created under NCE_HIP_PERSISTENT=1): runs of
        # weights-resident convolutions as one launch each. Not the headline: the default path is.
        saved = os.environ.get("NCE_HIP_PERSISTENT")
        os.environ["NCE_HIP_PERSISTENT"] = "1"
        try:
            ex_pk = nce.Executor(device_id=0, log_level=1)
            try:
                r = measure_graph(ex_pk, graph_steps, graph_warm)
                ex_pk.synchronize(torch.cuda.current_stream().cuda_stream)  # (reports a persistent launch that gave up)
                r["roofline"]["note"] = "NCE_HIP_PERSISTENT=1: launches 12..53 of the graph as one persistent launch"
                others["cfg5_persistent_segments"] = r
            finally:
                ex_pk.destroy()
        except Exception as e:  # the headline does not depend on this line
            others["cfg5_persistent_segments"] = {"error": str(e)[:200]}
        finally:
            if saved is None:
                del os.environ["NCE_HIP_PERSISTENT"]
            else:
                os.environ["NCE_HIP_PERSISTENT"] = saved
        line["other_workloads"] = others
        if not args.no_scaled:
            scaled = {}
            for name, (mk, bd) in make_scaled_workloads().items():
                _, r = measure(ex, name, mk, bd, 20, 3)
                scaled[name] = r
            line["scaled_workloads"] = scaled
    ex.destroy()
    if not args.no_cpu:  # after every GPU measurement: seconds of host-only work would let the device clocks fall
        if case is not None:
            line["cpu_baseline"] = cpu_baseline(case, bound)
        elif args.workload == "cfg5":
            line["cpu_baseline"] = cpu_baseline_graph()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
