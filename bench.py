#!/usr/bin/env python3
"""Headline benchmark: rows/s of decision-forest inference on one MI355X.

Workload: BASELINE.json configs[1] - 1000 trees, depth <= 8, 28 features,
binary:logistic, 2^20-row batch, rows already resident in HBM.  One "step" is
one pass of the hot path (walk kernel + output transform) over the batch; the
timed steps are enqueued back to back on one stream and synchronised once.
Prints ONE JSON line with the throughput, the roofline fractions of the walk
kernel (measured live with HIP events on the runtime's own stream) and the CPU
baseline (the oracle's multithreaded one-tree-at-a-time schedule) timed on the
host cores on a bounded sample.
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                      # MI355X HBM3E, published
LDS_PEAK_GBS = 256 * 256 * 2.4             # 256 CUs x 256 B/clk x 2.4 GHz = 157 286 GB/s, nominal


def print_lds_read_costs():
    """Table of cycles per wave-level LDS read per compute unit (nominal shader clock), from the bench-only library."""
    import torch                                                  # initialises the device the library measures on
    from treebeard_amd.runtime_api import LDS_READ_OPS, lds_read_cost
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU")
    patterns = [(0, "lane i reads element i"), (1, "random over 48 KB"), (2, "random over 1 KB"),
                (5, "random among 32 elements"), (6, "random among 64 elements"), (7, "random among 128 elements")]
    masks = ["all lanes", "lanes 0-31", "even lanes", "random half", "random quarter"]
    print("| instruction | address pattern | lanes active | cycles per read per CU |")
    print("|---|---|---|---|")
    for op, name in enumerate(LDS_READ_OPS):
        for pattern, pattern_name in patterns:
            if pattern >= 5 and name not in ("ds_read_b32", "ds_read_b64", "ds_read2_b32"):
                continue
            for mask, mask_name in enumerate(masks):
                if mask > 0 and name not in ("ds_read_b32", "ds_read_b64"):
                    continue
                print("| %s | %s | %s | %.2f |" % (name, pattern_name, mask_name, lds_read_cost(op, pattern, mask)), flush=True)


def plan_key(plan):
    """The fields of a plan description that decide which kernel runs and how (what a traffic figure is tied to)."""
    keep = ("kernel", "rowsPerBlock", "treeThreads", "treeLanes", "interleave", "groupBytes", "treeSlices", "quantizedRows",
            "rankRows16", "tileSize", "staging", "peelWalks")
    fields = dict(item.split("=", 1) for item in plan.split() if "=" in item)
    return " ".join("%s=%s" % (k, fields[k]) for k in keep if k in fields)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (default: the headline, 2)")
    ap.add_argument("--rows", type=int, default=0, help="override the batch size")
    ap.add_argument("--tile-size", type=int, default=1, help="CompilerOptions tile size (2, 3, 4 run the tiled walk kernel)")
    ap.add_argument("--group-staging", type=int, default=0, choices=[0, 1, 2],
                    help="how tree groups reach LDS: 0 by rule, 1 through prefetch registers, 2 direct global-to-LDS copies")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pin-plan", default="", metavar="ROWS,THREADS,K,GROUPBYTES,SLICES[,peel][,rank16]",
                    help="skip the search and pin this shape of the row-parallel kernel (what a tuned run printed as its plan): "
                         "the profiling commands use it, so that every launch of the traced kernel has the measured shape")
    ap.add_argument("--plan", choices=["tuned", "default"], default="tuned",
                    help="tuned: the library's timed launch-plan search (what the reference's findBestGPUScheduleAndCompileModel "
                         "stands for) picks the plan on this batch before anything is measured; default: the analytic plan")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU-baseline duration")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="also run one plain device copy of this many MiB (counter calibration for rocprofv3 --pmc)")
    ap.add_argument("--lds-read-costs", action="store_true",
                    help="print what the LDS of this device charges per wave-level read (instruction x address pattern x exec mask) and exit")
    args = ap.parse_args()
    if args.lds_read_costs:
        return print_lds_read_costs()
    if args.gpus != 1:
        sys.exit("bench.py: this engine runs on ONE GPU (a batch would shard by rows, each GPU holding the whole model) - use --gpus 1")

    import numpy as np
    import torch

    from treebeard_amd import synth, treebeard

    cfg = synth.CONFIGS[args.config]
    rows = args.rows or cfg.batch
    cache = os.path.join(tempfile.gettempdir(), "treebeard_amd_models")
    model = synth.model_path(args.config, cache)
    x = cfg.batch_rows(rows)
    options = treebeard.CompilerOptions(rows, args.tile_size)
    if cfg.num_class > 0:                       # class ids as int8, the reference's multiclass setting
        options.SetReturnTypeWidth(8)
        options.SetReturnTypeIsFloatType(False)
    runner = treebeard.TreebeardInferenceRunner.FromModelFile(model, "", options)
    if args.group_staging:
        runner.set_group_staging(args.group_staging)
    multiclass = runner.num_classes() > 0
    dx = torch.from_numpy(x).cuda()
    out = torch.zeros(rows, dtype=torch.int8 if multiclass else torch.float32, device="cuda")
    default_plan = runner.describe_plan()
    default_plan_ms = None
    if args.pin_plan:
        parts = args.pin_plan.split(",")
        shape = [int(v) for v in parts[:5]]
        if "rank16" in parts[5:]:
            runner.set_rank16_plan(*shape)
        else:
            runner.set_plan(*shape)
        if "peel" in parts[5:]:
            runner.enable_peeled_walks(dx.data_ptr(), rows)
    elif args.plan == "tuned":
        # the analytic plan's own time, for comparison: after enough launches for the clocks to have ramped up, the
        # better of two passes (the search judges its finalists the same way)
        runner.time_kernels3(dx.data_ptr(), out.data_ptr(), rows, 40)
        default_plan_ms = min(sum(runner.time_kernels3(dx.data_ptr(), out.data_ptr(), rows, 10)) for _ in range(2))
        runner.autotune(dx.data_ptr(), rows)
    if args.copy_calibration:
        # a plain device copy of known size: scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run
        a = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        b.copy_(a)
        torch.cuda.synchronize()

    # kernel-only durations: HIP events on the stream the kernels are launched on (the runtime's own).  Measured
    # before the timed steps, which therefore start on a device that is already at its working clock.
    runner.time_kernels3(dx.data_ptr(), out.data_ptr(), rows, max(args.steps, 5))      # (first pass: clocks ramp up)
    walk_ms, fin_ms, bin_ms = runner.time_kernels3(dx.data_ptr(), out.data_ptr(), rows, max(args.steps, 5))
    path_ms = walk_ms + fin_ms + bin_ms

    # A step = one pass of the hot path over the resident batch.  The steps are handed over the way a serving loop
    # hands over its batches: enqueued back to back on the caller's stream (tbmi_run_device_async), one
    # synchronisation on either side of the timed region.  The same steps through tbmi_run_device, which waits
    # for every call, are timed beside them (`ms_per_step_sync_every_call`).
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        runner.run_device_async(dx.data_ptr(), out.data_ptr(), rows, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        runner.run_device_async(dx.data_ptr(), out.data_ptr(), rows, stream)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    rows_per_s = rows / (elapsed / args.steps)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        runner.run_device(dx.data_ptr(), out.data_ptr(), rows)      # returns when the runtime's stream has drained
    torch.cuda.synchronize()
    ms_per_step_sync = (time.perf_counter() - t0) / args.steps * 1e3

    # algorithmic bytes per row.  HBM: the row once (4 F) + the output.  LDS: every visited internal node reads
    # 6 B of node (f32 threshold + i16 feature index) and the 4 B feature value from the LDS row tile, every tree
    # ends with a 4 B leaf read; the visit count is measured exactly by the oracle on a sample of the same rows.
    from oracle import cpu_oracle, model_io
    forest = model_io.load_xgboost_json(model)
    sample = min(rows, 8192)
    steps_per_row = cpu_oracle.total_steps(forest, x[:sample]) / sample
    hbm_bytes_row = 4 * cfg.num_features + (1 if multiclass else 4)
    lds_bytes_row = steps_per_row * 10 + 4 * forest.num_trees
    hbm_time = hbm_bytes_row * rows / (HBM_PEAK_GBS * 1e9)
    lds_time = lds_bytes_row * rows / (LDS_PEAK_GBS * 1e9)
    binding = "lds" if lds_time > hbm_time else "hbm"
    plan = runner.describe_plan()
    quantized = "quantizedRows=1" in plan or "rankRows16=1" in plan       # a ranking kernel runs in front of the walk
    plan_fields = dict(item.split("=", 1) for item in plan.split() if "=" in item)
    kernel = ("WalkRowsTiledKernel" if " tileSize=1 " not in plan else "WalkRowsLdsKernel") if "rows_lds" in plan else \
        ("WalkGlobalKernel" if "global_walk" in plan else "WalkTreeParallelKernel")
    # the rank-quantised path reads the f32 rows in its binning kernel: both kernels count for the HBM roofline
    hbm_ms = walk_ms + bin_ms if quantized else walk_ms
    hbm_gbs = hbm_bytes_row * rows / (hbm_ms * 1e-3) / 1e9
    lds_gbs = lds_bytes_row * rows / (walk_ms * 1e-3) / 1e9
    # measured alongside the published peak: a plain device copy (bytes read + bytes written per second)
    # (left out of counter-calibration runs, which want exactly one copy of known size in their trace)
    copy_gbs = None
    if not args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(5):
            dst.copy_(src)
        ev1.record()
        torch.cuda.synchronize()
        copy_gbs = 5 * 2 * (1 << 30) / (ev0.elapsed_time(ev1) * 1e-3) / 1e9
        del src, dst
    # ... and the LDS: conflict-free reads of 4, 8 and 16 bytes per lane on every CU (the library's micro-benchmark)
    lds_measured = None
    if not args.copy_calibration:
        from treebeard_amd.runtime_api import lds_read_bandwidth      # the bench-only library libtbamd_bench.so
        lds_measured = {"b%d" % (8 * width): lds_read_bandwidth(width) / 1e9 for width in (4, 8, 16)}
    # What the LDS pipes need at those measured rates for this kernel's own mix (an 8-byte node read and a 4-byte
    # feature read per level, a 4-byte leaf read per tree): for the visited nodes only, and for the lock-step walk
    # that takes every row through the depth of each tree (the depth of the deepest tree of a bundle, in fact).
    lds_floor = None
    if lds_measured and binding == "lds":
        per_level = 8.0 / (lds_measured["b64"] * 1e9) + 4.0 / (lds_measured["b32"] * 1e9)
        per_leaf = 4.0 / (lds_measured["b32"] * 1e9)
        # (peeled walks stop trees early: the plan says how many levels its lock-step walk takes per row)
        depth_sum = float(plan_fields.get("lockStepSteps") or sum(forest.depth(t) for t in range(forest.num_trees)))
        visited_ms = rows * (steps_per_row * per_level + forest.num_trees * per_leaf) * 1e3
        lockstep_ms = rows * (depth_sum * per_level + forest.num_trees * per_leaf) * 1e3
        lds_floor = {"visited_nodes_ms": visited_ms, "frac_of_visited_floor": visited_ms / walk_ms,
                     "lockstep_levels_per_row": depth_sum, "lockstep_ms": lockstep_ms,
                     "frac_of_lockstep_floor": lockstep_ms / walk_ms}
    # HBM bytes per launch of the timed kernels, from rocprofv3 FETCH_SIZE + WRITE_SIZE runs of this same command
    # (scaled by a plain copy of known size); read from the committed summary, not measured in this run
    traffic, traffic_note = None, None
    traffic_file = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(traffic_file):
        with open(traffic_file) as fh:
            entries = json.load(fh).get("%s@%d" % (cfg.name, rows), [])
        # the counters were taken on one launch plan each: a figure measured on another plan is not this run's traffic
        match = [e for e in entries if e.get("plan") == plan_key(plan)]
        if match:
            traffic = match[0].get("bytes_per_launch")
        elif entries:
            traffic_note = ("profiles/hbm_traffic.json holds figures for the plans %s; this run used [%s]"
                            % ("; ".join("[%s]" % e.get("plan") for e in entries), plan_key(plan)))

    # The roofline that binds this workload (the larger of the two times above): LDS node + feature reads for the
    # narrow models, HBM row streaming for the wide one.  `achieved` = algorithmic bytes per launch / the dominant
    # kernel's launch duration (for the rank-quantised path the binning kernel reads the rows, so both count).
    hbm_view = {"bound": "hbm", "achieved": hbm_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": hbm_gbs / HBM_PEAK_GBS,
                "algorithmic_bytes_per_row": hbm_bytes_row, "measured_copy_gbs": copy_gbs,
                "frac_of_measured_copy": hbm_gbs / copy_gbs if copy_gbs else None}
    lds_view = {"bound": "lds", "achieved": lds_gbs, "peak": LDS_PEAK_GBS, "unit": "GB/s", "frac": lds_gbs / LDS_PEAK_GBS,
                "algorithmic_bytes_per_row": lds_bytes_row, "visited_nodes_per_row": steps_per_row,
                "measured_lds_read_gbs": lds_measured, "lds_floor": lds_floor,
                "frac_of_measured_lds": (lds_gbs / lds_measured["b128"]) if lds_measured else None,
                "peak_note": "256 CUs x 256 B/clk x 2.4 GHz; a scalar walk moves 10 B per lane in two LDS "
                             "instructions of about 2.5 clk each (measured), so about 50 % is its ceiling"}
    roofline = dict(lds_view if binding == "lds" else hbm_view)
    roofline.update({"traffic": traffic, "traffic_source": "profiles/hbm_traffic.json (rocprofv3 FETCH_SIZE + WRITE_SIZE "
                                                           "of this command, scaled by a plain copy)" if traffic else traffic_note,
                     "kernel": ("RankRows16Kernel+" if "rankRows16=1" in plan else "BinRowsKernel+" if quantized else "") + kernel,
                     "kernel_ms": hbm_ms if binding == "hbm" else walk_ms,
                     "walk_ms": walk_ms, "finalize_ms": fin_ms, "bin_ms": bin_ms, "path_ms": path_ms})

    line = {
        "metric": "rows/sec at 1 MI355X (2^20-row batch) + % of binding HBM/LDS roofline",
        "value": rows_per_s, "unit": "rows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_sync_every_call": ms_per_step_sync, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg.name, "rows": rows, "trees": forest.num_trees, "features": cfg.num_features,
                   "objective": cfg.objective, "plan": plan,
                   "plan_source": "pinned (--pin-plan %s)" % args.pin_plan if args.pin_plan
                   else "timed search over launch plans on this batch (tbmi_autotune)" if args.plan == "tuned" else "analytic default", "default_plan": default_plan, "default_plan_path_ms": default_plan_ms},
        "roofline": roofline,
        "roofline_other": hbm_view if binding == "lds" else lds_view,   # the memory roofline that does not bind
    }

    if not args.no_cpu_baseline:
        # The reference's multithreaded CPU configuration restated in oracle/tiled_oracle.c: uniform tiling with
        # tile size 8, sparse tile layout + LUT, trees ordered by depth, the batch split evenly over the threads,
        # one tree at a time inside a chunk, f32 accumulation.  Timed on a bounded sample of the same batch.
        threads = cpu_oracle.max_threads()
        order = np.argsort([forest.depth(t) for t in range(forest.num_trees)], kind="stable").astype(np.int32)
        tiled = cpu_oracle.TiledForest(forest, 8)
        if multiclass:
            run = lambda n: tiled.predict_tree_outer_multiclass(x[:n], tree_order=order, threads=threads)[0].astype(np.float32)
        else:
            run = lambda n: tiled.predict_tree_outer(x[:n], tree_order=order, threads=threads)
        what = ("uniform tiling, tile size 8, sparse layout + LUT, depth-ordered trees, one tree at a time, "
                "batch split over %d threads%s" % (threads, ", f32 class sums and the generated code's arg-max" if multiclass else ""))
        probe = min(rows, 4096)
        run(probe)
        t0 = time.perf_counter()
        run(probe)
        per_row = (time.perf_counter() - t0) / probe
        cpu_rows = int(min(rows, max(probe, args.cpu_seconds / max(per_row, 1e-9))))
        t0 = time.perf_counter()
        cpu_out = run(cpu_rows)
        cpu_s = time.perf_counter() - t0
        line["cpu_baseline"] = {"value": cpu_rows / cpu_s, "unit": "rows/s", "cores": threads, "kind": "port",
                                "sample": "first %d rows of the same batch; %s" % (cpu_rows, what)}
        # the scalar walker (one thread, one row at a time, every tree) on a small sample, for scale
        scalar_rows = int(min(cpu_rows, 2048))
        t0 = time.perf_counter()
        cpu_oracle.predict(forest, x[:scalar_rows], threads=1)
        line["cpu_baseline"]["scalar_one_thread_rows_per_s"] = scalar_rows / (time.perf_counter() - t0)
        got = out[:cpu_rows].cpu().numpy().astype(np.float32)
        line["cpu_baseline"]["max_abs_diff_vs_gpu"] = float(np.abs(got - cpu_out).max())
        line["cpu_baseline"]["diff_note"] = ("this baseline adds the trees in f32 like the reference's generated code; "
                                             "the parity tests compare with the double-accumulating scalar walker")
    print(json.dumps(line))


if __name__ == "__main__":
    main()
