#!/usr/bin/env python3
"""Benchmark of the relax-star reach path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--method relax-star-area]

A step is one full ``NN.reach`` of the benchmark configuration (default: config 2, the fully
connected 784-1024-1024-1024-10 net with a 784-generator input box) with the input set and the
weights already resident in HBM; it ends with the output set and its estimated output bounds
resident in HBM.  Prints ONE JSON line:

  metric/value   generator-neuron updates per second = sum over layer steps of N_out*(n_out+1),
                 divided by reach wall-time (ms_per_step is the reach wall-time itself)
  roofline       the dominant kernel (the fp64 MFMA GEMM of the hidden FC layers): dense flop
                 2*M*K*(n+1) per launch over its HIP-event duration, against 78.6 TFLOP/s
  cpu_baseline   the CPU oracle (numpy/OpenBLAS restatement of NNV's path, "port") timed on this
                 host on a bounded sample of the same workload
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

import nnv_amd  # noqa: E402

FP64_MFMA_PEAK_TFLOPS = 78.6
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and
# scaled by the 1 GiB copy kernel of the same run (profiles/<workload>_hbm_traffic.md): (read, write) MiB
# averaged over the launches of a step (dense GEMM: the 64x64, 64x96 and 128x80 tile instantiations; default
# path: the mapped 64x64 GEMM over the kept rows; gather: the four FC layers, three of which leave their
# columns unwritten)
MEASURED_TRAFFIC_MIB = {("cfg2_fc_784_1024x3_10", "gemm_f64_kernel", "dense"): (51.30, 12.36),
                        ("cfg2_fc_784_1024x3_10", "gemm_f64_kernel", "structured"): (8.89, 6.54),
                        ("cfg2_fc_784_1024x3_10", "gather_columns_kernel", "structured"): (4.88, 0.79)}


def layer_shapes(reach_set):
    out = []
    for s in reach_set:
        sets = s if isinstance(s, (list, nnv_amd.SetArray)) else [s]
        for t in sets:
            N, n, _ = t._h.dims()
            out.append((N, n))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default: as many as fill about 0.3 s, between 10 and 1000)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: steps / 10, at least 5)")
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--method", default="relax-star-area")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--dense", action="store_true",
                    help="run every FC layer as the full dense contraction (no skipping of structural zeros)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    ap.add_argument("--lean", action="store_true",
                    help="only the timed steps and the per-kernel timing pass (no dense-contraction, host-to-host, "
                         "all-sets-written and specification passes): what the rocprofv3 summaries in profiles/ run, so "
                         "that their kernel tables hold the kernels of the measured path only")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (sets shard across GPUs without communication; "
                 "that path is not built) - use --gpus 1")

    from nnv_amd.configs import count_updates, device_input_sets, make_config, make_extended_cnn

    cfg = make_extended_cnn(32, 3) if args.config == 6 else make_config(args.config)
    ctx = nnv_amd.default_context()
    ctx.set_dense_affine(args.dense)
    net = nnv_amd.NN.from_config(cfg["layers"], cfg["name"])
    opts = {"reachMethod": args.method, "relaxFactor": 1}
    dev_in = device_input_sets(cfg, ctx)
    lib, h = ctx.lib, ctx.handle

    def step():
        out = net.reach(dev_in, opts)
        outs = out if isinstance(out, (list, nnv_amd.SetArray)) else [out]
        arr = outs.handles() if isinstance(outs, nnv_amd.SetArray) else (ctypes.c_void_p * len(outs))(*[o_._h.h for o_ in outs])
        # output bounds of all sets in one batched call, left on the device
        nnv_amd._lib.check(lib.nnvhip_estimate_ranges_batch(h, len(outs), arr, None, None))
        return out

    if args.steps is None:
        # a reach takes between 0.1 ms and 0.2 s depending on the workload: size the timed region so that
        # clocks have settled and the timer's granularity does not matter
        for _ in range(3):
            step()
        ctx.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            step()
        ctx.synchronize()
        args.steps = int(min(1000, max(10, 0.3 / max((time.perf_counter() - t0) / 3, 1e-6))))
    if args.warmup is None:
        args.warmup = max(5, args.steps // 10)
    for _ in range(args.warmup):
        step()
    ctx.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    ctx.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = 1e3 * wall / args.steps
    shapes = layer_shapes(net.reachSet)
    updates = count_updates(shapes)
    value = updates / (wall / args.steps)

    # ---- per-layer and per-kernel timing with HIP events on the library's stream -----------------
    # set_timing brackets every layer call (NN.reachTime) and, separately, every launch of the two
    # MFMA kernels with their own event pair, so the kernel's duration excludes host gaps.
    reps = max(5, min(args.steps, 20))

    def timed_pass(level):
        rs = dev_in
        for L in net.Layers:   # untimed pass: the layer-by-layer call pattern settles its own pool blocks
            rs = L.reach(rs, args.method, [], 1, None, "linprog")
        del rs
        ctx.set_timing(level)
        acc = np.zeros(len(net.Layers))
        for _ in range(reps):
            rs = dev_in
            for i, L in enumerate(net.Layers):
                rs = L.reach(rs, args.method, [], 1, None, "linprog")
                acc[i] += ctx.last_op_time_ms()
        ctx.set_timing(0)
        return acc / reps

    per_layer = timed_pass(1)          # NN.reachTime-style device time per layer
    for grp in range(8):
        ctx.kernel_time(grp)
    timed_pass(2)                      # per-kernel event pairs
    gemm_ms, gemm_launches, gemm_work = ctx.kernel_time(0)
    conv_ms, conv_launches, conv_work = ctx.kernel_time(1)
    rng_ms, rng_launches, rng_bytes = ctx.kernel_time(2)
    app_ms, app_launches, app_bytes = ctx.kernel_time(3)
    row_ms, row_launches, row_bytes = ctx.kernel_time(4)
    gat_ms, gat_launches, gat_bytes = ctx.kernel_time(5)
    cls_ms, cls_launches, cls_bytes = ctx.kernel_time(6)
    fin_ms, fin_launches, fin_bytes = ctx.kernel_time(7)

    # algorithmic (unpadded, dense) flop of the launches the kernel timers cover
    gemm_flop = conv_flop = 0.0
    relu_bytes, relu_ms = 0.0, 0.0
    # bytes of the output columns the gather passes stand for (8 * rows per one-hot input column), whether
    # a pass writes them or leaves them pending
    gat_dense_bytes = 0.0
    onehot_cols = [s._h.dims()[1] for s in (dev_in if isinstance(dev_in, (list, nnv_amd.SetArray)) else [dev_in])] \
        if cfg["layers"][0]["type"] == "fc" else None
    layer_report = []
    prev_sets = dev_in if isinstance(dev_in, (list, nnv_amd.SetArray)) else [dev_in]
    for i, (Ld, L) in enumerate(zip(cfg["layers"], net.Layers)):
        outs = net.reachSet[i] if isinstance(net.reachSet[i], (list, nnv_amd.SetArray)) else [net.reachSet[i]]
        entry = {"layer": i + 1, "type": Ld["type"], "ms": round(float(per_layer[i]), 4)}
        if Ld["type"] == "fc":
            M, K = Ld["W"].shape
            cols = sum(s._h.dims()[1] + 1 for s in outs)
            flop = 2.0 * M * K * cols
            entry["dense_equivalent_tflops"] = round(flop / (per_layer[i] * 1e-3) / 1e12, 3)
            if M > 32:  # the 64-row-tile kernel; skinnier layers use another instantiation
                gemm_flop += flop
            if onehot_cols is not None:
                gat_dense_bytes += 8.0 * M * sum(onehot_cols)
            onehot_cols = None
        elif Ld["type"] == "conv":
            fh, fw, cin, cout = Ld["W"].shape
            flop = 0.0
            for s in outs:
                N, n, _ = s._h.dims()
                flop += 2.0 * (N // cout) * cout * fh * fw * cin * (n + 1)
            entry["dense_equivalent_tflops"] = round(flop / (per_layer[i] * 1e-3) / 1e12, 3)
            conv_flop += flop
        elif Ld["type"] in ("batchnorm", "avgpool", "flatten", "imageinput"):
            b = sum(8.0 * (sp._h.dims()[0] + so._h.dims()[0]) * (sp._h.dims()[1] + 1) for sp, so in zip(prev_sets, outs))
            if per_layer[i] > 0:
                entry["algo_GBps"] = round(b / (per_layer[i] * 1e-3) / 1e9, 1)
        elif Ld["type"] == "relu":
            b = 0.0
            for sp, so in zip(prev_sets, outs):
                N, n, _ = sp._h.dims()
                m = so._h.dims()[1] - n
                # read of the rows the step keeps + write of the N x (n+1+m) output, plus the
                # estimateRanges read of V unless the producing FC layer already left the range sums
                fused = i > 0 and cfg["layers"][i - 1]["type"] == "fc" and len(outs) == 1
                ni, nc = ctypes.c_int64(), ctypes.c_int64()
                nnv_amd._lib.check(ctx.lib.nnvhip_star_relu_counts(so._h.h, ctypes.byref(ni), ctypes.byref(nc)))
                kept = N - ni.value - nc.value
                # (the m appended unit-vector columns stay implicit unless a later read asks for them)
                b += 8.0 * N * (n + 1) * (0 if fused else 1) + 8.0 * kept * (n + 1) + 8.0 * N * (n + 1)
            entry["algo_GBps"] = round(b / (per_layer[i] * 1e-3) / 1e9, 1)
            relu_bytes += b
            relu_ms += per_layer[i]
            onehot_cols = [so._h.dims()[1] - sp._h.dims()[1] for sp, so in zip(prev_sets, outs)]   # the appended columns
        layer_report.append(entry)
        prev_sets = outs
        if Ld["type"] != "relu":
            onehot_cols = None

    # MFMA kernels: flop the kernel executed (the library's own count for its launches: products with
    # structural zeros that the FC map skips are not counted) over the kernels' HIP-event durations;
    # dense_equivalent = the dense count of the same layers, 2*M*K*(n+1), as the reference executes them
    def mfma_roofline(name, work_total, dense_flop_per_step, ms_total, launches):
        ach = work_total / (ms_total * 1e-3) / 1e12
        return {"kernel": name, "bound": "mfma", "achieved": round(ach, 3), "peak": FP64_MFMA_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": round(ach / FP64_MFMA_PEAK_TFLOPS, 4), "traffic": None,
                "launches_per_step": launches // reps, "avg_launch_ms": round(ms_total / launches, 5),
                "flop_per_launch": work_total / launches,
                "dense_equivalent_flop_per_step": dense_flop_per_step,
                "dense_equivalent_achieved": round(dense_flop_per_step * reps / (ms_total * 1e-3) / 1e12, 3),
                "ms_per_step": round(ms_total / reps, 5)}

    def hbm_roofline(name, ms_, n_, b_):
        g = b_ / (ms_ * 1e-3) / 1e9
        return {"kernel": name, "bound": "hbm", "achieved": round(g, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(g / HBM_PEAK_GBS, 4), "traffic": None, "launches_per_step": n_ // reps,
                "avg_launch_ms": round(ms_ / n_, 5), "bytes_per_launch": b_ / n_, "ms_per_step": round(ms_ / reps, 5)}

    # the dominant kernel group of a reach, by summed kernel time
    groups = []
    if gemm_launches:
        groups.append((gemm_ms, mfma_roofline("gemm_f64_kernel", gemm_work, gemm_flop, gemm_ms, gemm_launches)))
    if conv_launches:
        groups.append((conv_ms, mfma_roofline("conv2d_f64_kernel", conv_work, conv_flop, conv_ms, conv_launches)))
    if rng_launches:
        groups.append((rng_ms, hbm_roofline("ranges_partial_kernel", rng_ms, rng_launches, rng_bytes)))
    if app_launches:
        groups.append((app_ms, hbm_roofline("relu_apply_kernel", app_ms, app_launches, app_bytes)))
    if row_launches:
        groups.append((row_ms, hbm_roofline("row-wise affine layers (rowmap/avgpool/permute kernels)", row_ms, row_launches, row_bytes)))
    if gat_launches:
        g = hbm_roofline("gather_columns_kernel", gat_ms, gat_launches, gat_bytes)
        if not ctx.eager_columns and not args.dense:
            # all FC layers but the last leave the gathered columns unwritten (range sums only): those
            # launches run out of the cache-resident weights and are bound by L2 / ALU rate, not by HBM
            g["columns_left_unwritten"] = True
            if all(Ld["type"] in ("fc", "relu") for Ld in cfg["layers"]):   # (CNNs: the group also holds the stamp passes)
                g["dense_equivalent_GBps"] = round(gat_dense_bytes * reps / (gat_ms * 1e-3) / 1e9, 1)
        groups.append((gat_ms, g))
    if fin_launches:
        groups.append((fin_ms, hbm_roofline("ranges_final_kernel", fin_ms, fin_launches, fin_bytes)))
    groups.sort(key=lambda g: -g[0])
    roofline = dict(groups[0][1])
    roofline["other_kernels"] = [g[1] for g in groups[1:]]
    n_sets = len(dev_in) if isinstance(dev_in, (list, nnv_amd.SetArray)) else 1
    if cls_launches:
        # One block per set (classification, in-block sort of the crossing list, new predicate bounds): a
        # dependent chain on a single CU, bound by latency and not by a roofline.  It is listed with the
        # bytes it touches; with a single input set it can be the longest kernel of a reach, and the
        # roofline object above then describes the longest throughput-bound kernel.
        c = hbm_roofline("relu_classify_kernel", cls_ms, cls_launches, cls_bytes)
        c["latency_bound"] = True
        c["blocks_per_launch"] = n_sets
        roofline["other_kernels"].append(c)
        if cls_ms > groups[0][0]:
            roofline["longest_kernel_by_time"] = "relu_classify_kernel (latency bound, %d block(s) per launch)" % n_sets
    # the MFMA GEMM on the full dense problem of the same reach (what Star.affineMap executes in the
    # reference): a short extra pass with the skipping of structural zeros switched off
    if gemm_launches and not args.dense and not args.lean:
        ctx.set_dense_affine(True)
        step()
        ctx.synchronize()
        t1 = time.perf_counter()
        for _ in range(reps):
            step()
        ctx.synchronize()
        dense_ms_per_step = (time.perf_counter() - t1) / reps * 1e3
        ctx.kernel_time(0)
        timed_pass(2)
        d_ms, d_launches, d_work = ctx.kernel_time(0)
        ctx.set_dense_affine(False)
        net.reach(dev_in, opts)   # reachSet back to the default path for what follows
        if d_launches:
            dr = mfma_roofline("gemm_f64_kernel", d_work, gemm_flop, d_ms, d_launches)
            dr["reach_ms_per_step"] = round(dense_ms_per_step, 5)
            tr = MEASURED_TRAFFIC_MIB.get((cfg["name"], "gemm_f64_kernel", "dense"))
            if tr is not None and args.method == "relax-star-area":
                dr["traffic"] = round((tr[0] + tr[1]) * 1048576.0)
            roofline["dense_contraction"] = dr
    t = MEASURED_TRAFFIC_MIB.get((cfg["name"], roofline["kernel"], "dense" if args.dense else "structured"))
    if t is not None and args.method == "relax-star-area":
        roofline["traffic"] = round((t[0] + t[1]) * 1048576.0)
    if relu_ms > 0:
        # bytes the dense materialisation of the ReLU steps would move (read V for the ranges, read the kept
        # rows, write the output) over the time the steps took; the steps leave most of that undone (pending
        # row reset, range sums from the producing layer), so this can exceed the HBM peak
        roofline["relu_step_dense_equivalent_GBps"] = round(relu_bytes / (relu_ms * 1e-3) / 1e9, 1)

    # ---- the same step with the host buffers the boundary takes and returns (not `value`) -----------
    # lb / ub uploaded and the input set built on the device, the reach, the output bounds back on the host
    n_h2h = 0 if args.lean else max(5, min(args.steps, 50))
    ctx.synchronize()
    t1 = time.perf_counter()
    fresh = res = None
    for _ in range(n_h2h):
        fresh = device_input_sets(cfg, ctx)
        res = net.reach(fresh, opts)
        nnv_amd.Star.estimateRanges_array(res if isinstance(res, (list, nnv_amd.SetArray)) else [res])
    host_to_host_ms = 1e3 * (time.perf_counter() - t1) / max(n_h2h, 1)
    del fresh, res

    # ---- the same step with every intermediate set written out in full (not `value`) -------------
    # By default the sets between the layers keep what nobody reads before the next layer as a description
    # (a ReLU's row reset and appended columns, columns gathered from the weights) and write it on first
    # read; the returned set and its bounds are always written.  Here every layer writes its whole output.
    all_written_ms = None
    if not args.dense and not args.lean:
        ctx.set_eager_columns(True)
        ctx.set_eager_relu(True)
        try:
            for _ in range(3):
                step()
            ctx.synchronize()
            n_aw = max(5, min(args.steps, 100))
            t1 = time.perf_counter()
            for _ in range(n_aw):
                step()
            ctx.synchronize()
            all_written_ms = 1e3 * (time.perf_counter() - t1) / n_aw
        finally:
            ctx.set_eager_columns(False)
            ctx.set_eager_relu(False)
        net.reach(dev_in, opts)   # reachSet back to the default path for what follows

    # ---- specification check on the resident output sets (not part of `value`) -----------------
    spec = None
    last = net.Layers[-1]
    if hasattr(last, "Bias") and len(last.Bias) > 1 and not args.lean:
        from nnv_amd import verify
        out_sets = net.reachSet[-1]
        hs = net.robustness_set(0, "max")
        verify.halfspace_check(out_sets, hs)
        ctx.synchronize()
        t1 = time.perf_counter()
        for _ in range(10):
            verdict, _, _ = verify.halfspace_check(out_sets, hs)
        ctx.synchronize()
        spec = {"ms": round((time.perf_counter() - t1) / 10 * 1e3, 4), "sets": int(verdict.shape[0]),
                "halfspaces": int(verdict.shape[1]),
                "decided_without_lp": int(np.sum(verdict != verify.HS_UNDECIDED)), "pairs": int(verdict.size),
                "what": "LP-free pass of verify_specification for robustness_set(target=0): G*[c V], row bounds, verdicts"}

    # practical HBM ceiling on this box: a plain copy kernel over 1 GiB (read + write bytes)
    roofline["measured_mfma_TFLOPs"] = round(ctx.probe_mfma_peak(3), 2)     # register-resident MFMA loop
    roofline["measured_copy_GBps"] = round(ctx.probe_copy_bandwidth(1 << 30, 5), 1)
    ctx.trim_pool()

    # ---- CPU baseline: the oracle on this host -------------------------------------------------
    cpu = None
    if not args.no_cpu:
        from oracle import nnv_oracle as o
        if "partition" in cfg:
            ora_in = [o.star_from_box(l, u) for (l, u) in o.box_partition(
                cfg["lb"], cfg["ub"], cfg["partition"]["indexes"], cfg["partition"]["numbers"])]
        elif cfg["kind"] == "image":
            sh = cfg["image_shape"]
            ora_in = o.image_star_from_bounds(cfg["lb"].reshape(sh, order="F"), cfg["ub"].reshape(sh, order="F"))
        else:
            ora_in = o.star_from_box(cfg["lb"], cfg["ub"])
        n_cpu, t_cpu = 0, 0.0
        while t_cpu < args.cpu_seconds and n_cpu < 200:
            t1 = time.perf_counter()
            o.nn_reach(cfg["layers"], ora_in, args.method, 1.0)
            t_cpu += time.perf_counter() - t1
            n_cpu += 1
        threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        cpu = {"value": updates / (t_cpu / n_cpu), "unit": "updates/s", "cores": threads, "kind": "port",
               "ms_per_reach": round(1e3 * t_cpu / n_cpu, 2),
               "sample": "%d full %s reach(es) by the numpy/OpenBLAS oracle (dense C built at every ReLU, as NNV does)"
                         % (n_cpu, cfg["name"])}

    print(json.dumps({
        "metric": "generator_neuron_updates_per_s", "value": value, "unit": "updates/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": cfg["name"], "reach_method": args.method, "relax_factor": 1,
                   "fc_affine_map": "dense" if args.dense else "structural zeros skipped (one-hot generator columns, reset rows); exact",
                   "sets": len(dev_in) if isinstance(dev_in, (list, nnv_amd.SetArray)) else 1,
                   "updates_per_step": updates,
                   "intermediate_sets": "dense" if args.dense else
                   "the sets between layers record a ReLU's row reset / appended columns and the columns an FC layer "
                   "gathers from its weights and write them on first read; the returned set and its bounds are written",
                   "predicates_per_layer": [n for (_, n) in shapes][:len(net.Layers)] if not isinstance(dev_in, (list, nnv_amd.SetArray)) else None},
        "roofline": roofline, "cpu_baseline": cpu, "spec_check": spec,
        "host_to_host": None if n_h2h == 0 else
        {"ms_per_step": round(host_to_host_ms, 4), "steps": n_h2h,
         "what": "input bounds uploaded and the set(s) built, reach, output bounds fetched to the host"},
        "all_sets_written": None if all_written_ms is None else
        {"ms_per_step": round(all_written_ms, 5), "value": updates / (all_written_ms * 1e-3),
         "what": "the same step with every layer writing its whole output matrix in the call (nothing left for a first read)"},
        "layers": layer_report,
    }))


if __name__ == "__main__":
    main()
