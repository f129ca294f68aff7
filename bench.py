#!/usr/bin/env python3
"""Benchmark of the relax-star reach path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config k] [--method relax-star-area]

A step is one full ``NN.reach`` of a benchmark configuration with the input set(s) and the weights
already resident in HBM; it ends with the output set(s) and their estimated output bounds resident in
HBM.  Without ``--config`` all five configurations are measured in one run and ONE JSON line is printed:

  headline       configuration 5 (the 1024 sub-boxes of config 2's input box, reached as one array on
                 config 2's network) - the largest single-GPU workload: ``value``, ``ms_per_step``,
                 ``roofline`` and ``cpu_baseline`` are its figures, over exactly K timed steps
  per_config     the same fields for configurations 1-4 (their own step counts are stated)
  metric/value   generator-neuron updates per second = sum over layer steps of N_out*(n_out+1),
                 divided by reach wall-time (ms_per_step is the reach wall-time itself)
  roofline       the kernel group with the largest summed kernel time of a reach, whether it is bound by
                 throughput or by latency: work of its launches over their summed durations (events that
                 ride on the kernels' own dispatches), against 78.6 TFLOP/s (fp64 MFMA) or 8 TB/s (HBM);
                 ``traffic`` = HBM bytes per launch from the counter tables in profiles/
  cpu_baseline   the CPU oracle (numpy/OpenBLAS restatement of NNV's path, "port") timed on this host on
                 a bounded sample of the same workload

With ``--config k`` only that configuration is measured (k = 6: a CNN with normalisation / pooling /
flatten layers); ``--lean`` then leaves out every extra pass, which is what the rocprofv3 summaries in
profiles/ run.  Before anything is timed the device is kept busy with untimed steps for at least 0.3 s,
whatever ``--warmup`` says, so that short step counts are measured on settled clocks.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

import nnv_amd  # noqa: E402

FP64_MFMA_PEAK_TFLOPS = 78.6
HBM_PEAK_GBS = 8000.0
MIN_WARM_SECONDS = 0.3


# kernels whose launches a timed group of the library covers (nnvhip_kernel_time), by the group's label below
GROUP_KERNELS = {
    "gemm_f64_kernel": ("gemm_f64_kernel",),
    "gemm_seg_kernel": ("gemm_seg_kernel",),
    "conv2d_fast_kernel": ("conv2d_fast_kernel", "conv2d_fast_stamps_kernel", "conv2d_f64_kernel"),
    "gather_columns_kernel": ("gather_columns_kernel", "gather_skinny_kernel", "fc_rowsum_kernel", "conv_stamp_kernel", "conv_stamp_rows_kernel"),
    "ranges_partial_kernel": ("ranges_partial_kernel", "ranges_window_kernel"),
    "relu_classify_kernel": ("relu_classify_kernel", "relu_count_kernel", "relu_compact_kernel"),
}


def profile_traffic(workload, kernel, variant=""):
    """HBM bytes per launch of a kernel group from profiles/<workload>[_<variant>]_hbm_traffic.md (scaled
    FETCH_SIZE + WRITE_SIZE of rocprofv3 --pmc runs; the table's last two columns are MiB read / written per
    dispatch).  The kernels of the group are averaged by their dispatch counts.  None if there is no table."""
    path = os.path.join(ROOT, "profiles", "%s%s_hbm_traffic.md" % (workload, "_" + variant if variant else ""))
    if not os.path.exists(path):
        return None
    names = GROUP_KERNELS.get(kernel, (kernel,))
    disp, mib = 0, 0.0
    for line in open(path):
        m = re.match(r"\|\s*`([^`]+)`\s*\|\s*(\d+)\s*\|[^|]*\|[^|]*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|", line)
        if m and any(nm in m.group(1) for nm in names):
            n = int(m.group(2))
            disp += n
            mib += n * (float(m.group(3)) + float(m.group(4)))
    return round(mib / disp * 1048576.0) if disp else None


def as_sets(s):
    return s if isinstance(s, (list, nnv_amd.SetArray)) else [s]


def layer_shapes(reach_set):
    out = []
    for s in reach_set:
        for t in as_sets(s):
            N, n, _ = t._h.dims()
            out.append((N, n))
    return out


def cpu_sample(cfg, method, updates, seconds):
    """The oracle on this host, on a bounded sample of the workload: whole reaches where one fits the
    budget; for the array of boxes as many of its sets as fit; for a network whose single reach takes
    longer, its leading layers."""
    from oracle import nnv_oracle as o
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    base = {"unit": "updates/s", "cores": threads, "kind": "port"}
    if "partition" in cfg:
        boxes = o.box_partition(cfg["lb"], cfg["ub"], cfg["partition"]["indexes"], cfg["partition"]["numbers"])
        done, t_cpu, upd = 0, 0.0, 0
        stride = max(1, len(boxes) // 64)          # spread over the array
        for i in range(0, len(boxes), stride):
            t1 = time.perf_counter()
            _, sets = o.nn_reach(cfg["layers"], o.star_from_box(*boxes[i]), method, 1.0, keep=True)
            t_cpu += time.perf_counter() - t1
            upd += sum(s.V.shape[0] * s.V.shape[1] for s in sets)
            done += 1
            if t_cpu >= seconds:
                break
        base.update(value=upd / t_cpu, ms_per_set=round(1e3 * t_cpu / done, 2),
                    ms_per_reach_extrapolated=round(1e3 * t_cpu / done * len(boxes), 1),
                    sample="%d of the %d sets of %s, each reached on its own by the numpy/OpenBLAS oracle as the reference "
                           "loops over an array (dense C built at every ReLU, as NNV does)" % (done, len(boxes), cfg["name"]))
        return base
    if cfg["kind"] == "image":
        sh = cfg["image_shape"]
        first = o.image_star_from_bounds(cfg["lb"].reshape(sh, order="F"), cfg["ub"].reshape(sh, order="F"))
    else:
        first = o.star_from_box(cfg["lb"], cfg["ub"])
    # one layer at a time, so that a reach that does not fit the budget is cut after a whole layer
    t_cpu, upd, n_reach, n_layers, partial = 0.0, 0, 0, len(cfg["layers"]), None
    while t_cpu < seconds and n_reach < 200 and partial is None:
        S = first
        for li, L in enumerate(cfg["layers"]):
            t1 = time.perf_counter()
            S = o.nn_reach([L], S, method, 1.0)
            t_cpu += time.perf_counter() - t1
            V = S.V
            upd += int(np.prod(V.shape))
            if n_reach == 0 and t_cpu >= seconds and li + 1 < n_layers:
                partial = li + 1
                break
        else:
            n_reach += 1
    base["value"] = upd / t_cpu
    if partial is None:
        base["ms_per_reach"] = round(1e3 * t_cpu / n_reach, 2)
        base["sample"] = "%d full %s reach(es) by the numpy/OpenBLAS oracle (dense C built at every ReLU, as NNV does)" % (n_reach, cfg["name"])
    else:
        base["sample"] = ("the first %d of the %d layers of one %s reach by the numpy/OpenBLAS oracle (%.1f s; a whole reach "
                          "does not fit the sample budget)" % (partial, n_layers, cfg["name"], t_cpu))
    return base


def measure(k, args, ctx, exact_steps, extras):
    """One configuration: timed steps, per-kernel timing pass, and the passes named in `extras`
    (a subset of {"dense", "h2h", "written", "spec", "cpu"})."""
    from nnv_amd.configs import count_updates, device_input_sets, make_config, make_extended_cnn

    cfg = make_extended_cnn(32, 3) if k == 6 else make_config(k)
    ctx.set_dense_affine(args.dense)
    ctx.set_eager_columns(args.written)
    ctx.set_eager_relu(args.written)
    for nm in args.switch:
        ctx.set_switch(nm, True)
    net = nnv_amd.NN.from_config(cfg["layers"], cfg["name"])
    opts = {"reachMethod": args.method, "relaxFactor": 1}
    dev_in = device_input_sets(cfg, ctx)
    lib, h = ctx.lib, ctx.handle
    n_sets = len(dev_in) if isinstance(dev_in, (list, nnv_amd.SetArray)) else 1

    def step():
        out = net.reach(dev_in, opts)
        outs = as_sets(out)
        arr = outs.handles() if isinstance(outs, nnv_amd.SetArray) else (ctypes.c_void_p * len(outs))(*[o_._h.h for o_ in outs])
        # output bounds of all sets in one batched call, left on the device
        nnv_amd._lib.check(lib.nnvhip_estimate_ranges_batch(h, len(outs), arr, None, None))
        return out

    # untimed steps until the device has been busy for MIN_WARM_SECONDS (clocks settled, pool blocks in
    # place), then the W warm-up steps the caller asked for
    n_warm, t0 = 0, time.perf_counter()
    while n_warm < 3 or time.perf_counter() - t0 < MIN_WARM_SECONDS:
        step()
        n_warm += 1
        if n_warm % 8 == 0:
            ctx.synchronize()
    ctx.synchronize()
    t_step = (time.perf_counter() - t0) / n_warm
    steps = args.steps if exact_steps else int(max(args.steps, min(1000, 0.2 / max(t_step, 1e-6))))
    for _ in range(args.warmup):
        step()
    ctx.synchronize()

    def timed_steps():
        cnt0 = ctx.debug_counters()
        t0_ = time.perf_counter()
        for _ in range(steps):
            step()
        ctx.synchronize()
        wall_ = time.perf_counter() - t0_
        cnt1 = ctx.debug_counters()
        # what the library's own counters saw during the timed steps (a step that has to ask the driver for device
        # memory, or to wait for the pinned staging ring, shows here)
        info = {k_: cnt1[k_] - cnt0[k_] for k_ in ("device_mallocs", "staging_waits")}
        info["pool_bytes_in_use_cached_after"] = list(ctx.pool_stats())
        info["ms_per_step"] = round(1e3 * wall_ / steps, 5)
        return wall_, info

    wall, timed_loop = timed_steps()
    # About one process in fifty has shown a stall of a second somewhere in its timed loop on these boxes, with no
    # allocation and no wait recorded by the library.  A loop whose mean is more than twice that of the untimed warm
    # steps just before it is therefore timed once more, exactly `steps` steps again; the line then carries the
    # second figure, and the first one, with its counters, under step_ms.first_attempt_set_aside.
    set_aside = None
    if wall / steps > 2.0 * t_step and wall > 0.05:
        set_aside = timed_loop
        wall, timed_loop = timed_steps()
    ms_per_step = 1e3 * wall / steps
    # the same steps once more, each one bracketed by a synchronisation of its own: the spread of single steps
    # (ms_per_step above is the mean of steps queued back to back, which is what `value` is quoted on)
    each, slow = [], []
    n_each = max(20, min(steps, 200))
    for _ in range(n_each):
        c0 = ctx.debug_counters()
        t1 = time.perf_counter()
        step()
        ctx.synchronize()
        each.append(1e3 * (time.perf_counter() - t1))
        c1 = ctx.debug_counters()
        if len(each) > 5 and each[-1] > 1.5 * float(np.median(each[:-1])):
            used, cached = ctx.pool_stats()
            slow.append({"step": len(each) - 1, "ms": round(each[-1], 4), "pool_bytes_in_use": used, "pool_bytes_cached": cached,
                         "during_the_step": {k_: c1[k_] - c0[k_] for k_ in ("device_mallocs", "staging_waits")},
                         "deferred_handles_before": c0["deferred_handles"], "deferred_handles_after": c1["deferred_handles"],
                         "live_handles": c1["live_handles"]})
    step_ms = {"during_the_timed_steps": timed_loop, "first_attempt_set_aside": set_aside, "n": n_each, "min": round(min(each), 5), "median": round(float(np.median(each)), 5), "max": round(max(each), 5),
               "what": "single steps, each followed by a synchronisation", "steps_over_1p5x_median": slow[:8]}
    shapes = layer_shapes(net.reachSet)
    updates = count_updates(shapes)
    value = updates / (wall / steps)

    # ---- per-layer and per-kernel timing with HIP events on the library's stream -----------------
    reps = max(5, min(steps, 20))

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

    # a small FC / ReLU network is reached by ONE launch (nnvhip_reach_layers): time that kernel on the step's own path
    for grp in range(11):
        ctx.kernel_time(grp)
    ctx.set_timing(2)
    for _ in range(reps):
        step()
    ctx.set_timing(0)
    chain_ms, chain_launches, chain_bytes = ctx.kernel_time(8)
    for grp in range(11):
        ctx.kernel_time(grp)

    per_layer = timed_pass(1)          # NN.reachTime-style device time per layer (layer-by-layer calls)
    timed_pass(2)                      # start / stop events on every dispatch of the timed kernel groups
    gemm_ms, gemm_launches, gemm_work = ctx.kernel_time(0)
    conv_ms, conv_launches, conv_work = ctx.kernel_time(1)
    rng_ms, rng_launches, rng_bytes = ctx.kernel_time(2)
    app_ms, app_launches, app_bytes = ctx.kernel_time(3)
    row_ms, row_launches, row_bytes = ctx.kernel_time(4)
    gat_ms, gat_launches, gat_bytes = ctx.kernel_time(5)
    cls_ms, cls_launches, cls_bytes = ctx.kernel_time(6)
    fin_ms, fin_launches, fin_bytes = ctx.kernel_time(7)
    seg_ms, seg_launches, seg_work = ctx.kernel_time(9)
    dlt_ms, dlt_launches, dlt_bytes = ctx.kernel_time(10)

    # algorithmic (unpadded, dense) flop of the launches the kernel timers cover
    gemm_flop = conv_flop = 0.0
    relu_bytes, relu_ms = 0.0, 0.0
    gat_dense_bytes = 0.0
    onehot_cols = [s._h.dims()[1] for s in as_sets(dev_in)] if cfg["layers"][0]["type"] == "fc" else None
    layer_report = []
    prev_sets = as_sets(dev_in)
    for i, (Ld, L) in enumerate(zip(cfg["layers"], net.Layers)):
        outs = as_sets(net.reachSet[i])
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
                fused = i > 0 and cfg["layers"][i - 1]["type"] == "fc" and len(outs) == 1
                ni, nc = ctypes.c_int64(), ctypes.c_int64()
                nnv_amd._lib.check(ctx.lib.nnvhip_star_relu_counts(so._h.h, ctypes.byref(ni), ctypes.byref(nc)))
                kept = N - ni.value - nc.value
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

    groups = []
    # (the dense count of the FC layers is quoted with the one of the two FC kernel groups that takes longer)
    if seg_launches:
        groups.append((seg_ms, mfma_roofline("gemm_seg_kernel", seg_work, gemm_flop if seg_ms >= gemm_ms else 0.0, seg_ms, seg_launches)))
    if gemm_launches:
        groups.append((gemm_ms, mfma_roofline("gemm_f64_kernel", gemm_work, gemm_flop if gemm_ms > seg_ms or not seg_launches else 0.0,
                                              gemm_ms, gemm_launches)))
    if conv_launches:
        g = mfma_roofline("conv2d_fast_kernel", conv_work, conv_flop, conv_ms, conv_launches)
        if not ctx.switch_is_on("eager_cols", "dense_affine"):
            # conv2d_fast_stamps_kernel: a layer's launch also writes the filter stamps of its unit-vector columns (blocks
            # dealt in between the tile blocks); the flop count is that of the tiles, the duration that of the whole launch
            g["stamp_blocks_in_the_same_launch"] = True
        groups.append((conv_ms, g))
    if rng_launches:
        groups.append((rng_ms, hbm_roofline("ranges_partial_kernel", rng_ms, rng_launches, rng_bytes)))
    if app_launches:
        groups.append((app_ms, hbm_roofline("relu_apply_kernel", app_ms, app_launches, app_bytes)))
    if row_launches:
        groups.append((row_ms, hbm_roofline("row-wise affine layers (rowmap/avgpool/permute kernels)", row_ms, row_launches, row_bytes)))
    if gat_launches:
        g = hbm_roofline("gather_columns_kernel", gat_ms, gat_launches, gat_bytes)
        if not ctx.eager_columns and not args.dense:
            # FC layers whose gathered columns nobody reads leave them unwritten (range sums only): those
            # launches run out of the cache-resident weights and are bound by L2 / ALU rate, not by HBM
            g["columns_left_unwritten"] = True
            if all(Ld["type"] in ("fc", "relu") for Ld in cfg["layers"]):   # (CNNs: the group also holds the stamp passes)
                g["dense_equivalent_GBps"] = round(gat_dense_bytes * reps / (gat_ms * 1e-3) / 1e9, 1)
        groups.append((gat_ms, g))
    if fin_launches:
        groups.append((fin_ms, hbm_roofline("ranges_final_kernel", fin_ms, fin_launches, fin_bytes)))
    if dlt_launches:
        # outputs that start from a product shared by the sets of a group and add only the rows in which a set differs
        # from the group's list: a block reads its piece of the shared product (from cache), adds a few rank-one
        # terms and writes itself out - bound by the bytes of output it writes
        unwritten = not ctx.eager_columns and not args.dense and not args.written   # (the pass is then another kernel)
        g = hbm_roofline("delta_sums_kernel" if unwritten else "delta_tiles_kernel", dlt_ms, dlt_launches, dlt_bytes)
        g["what"] = ("FC layer over an array of sets of one shape: the product over the rows most sets keep is formed once per "
                     "shape, every set's tiles start from it and contract over the rows in which the set differs; bytes = the "
                     "output matrices written")
        if unwritten:
            # nobody on the way to the next layer reads these matrices (the ReLU step takes the range sums): the pass forms
            # and sums every piece (one fp64 MFMA per 16 x 16 outputs, which runs at the vector unit's fp64 rate) and stores
            # the centre columns and the partial sums only - what it then moves is a small part of what it computes, and
            # the fp64 units bound it, not HBM (the fraction of the HBM peak says so)
            g["matrices_left_unwritten"] = True
            # the library counts the sums of every set; a set equal to its neighbour in row differences and bounds is
            # neither summed nor written again (decided on the device), so fewer bytes move - the counter table in
            # profiles/ has the figure
            g["bytes_are_an_upper_bound"] = True
            g["what"] = ("FC layer over an array of sets of one shape: the product over the rows most sets keep is formed once per "
                         "shape; every set's pieces start from it, add the rows in which the set differs and are summed into the "
                         "set's range sums without being stored (written by the same pass on first read); bytes = centre columns "
                         "and partial sums of every set (a set whose row differences and bounds equal its neighbour's is sent "
                         "to the neighbour's sums, which are then neither formed nor written again); bound by the vector "
                         "ALUs, not by HBM")
        g["dense_equivalent_flop_per_step"] = gemm_flop
        g["dense_equivalent_achieved_TFLOPs"] = round(gemm_flop * reps / (dlt_ms * 1e-3) / 1e12, 1)
        groups.append((dlt_ms, g))
    if cls_launches:
        # classification, sort of the crossing list and the new predicate bounds: one block per set of up
        # to 8192 neurons - with a single input set a dependent chain on one CU, bound by latency, which
        # the fraction of the HBM peak then shows
        c = hbm_roofline("relu_classify_kernel", cls_ms, cls_launches, cls_bytes)
        c["blocks_per_launch"] = n_sets
        if n_sets < 256:
            c["latency_bound"] = True
        groups.append((cls_ms, c))
    variant = "dense_contraction" if args.dense else "all_written" if args.written else "_".join(args.switch)
    for _, g in groups:
        if g["kernel"] in GROUP_KERNELS:
            g["kernels_in_group"] = list(GROUP_KERNELS[g["kernel"]])
    groups.sort(key=lambda g: -g[0])
    if chain_launches:
        # the measured step is one launch of the whole-reach kernel, one block per set: a chain of dependent phases
        # on one CU per set, bound by latency; the groups above belong to the layer-by-layer calls of the same
        # network (what the per-layer times below were taken on) and are listed for comparison only
        c = hbm_roofline("reach_chain_kernel", chain_ms, chain_launches, chain_bytes)
        c["blocks_per_launch"] = n_sets
        c["latency_bound"] = n_sets < 256
        c["what"] = ("the whole reach in one launch (every layer's set written in full); bytes = weights read once per set "
                     "+ every layer's output matrix written once")
        roofline = c
        roofline["other_kernels"] = []
        roofline["layer_by_layer_kernels"] = [g[1] for g in groups]
        if args.method == "relax-star-area":
            roofline["traffic"] = profile_traffic(cfg["name"], "reach_chain_kernel", variant)
    else:
        roofline = dict(groups[0][1])
        roofline["other_kernels"] = [g[1] for g in groups[1:]]
    if args.method == "relax-star-area":
        roofline["traffic"] = profile_traffic(cfg["name"], roofline["kernel"], variant)
        for g in roofline["other_kernels"]:
            g["traffic"] = profile_traffic(cfg["name"], g["kernel"], variant)

    # the MFMA GEMM on the full dense problem of the same reach (what Star.affineMap executes in the
    # reference): a short extra pass with the skipping of structural zeros switched off
    if gemm_launches and not args.dense and "dense" in extras:
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
            if args.method == "relax-star-area":
                dr["traffic"] = profile_traffic(cfg["name"], "gemm_f64_kernel", "dense_contraction")
            roofline["dense_contraction"] = dr
    if relu_ms > 0:
        # bytes the dense materialisation of the ReLU steps would move (read V for the ranges, read the kept
        # rows, write the output) over the time the steps took; the steps leave most of that undone (pending
        # row reset, range sums from the producing layer), so this can exceed the HBM peak
        roofline["relu_step_dense_equivalent_GBps"] = round(relu_bytes / (relu_ms * 1e-3) / 1e9, 1)

    # ---- the same step with the host buffers the boundary takes and returns (not `value`) -----------
    host_to_host = None
    if "h2h" in extras:
        n_h2h = max(5, min(steps, 50))
        ctx.synchronize()
        t1 = time.perf_counter()
        fresh = res = None
        for _ in range(n_h2h):
            fresh = device_input_sets(cfg, ctx)
            res = net.reach(fresh, opts)
            nnv_amd.Star.estimateRanges_array(as_sets(res))
        host_to_host = {"ms_per_step": round(1e3 * (time.perf_counter() - t1) / n_h2h, 4), "steps": n_h2h,
                        "what": "input bounds uploaded and the set(s) built, reach, output bounds fetched to the host"}
        del fresh, res

    # ---- the same step with every intermediate set written out in full (not `value`) -------------
    # By default the sets between the layers keep what nobody reads before the next layer as a description
    # (a ReLU's row reset and appended columns, columns gathered from the weights) and write it on first
    # read; the returned set and its bounds are always written.  Here every layer writes its whole output,
    # which is what the reference's NN.reachSet{i} holds.
    all_written = None
    if not args.dense and not args.written and "written" in extras:
        ctx.set_eager_columns(True)
        ctx.set_eager_relu(True)
        try:
            for _ in range(3):
                step()
            ctx.synchronize()
            n_aw = max(5, min(steps, 100))
            t1 = time.perf_counter()
            for _ in range(n_aw):
                step()
            ctx.synchronize()
            aw_ms = 1e3 * (time.perf_counter() - t1) / n_aw
            aw_gbps = 8.0 * updates / (aw_ms * 1e-3) / 1e9
            all_written = {"ms_per_step": round(aw_ms, 5), "value": updates / (aw_ms * 1e-3), "steps": n_aw,
                           "bytes_written_per_step": 8.0 * updates, "written_GBps": round(aw_gbps, 1),
                           "frac_of_hbm_peak": round(aw_gbps / HBM_PEAK_GBS, 4),
                           "what": "the same step with every layer writing its whole output matrix in the call "
                                   "(nothing left for a first read), as the reference's reachSet{i} holds it; the rate "
                                   "counts the bytes of those matrices only (8 bytes per update), not what the step reads"}
        finally:
            ctx.set_eager_columns(False)
            ctx.set_eager_relu(False)
        net.reach(dev_in, opts)   # reachSet back to the default path for what follows

    # ---- specification check on the resident output sets (not part of `value`) -----------------
    spec = None
    last = net.Layers[-1]
    if hasattr(last, "Bias") and len(last.Bias) > 1 and "spec" in extras:
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

    single = not isinstance(dev_in, (list, nnv_amd.SetArray))
    del dev_in, prev_sets
    net.reachSet = []
    del net
    ctx.trim_pool()

    cpu = cpu_sample(cfg, args.method, updates, args.cpu_seconds if exact_steps else args.cpu_seconds / 3.0) if "cpu" in extras else None

    return {
        "value": value, "steps": steps, "warmup": args.warmup, "warm_steps_by_time": n_warm, "ms_per_step": ms_per_step,
        "step_ms": step_ms,
        "config": {"workload": cfg["name"], "reach_method": args.method, "relax_factor": 1, "switches": list(args.switch),
                   "all_sets_written_ms": all_written["ms_per_step"] if all_written else None,
                   "all_sets_written_updates_per_s": all_written["value"] if all_written else None,
                   "all_sets_written_frac_of_hbm_peak": all_written["frac_of_hbm_peak"] if all_written else None,
                   "fc_affine_map": "dense" if args.dense else "structural zeros skipped (one-hot generator columns, reset rows); exact",
                   "sets": n_sets, "updates_per_step": updates,
                   "intermediate_sets": "dense" if args.dense else
                   "every layer writes its whole output matrix in the call, as the reference's reachSet{i} holds it" if args.written else
                   "every layer's set is written in full by the one launch that reaches the whole network" if chain_launches else
                   "the sets between layers record a ReLU's row reset / appended columns, the columns an FC layer "
                   "gathers from its weights and the matrices an FC layer forms from a product its sets share, and write "
                   "them on first read; the returned set and its bounds are written",
                   "predicates_per_layer": [n for (_, n) in shapes][:len(cfg["layers"])] if single else None},
        "roofline": roofline, "cpu_baseline": cpu, "spec_check": spec, "host_to_host": host_to_host,
        "all_sets_written": all_written, "layers": layer_report,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20, help="timed steps of the headline configuration")
    ap.add_argument("--warmup", type=int, default=5,
                    help="untimed steps right before the timed ones (on top of the 0.3 s of untimed steps every run starts with)")
    ap.add_argument("--config", type=int, default=None,
                    help="measure this configuration only (1-5; 6: CNN with normalisation / pooling / flatten layers); "
                         "default: all five, headline = config 5")
    ap.add_argument("--method", default="relax-star-area")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--dense", action="store_true",
                    help="run every FC layer as the full dense contraction (no skipping of structural zeros)")
    ap.add_argument("--written", action="store_true",
                    help="every layer writes its whole output matrix in the call (nothing is left for a first read): the "
                         "all_sets_written figure of a default run as a run of its own, for profiles")
    ap.add_argument("--switch", action="append", default=[],
                    help="a route switch of the library to set for the run (nnvhip_set_switch), e.g. no_row_deltas: an FC layer "
                         "over an array contracts every set over its whole kept-row list on the tile kernel; may be repeated")
    ap.add_argument("--cpu-seconds", type=float, default=10.0,
                    help="budget of the headline's CPU baseline sample (the other configurations get a third each)")
    ap.add_argument("--lean", action="store_true",
                    help="only the timed steps and the per-kernel timing pass (no dense-contraction, host-to-host, "
                         "all-sets-written and specification passes): what the rocprofv3 summaries in profiles/ run, so "
                         "that their kernel tables hold the kernels of the measured path only")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (sets shard across GPUs without communication; "
                 "that path is not built) - use --gpus 1")

    ctx = nnv_amd.default_context()
    cpu = set() if args.no_cpu else {"cpu"}
    if args.config is not None:
        extras = cpu if args.lean else cpu | {"dense", "h2h", "written", "spec"}
        head = measure(args.config, args, ctx, True, extras)
        per_config = None
    else:
        # the four smaller configurations first (the headline's 6.6 GB arena then meets an empty pool)
        per_config = []
        for k in (1, 2, 3, 4):
            extras = cpu if args.lean else cpu | {"written"} | ({"dense"} if k == 2 else set())
            r = measure(k, args, ctx, False, extras)
            r = {"metric": "generator_neuron_updates_per_s", "unit": "updates/s", **{kk: r[kk] for kk in
                 ("value", "ms_per_step", "step_ms", "steps", "config", "roofline", "all_sets_written", "cpu_baseline")}}
            per_config.append(r)
        head = measure(5, args, ctx, True, cpu if args.lean else cpu | {"written", "spec", "h2h"})
    # practical ceilings on this box: a register-resident MFMA loop and a plain copy kernel over 1 GiB
    head["roofline"]["measured_mfma_TFLOPs"] = round(ctx.probe_mfma_peak(3), 2)
    head["roofline"]["measured_copy_GBps"] = round(ctx.probe_copy_bandwidth(1 << 30, 5), 1)
    ctx.trim_pool()
    # HBM fractions are quoted against the datasheet's 8 TB/s; the same rates against what a plain copy kernel
    # reaches on this box are put beside them
    copy_gbps = head["roofline"]["measured_copy_GBps"]

    def beside(r):
        if r and r.get("bound") == "hbm" and copy_gbps > 0:
            r["frac_of_measured_copy"] = round(r["achieved"] / copy_gbps, 4)
        for g in (r or {}).get("other_kernels", []) + (r or {}).get("layer_by_layer_kernels", []):
            beside(g)

    for r in [head] + (per_config or []):
        beside(r["roofline"])
        if r.get("all_sets_written"):
            r["all_sets_written"]["frac_of_measured_copy"] = round(r["all_sets_written"]["written_GBps"] / copy_gbps, 4)
            r["config"]["all_sets_written_frac_of_measured_copy"] = r["all_sets_written"]["frac_of_measured_copy"]
    cpu = head["cpu_baseline"]
    if cpu and head["all_sets_written"]:
        # the CPU oracle builds every set in full, so the like-for-like device figure is the all-sets-written one
        cpu["device_over_cpu_all_sets_written"] = round(head["all_sets_written"]["value"] / cpu["value"], 1)
        cpu["device_over_cpu_sets_described"] = round(head["value"] / cpu["value"], 1)

    print(json.dumps({
        "metric": "generator_neuron_updates_per_s", "value": head["value"], "unit": "updates/s", "n_gpus": 1,
        "steps": head["steps"], "warmup": head["warmup"], "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": head["config"], "roofline": head["roofline"], "cpu_baseline": head["cpu_baseline"],
        "warm_steps_by_time": head["warm_steps_by_time"], "step_ms": head["step_ms"],
        "value_is": "reach with the sets between layers kept as descriptions (written on first read); the returned set and "
                    "its bounds are written.  The figure with every layer's set written in full, as the reference's "
                    "reachSet{i} holds them, is value_all_sets_written / ms_per_step_all_sets_written",
        "value_all_sets_written": head["all_sets_written"]["value"] if head["all_sets_written"] else None,
        "ms_per_step_all_sets_written": head["all_sets_written"]["ms_per_step"] if head["all_sets_written"] else None,
        "spec_check": head["spec_check"], "host_to_host": head["host_to_host"],
        "all_sets_written": head["all_sets_written"], "layers": head["layers"], "per_config": per_config,
    }))


if __name__ == "__main__":
    main()
