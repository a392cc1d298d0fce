#!/usr/bin/env python3
"""Benchmark of the GCN aggregation path on one MI355X.

A step is one epoch's worth of aggregation for the 2-layer GCN of the reference's driver
(hidden 16, 22 classes): forward aggregation at width 16 and 22, pruned backward aggregation
at width 22 (last layer) and 16 (first layer), launched back to back through the C ABI with
every input resident in HBM.  The dense X*W products are not part of the metric.

Prints ONE JSON line:  metric = the headline metric below, value = algorithmic GB/s of the epoch's
aggregation, ms_per_step = aggregation ms per epoch, plus `roofline` for the dominant kernel
(HIP-event time of the kernel alone) and `cpu_baseline` (the CPU checker's OpenMP restatement
timed on the host cores on one epoch of the same workload).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
METRIC = "fwd+bwd aggregation ms/epoch and achieved HBM GB/s (% peak), 1 MI355X"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="cfg4_rmat22",
                    help="cfg1_uniform, cfg2_chunglu, cfg3_rmat20, cfg4_rmat22 (the metric's configuration), or "
                         "rmat:<scale>:<pairs per vertex> for an R-MAT graph of another size")
    ap.add_argument("--train_ratio", type=float, default=0.1)
    ap.add_argument("--backsize_mode", default="constant", choices=["constant", "map", "threshold", "wave64"])
    ap.add_argument("--backsize", type=int, default=32)
    ap.add_argument("--part_size", type=int, default=0, help="forward group size (0 = int(avg degree))")
    ap.add_argument("--team", type=int, default=0, help="force lanes per group (0 = automatic)")
    ap.add_argument("--rounds", type=int, default=0, help="force group rounds per wave (0 = automatic)")
    ap.add_argument("--plan_shift", type=int, default=0, help="force log2 of the plan's column block")
    ap.add_argument("--plan_keep", type=int, default=-1, help="rows with at most this many groups stay together")
    ap.add_argument("--force_plan", action="store_true", help="use execution plans even for small feature tables")
    ap.add_argument("--no_length_classes", action="store_true", help="plans without the length-class key")
    ap.add_argument("--stepwise_prep", action="store_true",
                    help="prepare the backward paths with the reference's separate marking and compaction steps")
    ap.add_argument("--no_plan", action="store_true",
                    help="process the groups in CSR order instead of the column-blocked execution plan")
    ap.add_argument("--no_workspace", action="store_true",
                    help="aggregate without the feature workspace (per-edge scale gather, no scratch)")
    ap.add_argument("--no_cpu_baseline", action="store_true")
    ap.add_argument("--no_train", action="store_true", help="skip the 100-epoch training timing")
    ap.add_argument("--train_epochs", type=int, default=100)
    ap.add_argument("--copy_probe", action="store_true",
                    help="also launch a plain 1 GiB device copy 3 times (calibrates byte counters under rocprofv3)")
    ap.add_argument("--verbose", action="store_true")
    return ap.parse_args()


def log(args, *a):
    if args.verbose:
        print(*a, file=sys.stderr, flush=True)


def _event_ms(fn, reps):
    import torch
    for _ in range(2):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def pipeline_figures(g, wl, kernels, x16, x22, out16, out22, args):
    from eppgcn_amd import capi, graphs
    n, dev = g.num_nodes, x16.device
    reps = max(3, min(args.steps, 10))
    w0 = graphs.uniform_weights(3, 96, 16).to(dev)
    w1 = graphs.uniform_weights(4, 16, 22).to(dev)
    x96 = graphs.normal32(1, (n, 96), dev, 5)
    t16 = capi.update_forward(x96, w0, scale=g.degrees, ld_out=capi.feature_workspace_pitch(16))
    t22 = capi.update_forward(x16, w1, scale=g.degrees, relu_input=True, ld_out=capi.feature_workspace_pitch(22))

    def fwd16():
        capi.spmm_forward(None, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                          g.row_pointers, out16, workspace=t16.view(-1), plan=wl.plans.get(16), prescaled_dim=16)

    def fwd22():
        capi.spmm_forward(None, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 16, 8,
                          g.row_pointers, out22, workspace=t22.view(-1), plan=wl.plans.get(22), prescaled_dim=22)

    def step():
        fwd16(); fwd22(); kernels[2][1](); kernels[3][1]()

    fig = {"agg_ms_per_epoch_forward_prescaled": round(_event_ms(step, reps), 4)}
    f32 = 4
    dense = [
        ("x96_w0_scaled_table", lambda: capi.update_forward(x96, w0, scale=g.degrees, ld_out=16, out=t16),
         n * (96 + 16 + 1) * f32),
        ("relu_y1_w1_scaled_table", lambda: capi.update_forward(x16, w1, scale=g.degrees, relu_input=True, ld_out=32,
                                                                out=t22), n * (16 + 32 + 1) * f32),
        ("g1_w1t_relu_masked", lambda: capi.update_backward_input(x22, w1, relu_ref=x16), n * (22 + 16 + 16) * f32),
        ("x96t_g0_weight_grad", lambda: capi.update_backward_weight(x96, x16), n * (96 + 16) * f32),
        ("relu_y1t_g1_weight_grad", lambda: capi.update_backward_weight(x16, x22, relu_input=True), n * (16 + 22) * f32),
    ]
    fig["dense_update"] = {}
    for name, fn, nbytes in dense:
        ms = _event_ms(fn, reps)
        fig["dense_update"][name] = {"ms": round(ms, 4), "alg_bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                                     "pct_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS * 100, 2)}
    return fig


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (no multi-GPU path exists).",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from eppgcn_amd import capi, graphs, workload

    capi.load()                      # fails loudly when the HIP library is missing
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs the MI355X (no CPU fallback exists)")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    t0 = time.perf_counter()
    g = graphs.make_graph(args.config, device=dev)
    torch.cuda.synchronize()
    log(args, "graph", g.stats(), f"{time.perf_counter() - t0:.1f}s")
    if args.plan_shift:
        capi.set_plan_shift(args.plan_shift)
    if args.no_length_classes:
        capi.set_plan_length_classes(False)
    if args.plan_keep >= 0:
        capi.set_plan_keep_rows(args.plan_keep)
    t0 = time.perf_counter()
    wl = workload.prepare(g, 2, args.train_ratio, 2, args.part_size or None, args.backsize_mode, args.backsize,
                          plan=False if args.no_plan else (True if args.force_plan else None),
                          fused=not args.stepwise_prep)
    torch.cuda.synchronize()
    prep_s = time.perf_counter() - t0
    n, e = g.num_nodes, g.num_edges
    dims = (16, 22)                  # aggregation widths of layer 0 and layer 1 (hidden, classes)

    # synthetic inputs of the real shapes: projected features, and gradients that are
    # zero outside the rows the corresponding mask allows (what autograd would deliver)
    x16 = graphs.normal32(1, (n, 16), dev, 0)
    x22 = graphs.normal32(1, (n, 22), dev, 1)
    dy22 = graphs.normal32(1, (n, 22), dev, 2) * wl.train_mask[:, None]
    dy16 = graphs.normal32(1, (n, 16), dev, 3) * wl.ngh_masks[0][:, None]
    out16, out22 = torch.empty_like(x16), torch.empty_like(x22)
    ws16, ws22 = ((capi.feature_workspace(n, 16, dev), capi.feature_workspace(n, 22, dev))
                  if not args.no_workspace else (None, None))
    p_last, p_first = wl.paths[1], wl.paths[0]
    if args.team:
        capi.set_team_size(args.team)
    if args.rounds:
        capi.set_rounds(args.rounds)

    def fwd16():
        capi.spmm_forward(x16, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                          g.row_pointers, out16, workspace=ws16, plan=wl.plans.get(16))

    def fwd22():
        capi.spmm_forward(x22, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 16, 8,
                          g.row_pointers, out22, workspace=ws22, plan=wl.plans.get(22))

    def bwd22():
        capi.ours_backward(dy22, p_last.ids, p_last.part_pointer, p_last.edge_list, g.degrees, p_last.num_parts,
                           p_last.part_size, 2, 4, 16, out22, workspace=ws22, plan=p_last.plan,
                           gathered_rows=p_last.gathered_rows)

    def bwd16():
        capi.ours_backward(dy16, p_first.ids, p_first.part_pointer, p_first.edge_list, g.degrees,
                           p_first.num_parts, p_first.part_size, 1, 4, 16, out16, workspace=ws16,
                           plan=p_first.plan, gathered_rows=p_first.gathered_rows)

    kernels = [
        ("fwd_agg_d16", fwd16, workload.bytes_forward(n, e, 16)),
        ("fwd_agg_d22", fwd22, workload.bytes_forward(n, e, 22)),
        ("bwd_agg_d22_last", bwd22, workload.bytes_pruned_backward(n, p_last.valid_len, p_last.num_parts, 22)),
        ("bwd_agg_d16_first", bwd16, workload.bytes_pruned_backward(n, p_first.valid_len, p_first.num_parts, 16)),
    ]
    bytes_epoch = sum(k[2] for k in kernels)

    def step():
        for _, fn, _ in kernels:
            fn()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = bytes_epoch / (ms_per_step * 1e-3) / 1e9

    # per-kernel time: the library's own HIP events on the launch stream, around the
    # aggregation kernel alone (the output clear is outside the bracket)
    capi.set_timing(True)
    per_kernel = {}
    reps = max(3, min(args.steps, 10))
    for name, fn, nbytes in kernels:
        which = 0 if name.startswith("fwd") else 1
        capi.clear_time()
        for _ in range(reps):
            fn()
        ms = capi.get_time_ms(which) / reps
        per_kernel[name] = {"ms": round(ms, 4), "alg_bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                            "pct_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS * 100, 2)}
    capi.set_timing(False)
    capi.clear_time()
    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    dominant = max(per_kernel, key=lambda k: per_kernel[k]["ms"])
    dk = per_kernel[dominant]
    roofline = {"bound": "hbm", "kernel": dominant, "achieved": dk["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(dk["GBps"] / PEAK_HBM_GBS, 4), "traffic": measured_traffic(args.config, dominant),
                "kernel_ms": dk["ms"], "alg_bytes_per_launch": dk["alg_bytes"]}

    result = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.config, "N": n, "E": e, "train_ratio": args.train_ratio,
                   "agg_widths": list(dims), "forward_group_size": wl.part_size,
                   "forward_groups": wl.num_parts, "backsize_mode": args.backsize_mode,
                   "backward_group_size": [p.part_size for p in wl.paths],
                   "kept_edges": [p.valid_len for p in wl.paths],
                   "backward_groups": [p.num_parts for p in wl.paths], "max_degree": g.stats()["max_degree"],
                   "feature_workspace": not args.no_workspace,
                   "column_blocked_plan": bool(wl.plans)},
        "agg_ms_per_epoch": round(ms_per_step, 4), "alg_bytes_per_epoch": bytes_epoch,
        "pct_of_peak_hbm": round(value / PEAK_HBM_GBS * 100, 2),
        "per_kernel": per_kernel, "path_preparation_s": round(prep_s, 3),
        "roofline": roofline,
    }

    # the same epoch as the training pipeline issues it: the forward tables arrive scaled and padded
    # from the dense update (built outside the timed region here), so only the backward launches
    # scale their input; and the dense update kernels themselves
    if not args.no_workspace:
        result["pipeline"] = pipeline_figures(g, wl, kernels, x16, x22, out16, out22, args)

    if not args.no_train:
        try:
            from eppgcn_amd import train
            result["train"] = train.time_gpu_training(g, wl, epochs=args.train_epochs, warmup=10)
        except Exception as exc:  # the training leg must never hide the kernel figures
            result["train"] = {"error": repr(exc)}

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args, g, wl, x16, x22, dy22, dy16, bytes_epoch)
        if not args.no_train and "error" not in result.get("train", {"error": 1}):
            try:
                from eppgcn_amd import train
                result["cpu_torch_sparse"] = train.time_cpu_sparse_training(g, wl.train_mask, epochs=args.train_epochs)
            except Exception as exc:
                result["cpu_torch_sparse"] = {"error": repr(exc)}
    print(json.dumps(result), flush=True)


def measured_traffic(config, kernel):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 counter summary (FETCH_SIZE +
    WRITE_SIZE of the same bench command), or None when no summary covers this workload."""
    import glob
    import re
    for path in glob.glob(os.path.join(ROOT, "profiles", "*.md")):
        m = re.search(r"traffic_bytes %s %s = ([0-9.e+]+)" % (re.escape(config), re.escape(kernel)),
                      open(path).read())
        if m:
            return float(m.group(1))
    return None


def cpu_baseline(args, g, wl, x16, x22, dy22, dy16, bytes_epoch):
    """The CPU checker's OpenMP restatement of the same four aggregations, one epoch, on the
    host cores.  A reported baseline, not a target."""
    from oracle import c_oracle as co
    co.load()
    col = g.column_index.cpu().numpy()
    s = g.degrees.cpu().numpy()
    pp, p2n = wl.part_ptr.cpu().numpy(), wl.part2node.cpu().numpy()
    n = g.num_nodes
    host = {k: v.cpu().numpy() for k, v in (("x16", x16), ("x22", x22), ("dy22", dy22), ("dy16", dy16))}
    paths = [(p.ids.cpu().numpy(), p.part_pointer.cpu().numpy(), p.edge_list.cpu().numpy(), p.num_parts)
             for p in wl.paths]
    def epoch():
        co.spmm_groups(host["x16"], col, s, pp, p2n, n, threads=True)
        co.spmm_groups(host["x22"], col, s, pp, p2n, n, threads=True)
        ids, bpp, el, npb = paths[1]
        co.ours_backward(host["dy22"], ids, bpp, el, s, npb, threads=True)
        ids, bpp, el, npb = paths[0]
        co.ours_backward(host["dy16"], ids, bpp, el, s, npb, threads=True)

    # bounded sample: whole epochs for about 10 s (at least 1 after a first, untimed one; at most 12)
    epoch()
    done, t0 = 0, time.perf_counter()
    while done < 12 and (done == 0 or time.perf_counter() - t0 < 10.0):
        epoch()
        done += 1
    dt = (time.perf_counter() - t0) / done
    return {"value": round(bytes_epoch / dt / 1e9, 2), "unit": "GB/s", "cores": co.num_threads(), "kind": "port",
            "ms_per_epoch": round(dt * 1e3, 1),
            "sample": f"mean of {done} whole epochs (4 aggregations each) of {args.config} after one untimed epoch, "
                      f"OpenMP C restatement, {co.num_threads()} threads of {os.cpu_count()} host cpus"}


if __name__ == "__main__":
    main()
