#!/usr/bin/env python3
"""Benchmark of the GCN aggregation path on one MI355X.

A step is one epoch's worth of aggregation for the 2-layer GCN of the reference's driver
(hidden 16, 22 classes): forward aggregation at width 16 and 22, pruned backward aggregation
at width 22 (last layer) and 16 (first layer), launched back to back through the C ABI with
every input resident in HBM.  The dense X*W products are not part of the metric.

Prints ONE JSON line:  metric = the headline metric below, value = algorithmic GB/s of the epoch's
aggregation (gather-model bytes / time: every walked edge is priced as if its row came from HBM, so
cache reuse shows up as a figure above what the memory system physically moved), ms_per_step =
aggregation ms per epoch, plus `roofline` for the dominant launch and `cpu_baseline` (the CPU
checker's OpenMP restatement timed on the host cores on one epoch of the same workload).

`roofline` prices the dominant *call*: output clear + pre-scaling pass + aggregation kernels, i.e. all
the work its algorithmic bytes are charged for, timed with HIP events on the launch stream
(`call_ms`; the parts are also timed apart by the library's own events).  `achieved` / `frac` are the
contract's figure: algorithmic (gather-model) bytes over the call time - a cache-amplified figure that
can pass 1.0 (`frac_basis` says so).  The physical, bounded figure is `hbm_frac`: the L2-miss
(fabric-side) traffic of the same call - TCC->EA read and write requests times their sizes, from the
committed rocprofv3 summary under profiles/, no fitted factor, used only while the kernel sources still
hash to what was profiled - over the same time; those counters sit between L2 and the fabric and cannot
tell the memory-side cache from HBM.  By default the same counters are also read live, before anything else
touches the GPU: two `rocprofv3 --pmc` child runs of this script's `--traffic_probe` mode (the four calls of a step,
three times each; about 20 s per run); where that works `roofline.traffic` is the live figure and the committed
summary is the cross-check (`traffic_committed`), where it does not (no rocprofv3, a time-out, this process itself
running under a profiler) the committed figure is used and `traffic_source` says so.  `kernel_only_frac` is the
aggregation kernels alone, `compulsory_frac` the lower bound with perfect reuse.
Before anything is timed every launch is checked against the same operator without plan and
workspace (different kernel instantiation, different summation order).
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
    ap.add_argument("--length_classes", action="store_true",
                    help="plans with the length-class key (the group kernel's optimum; off by default)")
    ap.add_argument("--fused_prep", action="store_true",
                    help="prepare the backward paths with the one-pass marking + compaction instead of the "
                         "reference's separate steps (same results, same time, no edge masks)")
    ap.add_argument("--no_plan", action="store_true",
                    help="process the groups in CSR order instead of the column-blocked execution plan")
    ap.add_argument("--no_stream", action="store_true",
                    help="keep planned launches on the group kernel instead of the plan's stream form")
    ap.add_argument("--degree_order", action="store_true",
                    help="renumber the vertices of the synthetic graph by descending degree inside blocks of 2^17 ids "
                         "before anything else (graphs.degree_order: what a caller who may choose its numbering gains; "
                         "NOT the benchmark's graph numbering, so not a headline figure - config.degree_order says so)")
    ap.add_argument("--wide_stream", action="store_true",
                    help="force the stream kernel's 64-bit addressing variant (it otherwise runs for tables of 4 GB and more)")
    ap.add_argument("--no_workspace", action="store_true",
                    help="aggregate without the feature workspace (per-edge scale gather, no scratch)")
    ap.add_argument("--no_cpu_baseline", action="store_true")
    ap.add_argument("--no_train", action="store_true", help="skip the 100-epoch training timing")
    ap.add_argument("--train_epochs", type=int, default=100)
    ap.add_argument("--copy_probe", action="store_true",
                    help="also launch a plain 1 GiB device copy 3 times (calibrates byte counters under rocprofv3)")
    ap.add_argument("--gather_probe", action="store_true",
                    help="also run the aggregation kernel 3 times each over permutation graphs with 64- and 128-byte "
                         "rows: every row of a 2^22-row table is gathered exactly once, so the bytes read are known "
                         "(calibrates FETCH_SIZE for row gathers under rocprofv3)")
    ap.add_argument("--no_check", action="store_true", help="skip the result check of the timed launches")
    ap.add_argument("--hip_graph", action="store_true",
                    help="also time the step replayed from a HIP graph of its four calls (removes the launch gaps that "
                         "matter on small graphs; reported as graph_ms_per_step, the headline value stays the eager step)")
    ap.add_argument("--no_live_traffic", action="store_true",
                    help="do not start the two rocprofv3 --pmc child runs that measure the calls' L2-miss traffic; "
                         "roofline.traffic then comes from the committed summary under profiles/")
    ap.add_argument("--traffic_probe", action="store_true",
                    help="(what the rocprofv3 child runs execute) set the workload up, issue the four calls of a step "
                         "three times each in a fixed order, print nothing, time nothing")
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
    t16 = capi.update_forward_table(x96, w0, g.degrees, plan=wl.plans.get(16))
    t22 = capi.update_forward_table(x16, w1, g.degrees, relu_input=True, plan=wl.plans.get(22))

    def fwd16():
        capi.spmm_forward(None, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                          g.row_pointers, out16, workspace=t16, plan=wl.plans.get(16), prescaled_dim=16)

    def fwd22():
        capi.spmm_forward(None, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 16, 8,
                          g.row_pointers, out22, workspace=t22, plan=wl.plans.get(22), prescaled_dim=22)

    def step():
        fwd16(); fwd22(); kernels[2][1](); kernels[3][1]()

    fig = {"agg_ms_per_epoch_forward_prescaled": round(_event_ms(step, reps), 4)}
    f32 = 4
    dense = [
        ("x96_w0_scaled_table", lambda: capi.update_forward_table(x96, w0, g.degrees, table=t16),
         n * (96 + 16 + 1) * f32),
        ("relu_y1_w1_scaled_table", lambda: capi.update_forward_table(x16, w1, g.degrees, relu_input=True, table=t22),
         n * (16 + 32 + 1) * f32),
        ("g1_w1t_relu_masked", lambda: capi.update_backward_input(x22, w1, relu_ref=x16), n * (22 + 16 + 16) * f32),
        ("x96t_g0_weight_grad", lambda: capi.update_backward_weight(x96, x16), n * (96 + 16) * f32),
        ("relu_y1t_g1_weight_grad", lambda: capi.update_backward_weight(x16, x22, relu_input=True), n * (16 + 22) * f32),
        # the two products above in one pass over G1 and Y1 (what the extension module's backward calls)
        ("hidden_layer_backward_pair", lambda: capi.update_backward(x16, w1, x22, relu_input=True),
         n * (22 + 16 + 16) * f32),
    ]
    fig["dense_update"] = {}
    for name, fn, nbytes in dense:
        ms = _event_ms(fn, reps)
        fig["dense_update"][name] = {"ms": round(ms, 4), "alg_bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1),
                                     "pct_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS * 100, 2)}
    return fig


# ---------------------------------------------------------------- live L2-miss traffic of the calls
CALL_ORDER = ("fwd_agg_d16", "fwd_agg_d22", "bwd_agg_d22_last", "bwd_agg_d16_first")
PROBE_REPS = 3
PMC_PASSES = (("TCC_EA0_RDREQ_sum", "TCC_EA0_RDREQ_32B_sum", "TCC_EA0_RDREQ_64B_sum", "TCC_EA0_RDREQ_128B_sum"),
              ("TCC_EA0_WRREQ_sum", "TCC_EA0_WRREQ_64B_sum"))
# kernels of a call before its stream kernel: output clear for rows without slots, pre-scaling pass
CALL_PROLOGUE = ("zero_words_kernel", "zero_listed_rows_kernel", "zero_rows_unless_kernel", "scale_rows", "scale_listed_rows_kernel")


def _short_kernel_name(name):
    return name.replace("void ", "").replace("eppgcn::", "").split("(")[0]


def call_bytes_from_counters(csv_path, bytes_of):
    """{call name: average of bytes_of(counters) per call} from one rocprofv3 counter_collection CSV of a
    `--traffic_probe` run.  The probe issues the four calls in CALL_ORDER, PROBE_REPS times, and nothing else runs
    a stream kernel, so the k-th stream-kernel dispatch belongs to call k mod 4; a call is that dispatch, the (at
    most two) clear / pre-scaling dispatches right before it and the fix-up dispatch right after it."""
    import csv
    disp = {}
    with open(csv_path, newline="") as f:
        for r in csv.DictReader(f):
            d = disp.setdefault(int(r["Dispatch_Id"]), [_short_kernel_name(r["Kernel_Name"]), {}])
            d[1][r["Counter_Name"]] = d[1].get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    seq = [disp[k] for k in sorted(disp)]
    at = [i for i, (name, _) in enumerate(seq) if name.startswith("aggregate_stream_kernel")]
    if len(at) != len(CALL_ORDER) * PROBE_REPS:
        raise RuntimeError(f"{len(at)} stream-kernel dispatches in the probe run, expected {len(CALL_ORDER) * PROBE_REPS}")
    total = {name: 0.0 for name in CALL_ORDER}
    for k, i in enumerate(at):
        members = [i]
        j = i - 1
        while j >= 0 and i - j <= 2 and seq[j][0].startswith(CALL_PROLOGUE):
            members.append(j)
            j -= 1
        if i + 1 < len(seq) and seq[i + 1][0].startswith("stream_fixup_kernel"):
            members.append(i + 1)
        total[CALL_ORDER[k % len(CALL_ORDER)]] += sum(bytes_of(seq[m][1]) for m in members)
    return {name: v / PROBE_REPS for name, v in total.items()}


def live_traffic(timeout_s=240):
    """({call name: L2-miss bytes per call}, note) measured now: two child runs of `rocprofv3 --pmc <counters> --
    python3 bench.py <same flags> --traffic_probe`, read requests in one, write requests in the other (one run
    holds at most four TCC counters).  Must be called before this process touches the GPU.  (None, reason) when
    it cannot be done; never raises."""
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    if any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ) or "rocprof" in os.environ.get("LD_PRELOAD", ""):
        return None, "this process runs under a profiler itself: no nested counter runs"
    tool = shutil.which("rocprofv3") or os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "rocprofv3")
    if not os.path.exists(tool):
        return None, "rocprofv3 not found"
    flags = [a for a in sys.argv[1:]]
    read_b = lambda c: 32.0 * c.get("TCC_EA0_RDREQ_32B_sum", 0.0) + 64.0 * c.get("TCC_EA0_RDREQ_64B_sum", 0.0) + \
        128.0 * c.get("TCC_EA0_RDREQ_128B_sum", 0.0)
    write_b = lambda c: 64.0 * c.get("TCC_EA0_WRREQ_64B_sum", 0.0) + \
        32.0 * (c.get("TCC_EA0_WRREQ_sum", 0.0) - c.get("TCC_EA0_WRREQ_64B_sum", 0.0))
    parts = []
    work = tempfile.mkdtemp(prefix="eppgcn_traffic_", dir="/tmp")
    try:
        for counters, bytes_of in zip(PMC_PASSES, (read_b, write_b)):
            out_dir = os.path.join(work, counters[0])
            cmd = [tool, "--pmc", *counters, "--output-format", "csv", "-d", out_dir, "-o", "run", "--",
                   sys.executable, os.path.join(ROOT, "bench.py"), *flags, "--traffic_probe"]
            env = dict(os.environ, TMPDIR="/tmp")
            proc = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE,
                                    start_new_session=True)
            try:
                _, err = proc.communicate(timeout=timeout_s)
            except subprocess.TimeoutExpired:
                os.killpg(proc.pid, signal.SIGKILL)      # the process group this call started, nothing else
                proc.communicate()
                return None, f"counter run ({counters[0]} ...) exceeded {timeout_s} s and was stopped"
            if proc.returncode != 0:
                tail = err.decode(errors="replace").strip().splitlines()[-1:] or [""]
                return None, f"counter run ({counters[0]} ...) ended with code {proc.returncode}: {tail[0][:200]}"
            found = glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True)
            if not found:
                return None, "the counter run left no counter_collection.csv"
            parts.append(call_bytes_from_counters(found[0], bytes_of))
    except Exception as exc:               # a measurement aid must never take the benchmark down
        return None, f"live counters failed: {exc!r}"
    finally:
        shutil.rmtree(work, ignore_errors=True)
    return {name: float(round(parts[0][name] + parts[1][name])) for name in CALL_ORDER}, \
        "measured in this run: rocprofv3 --pmc " + " ".join(PMC_PASSES[0]) + " / " + " ".join(PMC_PASSES[1]) + \
        f" over `bench.py --traffic_probe` ({PROBE_REPS} calls each)"


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (no multi-GPU path exists).",
              file=sys.stderr)
        sys.exit(2)

    # the counter runs are child processes of their own and come first: nothing in this process has touched the GPU yet
    live, live_note = (None, "switched off (--no_live_traffic)") if (args.no_live_traffic or args.traffic_probe) \
        else live_traffic()
    log(args, "live traffic:", live, live_note)

    import torch
    from eppgcn_amd import capi, graphs, workload

    capi.load()                      # fails loudly when the HIP library is missing
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs the MI355X (no CPU fallback exists)")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    t0 = time.perf_counter()
    g = graphs.make_graph(args.config, device=dev)
    if args.degree_order:
        g = graphs.renumber(g, graphs.degree_order(g))
    torch.cuda.synchronize()
    log(args, "graph", g.stats(), f"{time.perf_counter() - t0:.1f}s")
    if args.no_stream:
        capi.set_stream_mode(False)      # before the plans are built: their order follows the kernel that will run
    elif args.wide_stream:
        capi.set_stream_mode(True, wide=True)
    if args.plan_shift:
        capi.set_plan_shift(args.plan_shift)
    if args.length_classes:
        capi.set_plan_length_classes(True)
    if args.plan_keep >= 0:
        capi.set_plan_keep_rows(args.plan_keep)
    t0 = time.perf_counter()
    wl = workload.prepare(g, 2, args.train_ratio, 2, args.part_size or None, args.backsize_mode, args.backsize,
                          plan=False if args.no_plan else (True if args.force_plan else None),
                          fused=args.fused_prep)
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
    p_last, p_first = wl.paths[1], wl.paths[0]
    # one workspace per width, shared by the forward and the backward launch of that width: the pre-scaled
    # table and, behind it, room for the partial sums of either plan's stream form
    ws16, ws22 = ((capi.feature_workspace(n, 16, dev, (wl.plans.get(16), p_first.plan)),
                   capi.feature_workspace(n, 22, dev, (wl.plans.get(22), p_last.plan)))
                  if not args.no_workspace else (None, None))
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

    if args.traffic_probe:
        assert tuple(k[0] for k in kernels) == CALL_ORDER
        for _ in range(PROBE_REPS):
            step()
        torch.cuda.synchronize()
        return

    checked = None if args.no_check else check_launches(g, wl, kernels, (x16, x22, dy22, dy16), (out16, out22))

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

    graph_ms = None
    if args.hip_graph:
        # the library records kernel nodes only (no memset nodes, no allocation), so the step can be captured as it is
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        # a replay must leave what the eager step leaves: the same bits through the stream form (fixed summation
        # order), the same values to rounding where the group kernel combines rows with float atomics
        ref16, ref22 = out16.clone(), out22.clone()
        step()
        torch.cuda.synchronize()
        same = (torch.equal(ref16, out16) and torch.equal(ref22, out22)) if capi.last_call_used_stream() else \
            (torch.allclose(ref16, out16, rtol=1e-4, atol=1e-5) and torch.allclose(ref22, out22, rtol=1e-4, atol=1e-5))
        if not same:
            raise SystemExit("bench.py: the step replayed from a HIP graph differs from the eager step")

    # per launch: the whole call (output clear + pre-scaling pass + aggregation kernel) between two HIP
    # events on the launch stream, calls issued back to back; and, from the library's own events on the
    # same stream, the three parts apart (with those enabled every part is followed by a host wait,
    # so they are taken in a pass of their own)
    per_kernel = {}
    reps = max(3, min(args.steps, 10))
    for name, fn, nbytes in kernels:
        call_ms = _event_ms(fn, reps)
        streamed = capi.last_call_used_stream()       # which kernel family the call just ran
        which = 0 if name.startswith("fwd") else 1
        capi.set_timing(True)
        capi.clear_time()
        for _ in range(reps):
            fn()
        ms, clear_ms, scale_ms = (capi.get_time_ms(w) / reps for w in (which, 3, 4))
        capi.set_timing(False)
        capi.clear_time()
        per_kernel[name] = {"call_ms": round(call_ms, 4), "kernel_ms": round(ms, 4), "clear_ms": round(clear_ms, 4),
                            "prescale_ms": round(scale_ms, 4), "stream_form": streamed, "alg_bytes": nbytes,
                            "alg_GBps": round(nbytes / call_ms / 1e6, 1),
                            "pct_peak": round(nbytes / call_ms / 1e6 / PEAK_HBM_GBS * 100, 2),
                            "kernel_only_pct_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS * 100, 2)}
    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.gather_probe:
        gather_probe(dev)
    dominant = max(per_kernel, key=lambda k: per_kernel[k]["call_ms"])
    dk = per_kernel[dominant]
    dim = 22 if "d22" in dominant else 16
    compulsory = workload.bytes_compulsory(n, e, dim)
    committed, committed_note = measured_traffic(args.config, dominant)
    if live is not None and all(per_kernel[k]["stream_form"] for k in per_kernel):
        traffic, traffic_note = live[dominant], live_note
    else:
        traffic, traffic_note = committed, committed_note + ("" if live_note.startswith("switched off") else
                                                              f" (live counters: {live_note})")
    sec = dk["call_ms"] * 1e-3
    roofline = {"bound": "hbm", "kernel": dominant,
                "launch": "whole call: output clear + pre-scaling pass + stream kernel + fix-up kernel "
                          "(group kernel where the stream form does not run)",
                "achieved": dk["alg_GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(dk["alg_GBps"] / PEAK_HBM_GBS, 4),
                "frac_basis": "algorithmic gather model, not a physical bound: every walked edge is priced as one row "
                              "read from HBM, rows served from the caches count as moved, so frac can pass 1.0 without "
                              "any work being skipped (the result check covers the timed launches); the bounded "
                              "figure is hbm_frac",
                "traffic": traffic, "traffic_source": traffic_note,
                "traffic_committed": committed, "traffic_committed_source": committed_note,
                "traffic_is": "L2-miss (fabric-side) bytes of the call: TCC->EA read requests x their sizes (32 / 64 / "
                              "128 B) + write requests x their sizes (32 / 64 B), rocprofv3 --pmc, no fitted factor; "
                              "the counters sit between L2 and the fabric, so a hit in the 256 MB memory-side cache "
                              "counts like an HBM access",
                "call_ms": dk["call_ms"], "kernel_ms": dk["kernel_ms"], "clear_ms": dk["clear_ms"],
                "prescale_ms": dk["prescale_ms"], "alg_bytes_per_launch": dk["alg_bytes"],
                "kernel_only_frac": round(dk["alg_bytes"] / (dk["kernel_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                "hbm_frac": None if traffic is None else round(traffic / sec / 1e9 / PEAK_HBM_GBS, 4),
                "compulsory_bytes": compulsory,
                "compulsory_frac": round(compulsory / sec / 1e9 / PEAK_HBM_GBS, 4)}

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
                   "feature_workspace": not args.no_workspace, "degree_order": bool(args.degree_order),
                   "column_blocked_plan": bool(wl.plans),
                   "stream_form": all(k["stream_form"] for k in per_kernel.values()),
                   "partial_sum_rows": {"fwd_agg_d16": getattr(wl.plans.get(16), "partial_rows", 0),
                                        "fwd_agg_d22": getattr(wl.plans.get(22), "partial_rows", 0),
                                        "bwd_agg_d22_last": getattr(p_last.plan, "partial_rows", 0),
                                        "bwd_agg_d16_first": getattr(p_first.plan, "partial_rows", 0)}},
        "agg_ms_per_epoch": round(ms_per_step, 4), "alg_bytes_per_epoch": bytes_epoch,
        "graph_ms_per_step": None if graph_ms is None else round(graph_ms, 4),
        "pct_of_peak_hbm": round(value / PEAK_HBM_GBS * 100, 2),
        "value_is": "algorithmic (gather-model) bytes of the epoch / wall time: a cache-amplified figure, not measured "
                    "traffic (that is l2_miss_traffic_GBps)",
        "per_kernel": per_kernel, "path_preparation_s": round(prep_s, 3),
        "result_check": checked,
        "roofline": roofline,
    }
    traffic_epoch = [live[k] for k in per_kernel] if traffic_note == live_note and live is not None else \
        [measured_traffic(args.config, k)[0] for k in per_kernel]
    if all(t is not None for t in traffic_epoch):
        # L2-miss (fabric-side) traffic of the four calls, from the same source as roofline.traffic
        result["l2_miss_traffic_bytes_per_epoch"] = sum(traffic_epoch)
        result["l2_miss_traffic_GBps"] = round(sum(traffic_epoch) / (ms_per_step * 1e-3) / 1e9, 1)
        result["l2_miss_traffic_pct_of_peak"] = round(result["l2_miss_traffic_GBps"] / PEAK_HBM_GBS * 100, 2)

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


PROFILED_SOURCES = ("aggregate.hip", "stream.hip", "common.hpp", "schedule.hip", "prepare.hip")


def kernel_source_hash():
    """sha256 (first 16 hex digits) over the sources that decide what an aggregation call moves: the
    kernels, the plan builder and the clear kernels.  A counter summary under profiles/ names the
    hash it was taken with."""
    import hashlib
    h = hashlib.sha256()
    for name in PROFILED_SOURCES:
        with open(os.path.join(ROOT, "eppgcn_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(config, kernel):
    """(L2-miss traffic in bytes per call of `kernel`, where it comes from) from the committed rocprofv3
    counter summary of the same bench command: TCC->EA read and write requests of the call's kernels times
    their sizes.
    (None, reason) when no summary covers this workload or the kernel sources have changed since it
    was taken - a stale counter must not pose as a measurement."""
    import glob
    import re
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        text = open(path).read()
        m = re.search(r"traffic_bytes %s %s = ([0-9.e+]+)" % (re.escape(config), re.escape(kernel)), text)
        if not m:
            continue
        h = re.search(r"kernel_source_sha256 = ([0-9a-f]+)", text)
        rel = os.path.relpath(path, ROOT)
        if not h or h.group(1) != kernel_source_hash():
            return None, f"{rel} was taken from other kernel sources ({h.group(1) if h else 'no hash'} != {kernel_source_hash()})"
        return float(m.group(1)), rel
    return None, "no counter summary under profiles/ covers this workload"


def gather_probe(dev):
    """Aggregation over a permutation graph: row r gathers exactly row perm[r] of a 2^22-row table that
    arrives pre-scaled, so one launch reads every table row once (64-byte rows at width 16, 128-byte
    rows at width 32) plus 16 bytes of indices and scale per row, and writes the output once.  Under
    rocprofv3 --pmc these launches (the only ones over `ForwardGroups` at these widths) give the
    factor between FETCH_SIZE and the bytes a row gather really moves."""
    import torch
    from eppgcn_amd import capi
    n = 1 << 22
    gen = torch.Generator(device=dev).manual_seed(5)
    col = torch.randperm(n, device=dev, generator=gen).int()
    part_ptr = torch.arange(n + 1, dtype=torch.int32, device=dev)
    part2node = torch.arange(n, dtype=torch.int32, device=dev)
    ones = torch.ones(n, device=dev)
    for dim in (16, 32):
        table = torch.empty(n, capi.feature_workspace_pitch(dim), device=dev).normal_()     # n is a multiple of 4096
        rows = capi.feature_workspace_rows(n, dev)
        out = torch.empty(n, dim, device=dev)
        for _ in range(3):
            capi.spmm_forward(None, col, ones, part_ptr, part2node, 1, 32, 8, None, out, workspace=table.view(-1),
                              prescaled_dim=dim)
        torch.cuda.synchronize()
        assert torch.equal(out, table[rows[col.long()]][:, :dim])
        del table, out


def check_launches(g, wl, kernels, inputs, outputs):
    """Every timed launch (plan + feature workspace + gathered-rows bitmap) against the same operator
    without plan and workspace - another kernel instantiation, per-edge scale gather, CSR order - within
    2e-5 * sum |w x| per element (the yardstick is the operator applied to |x|).  Raises on a mismatch:
    a number must never be printed for a kernel whose results are off."""
    import torch
    from eppgcn_amd import capi
    x16, x22, dy22, dy16 = inputs
    out16, out22 = outputs
    fwd = lambda x: capi.spmm_forward(x, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                                      g.row_pointers, None, workspace=None)
    p_last, p_first = wl.paths[1], wl.paths[0]
    bwd = lambda dy, p: capi.ours_backward(dy, p.ids, p.part_pointer, p.edge_list, g.degrees, p.num_parts, p.part_size,
                                           p.layer, 4, 16, None, workspace=None)
    plain = {"fwd_agg_d16": lambda: fwd(x16), "fwd_agg_d22": lambda: fwd(x22),
             "bwd_agg_d22_last": lambda: bwd(dy22, p_last), "bwd_agg_d16_first": lambda: bwd(dy16, p_first)}
    source = {"fwd_agg_d16": (x16, out16), "fwd_agg_d22": (x22, out22), "bwd_agg_d22_last": (dy22, out22),
              "bwd_agg_d16_first": (dy16, out16)}
    worst = {}
    for name, fn, _ in kernels:
        x, out = source[name]
        out.fill_(float("nan"))
        fn()
        want = plain[name]()
        yardstick = fwd(x.abs())
        ratio = float(((out - want).abs() / (2e-5 * yardstick + 1e-30)).max())
        if not ratio <= 1.0:
            raise SystemExit(f"bench.py: {name} differs from the unplanned, unscaled operator: "
                             f"max err / (2e-5 * sum|w x|) = {ratio:.3f}")
        worst[name] = round(ratio, 4)
        del want, yardstick
    return {"against": "same operator without plan and workspace", "tolerance": "2e-5 * sum|w x| per element",
            "max_err_over_tolerance": worst}


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
