"""Backward-path stress sweep (benchmark configuration 5): on one graph, train-mask ratios x
aggregation widths x backward group sizes.  For every cell, what a caller sees: the time of the
whole pruned backward *call* (output clear + pre-scaling pass + aggregation kernels; two HIP events
around back-to-back calls) next to the whole unpruned call, algorithmic GB/s and the speed-up on the
calls, the same pruned call for a consumer that takes the bitmap of the written rows instead of a
cleared output (``eppgcn_ours_backward_rows``: what the extension module's backward runs), the
aggregation kernels alone as sub-fields, and what the pruned path costs to prepare
(marking, compaction, split, gathered-rows bitmap, execution plan) with the number of backward
calls after which the preparation has paid for itself.

    python -m eppgcn_amd.sweep [--config cfg3_rmat20] [--ratios 0.01 0.1 0.5]
                               [--widths 16 64 256] [--groups 8 16 32 64] [--reps 5]

Every cell is checked before it is reported (pruned against unpruned backward within 2e-5 of the
absolute sum); a disagreement ends the sweep.  Prints one JSON line per cell and a final summary line.  Needs the MI355X.  Launches are set up
the way the extension module sets them up by itself: execution plans where the feature table has 4 MB
or more (column-blocked for the forward groups and for paths that keep at least half of the edges,
one block otherwise) and the gathered-rows bitmap for paths that read fewer than half of the rows;
``--no_plans`` measures the bare kernels.
"""
from __future__ import annotations

import argparse
import json
import time

import torch

from . import capi, graphs, param, workload


def _events_ms(fn, reps):
    fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="cfg3_rmat20")
    ap.add_argument("--ratios", type=float, nargs="+", default=[0.01, 0.1, 0.5])
    ap.add_argument("--widths", type=int, nargs="+", default=[16, 64, 256])
    ap.add_argument("--groups", type=int, nargs="+", default=[8, 16, 32, 64])
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--no_plans", action="store_true", help="no execution plans, no gathered-rows bitmap")
    args = ap.parse_args()

    capi.load()
    dev = torch.device("cuda:0")
    g = graphs.make_graph(args.config, device=dev)
    n, e = g.num_nodes, g.num_edges
    ps = max(param.MIN_AUTO_PART_SIZE, int(g.avg_degree))     # the decider's rule for the forward groups
    part_ptr, part2node = capi.build_part(ps, g.row_pointers, e)
    fwd_plans = {}

    def forward_plan(width):
        if args.no_plans or not capi.plan_recommended(n, width):
            return None
        if width not in fwd_plans:
            fwd_plans[width] = capi.build_plan(part_ptr, g.column_index, part2node.numel(), e, n, width,
                                               part2node=part2node)
        return fwd_plans[width]

    cells = []
    for ratio in args.ratios:
        mask = graphs.bernoulli_mask(n, ratio, 2, dev)
        bem = torch.full((e,), -1, dtype=torch.int32, device=dev)
        degs = torch.zeros(n, dtype=torch.int32, device=dev)

        def mark():
            bem.fill_(-1)
            degs.zero_()
            capi.mask_forward(part2node, part_ptr, g.column_index, mask, None, bem, degs, True)

        mark_ms = _events_ms(mark, args.reps)
        compact_ms = _events_ms(lambda: capi.compact_back_edge(bem, g.column_index), args.reps)
        ids, edge_list, valid_len = capi.compact_back_edge(bem, g.column_index)
        valid_node = capi.count_nonzero(degs)
        bitmap, distinct = capi.mark_gathered_rows(edge_list, valid_len, n)
        gathered = bitmap if (2 * distinct < n and not args.no_plans) else None
        bitmap_ms = _events_ms(lambda: capi.mark_gathered_rows(edge_list, valid_len, n), args.reps) if gathered is not None else 0.0
        for gs in args.groups:
            split_ms = _events_ms(lambda: capi.split_back_part(degs, e, gs), args.reps)
            part_pointer, num_parts, _ = capi.split_back_part(degs, e, gs)
            for width in args.widths:
                dy = graphs.normal32(7, (n, width), dev) * mask[:, None]
                out = torch.empty_like(dy)
                plan, plan_ms = None, 0.0
                if not args.no_plans and num_parts > 0 and capi.plan_recommended(n, width):
                    build = lambda: capi.build_plan(part_pointer, edge_list, num_parts, valid_len, n, width, ids=ids,
                                                    block_shift=0 if 2 * valid_len >= e else 31)
                    plan_ms = _events_ms(build, args.reps)       # includes the status read-back and its host wait
                    plan = build()
                # one workspace serves both plans of the cell: each plan's partial sums need their own room in it
                ws = capi.feature_workspace(n, width, dev, [p for p in (plan, forward_plan(width)) if p is not None])
                def pruned_call():
                    capi.ours_backward(dy, ids, part_pointer, edge_list, g.degrees, num_parts, gs, 1, 4, 16, out, ws,
                                       plan=plan, gathered_rows=gathered)

                def pruned_rows_call():
                    # for a consumer that takes the bitmap of the written rows (the layer's dense products): no clear
                    capi.ours_backward_rows(dy, ids, part_pointer, edge_list, g.degrees, num_parts, gs, 1, 4, 16, out, ws,
                                            plan=plan, gathered_rows=gathered)

                def unpruned_call():
                    capi.spmm_forward(dy, g.column_index, g.degrees, part_ptr, part2node, ps, 32, 8, None, out, True, ws,
                                      plan=forward_plan(width))

                def parts_ms(fn):
                    """the library's own events: aggregation kernels / output clear / pre-scaling pass (each followed
                    by a host wait, so they are taken apart from the call time)"""
                    capi.set_timing(True)
                    capi.clear_time()
                    for _ in range(args.reps):
                        fn()
                    res = [capi.get_time_ms(w) / args.reps for w in (1, 3, 4)]
                    capi.set_timing(False)
                    capi.clear_time()
                    return res

                # the whole call between two events, calls back to back (the first, untimed call of _events_ms loads the
                # kernels' code); then the parts
                pruned_ms = _events_ms(pruned_call, args.reps)
                streamed = capi.last_call_used_stream()
                unpruned_ms = _events_ms(unpruned_call, args.reps)
                pruned_rows_ms = _events_ms(pruned_rows_call, args.reps)
                pruned_kernel_ms, pruned_clear_ms, pruned_scale_ms = parts_ms(pruned_call)
                unpruned_kernel_ms, unpruned_clear_ms, unpruned_scale_ms = parts_ms(unpruned_call)
                unpruned_call()                   # `out` holds the unpruned result for the check below
                # a timed cell is a checked cell: `out` holds the unpruned result; the pruned one sums the same
                # terms in another order, so they agree within 2e-5 * sum |w x| (the yardstick comes from the
                # same operator applied to |dy|)
                pruned_out = capi.ours_backward(dy, ids, part_pointer, edge_list, g.degrees, num_parts, gs, 1, 4, 16, None,
                                                ws, plan=plan, gathered_rows=gathered)
                yardstick = capi.spmm_forward(dy.abs(), g.column_index, g.degrees, part_ptr, part2node, ps, 32, 8, None,
                                              None, True, ws, plan=forward_plan(width))
                worst = float(((pruned_out - out).abs() / (2e-5 * yardstick + 1e-30)).max())
                if not worst <= 1.0:
                    raise SystemExit(f"sweep: pruned and unpruned backward disagree at ratio {ratio}, width {width}, "
                                     f"group size {gs}: max err / limit = {worst:.3f}")
                del pruned_out, yardstick
                nbytes = workload.bytes_pruned_backward(n, valid_len, num_parts, width)
                del plan
                prep_ms = mark_ms + compact_ms + split_ms + bitmap_ms + plan_ms
                saved = unpruned_ms - pruned_ms
                cell = {"config": args.config, "ratio": ratio, "width": width, "group_size": gs,
                        "kept_edges": valid_len, "kept_rows": valid_node, "groups": num_parts,
                        "mark_ms": round(mark_ms, 4), "compact_ms": round(compact_ms, 4), "split_ms": round(split_ms, 4),
                        "bitmap_ms": round(bitmap_ms, 4), "plan_ms": round(plan_ms, 4), "prep_ms": round(prep_ms, 4),
                        "pruned_call_ms": round(pruned_ms, 4), "unpruned_call_ms": round(unpruned_ms, 4),
                        "pruned_rows_call_ms": round(pruned_rows_ms, 4),
                        "speedup_rows_call": round(unpruned_ms / pruned_rows_ms, 2),
                        "pruned_GBps": round(nbytes / pruned_ms / 1e6, 1),
                        "unpruned_GBps": round(workload.bytes_forward(n, e, width) / unpruned_ms / 1e6, 1),
                        "speedup": round(unpruned_ms / pruned_ms, 2),
                        "calls_to_break_even": round(prep_ms / saved, 1) if saved > 0 else None,
                        "pruned_parts_ms": {"kernels": round(pruned_kernel_ms, 4), "clear": round(pruned_clear_ms, 4),
                                            "prescale": round(pruned_scale_ms, 4)},
                        "unpruned_parts_ms": {"kernels": round(unpruned_kernel_ms, 4), "clear": round(unpruned_clear_ms, 4),
                                              "prescale": round(unpruned_scale_ms, 4)},
                        "speedup_kernels_only": round(unpruned_kernel_ms / pruned_kernel_ms, 2),
                        "stream_form": bool(streamed),
                        "pruned_vs_unpruned_err_over_limit": round(worst, 4)}
                cells.append(cell)
                print(json.dumps(cell), flush=True)
    best = {}
    for c in cells:
        key = (c["ratio"], c["width"])
        if key not in best or c["pruned_call_ms"] < best[key]["pruned_call_ms"]:
            best[key] = c
    print(json.dumps({"summary": "best group size per (ratio, width)",
                      "best": [{"ratio": k[0], "width": k[1], "group_size": v["group_size"],
                                "pruned_call_ms": v["pruned_call_ms"], "speedup": v["speedup"]}
                               for k, v in sorted(best.items())]}), flush=True)


if __name__ == "__main__":
    t0 = time.time()
    main()
