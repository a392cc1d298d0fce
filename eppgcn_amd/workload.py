"""Builds the device-resident state of one benchmark configuration the way the reference's
driver does (EPPGCN/gcn_main.py:120-168): forward neighbour groups, the mask chain over the
layers, and for every layer the compacted backward path split into groups.

Everything is computed by the HIP library through the C ABI; torch only holds the buffers.
Also home of the algorithmic byte counts the bandwidth figures are quoted on.
"""
from __future__ import annotations

import dataclasses
from typing import List

import torch

from . import capi, graphs, param


@dataclasses.dataclass
class BackwardPath:
    """Compacted execution path of one layer's backward aggregation."""
    layer: int               # 1-based conv layer this path belongs to
    ids: torch.Tensor        # int32 [E]   row of every kept edge (first valid_len entries)
    edge_list: torch.Tensor  # int32 [E]   column of every kept edge
    part_pointer: torch.Tensor  # int32 [E+1] group starts, terminator at num_parts
    node_degs: torch.Tensor  # int32 [N]   kept edges per row
    part_size: int
    num_parts: int
    valid_len: int
    valid_node: int
    plan: object = None      # column-blocked execution plan of this path (speed only)
    gathered_rows: torch.Tensor = None   # bitmap of the rows the path gathers, when fewer than half (speed only)


@dataclasses.dataclass
class Workload:
    graph: graphs.Graph
    part_size: int
    part_ptr: torch.Tensor
    part2node: torch.Tensor
    train_mask: torch.Tensor
    ngh_masks: List[torch.Tensor]
    paths: List[BackwardPath]     # paths[k] belongs to conv layer k (0-based), as edge_masks[k] does
    plans: dict = None            # feature width -> execution plan of the forward groups

    @property
    def num_parts(self) -> int:
        return int(self.part2node.numel())


def choose_back_part_size(mode: str, constant: int, valid_node: int, valid_len: int) -> int:
    """Backward group size: 'constant', 'map' (fitted regression, EPPGCN/GCNConv/EPPGCN.cpp:298-325;
    the wave64 rule where the regression drops below 1), 'threshold' (legacy rule of build_back_part, :246-258) or 'wave64' (the rule
    re-fitted for this library's kernels)."""
    if mode == "constant":
        return max(1, int(constant))
    if mode == "map":
        return capi.auto_back_part_size(valid_node, valid_len)[0]
    if mode == "threshold":
        return capi.threshold_back_part_size(valid_node, valid_len) or 64
    if mode == "wave64":
        return capi.wave64_back_part_size(valid_node, valid_len)
    raise ValueError(f"unknown backsize mode {mode!r}")


def prepare(graph: graphs.Graph, num_layers: int = 2, train_ratio: float = 0.1, mask_seed: int = 2,
            part_size: int = None, backsize_mode: str = "constant", backsize: int = 32,
            train_mask: torch.Tensor = None, widths=(16, 22), plan=None, fused: bool = False) -> Workload:
    """``fused``: mark and compact every layer in one pass (no E-entry edge masks) instead of the
    reference's separate steps.  The results are identical; the one-pass form saves 4 bytes per edge and
    layer of memory but is no faster (R-MAT scale 22, both layers: 7.0 ms either way), so the reference's
    steps are the default."""
    g = graph
    dev = g.column_index.device
    n, e = g.num_nodes, g.num_edges
    if plan is None:             # default: plans where the feature table outgrows the caches
        plan = capi.plan_recommended(n, max(widths))
    # EPPGCN/param.py:80 takes int(average degree); the floor is the wave64 re-fit of that rule
    ps = part_size or max(param.MIN_AUTO_PART_SIZE, int(g.avg_degree))
    part_ptr, part2node = capi.build_part(ps, g.row_pointers, e)
    if train_mask is None:
        train_mask = graphs.bernoulli_mask(n, train_ratio, mask_seed, dev)

    # per-run state, EPPGCN/dataset.py:135-156
    ngh_masks = [torch.zeros(n, dtype=torch.bool, device=dev) for _ in range(num_layers - 1)]
    edge_masks = ([None] * num_layers if fused else
                  [torch.full((e,), -1, dtype=torch.int32, device=dev) for _ in range(num_layers)])
    node_degs = [torch.zeros(n, dtype=torch.int32, device=dev) for _ in range(num_layers)]

    # mask chain, EPPGCN/gcn_main.py:130-139: step i runs in the forward of conv i
    for i in range(num_layers):
        src = train_mask if i == 0 else ngh_masks[i - 1]
        last = i == num_layers - 1
        dst = None if last else ngh_masks[i]
        k = num_layers - 1 - i
        if fused:
            edge_masks[k] = capi.mark_compact(part2node, part_ptr, g.column_index, src, dst, node_degs[k], last)
        else:
            capi.mask_forward(part2node, part_ptr, g.column_index, src, dst, edge_masks[k], node_degs[k], last)

    # buildBackPart, EPPGCN/gcn_main.py:151-168
    paths = []
    for k in range(num_layers):
        ids, edge_list, valid_len = (edge_masks[k] if fused else
                                     capi.compact_back_edge(edge_masks[k], g.column_index))
        edge_masks[k] = None
        valid_node = capi.count_nonzero(node_degs[k])
        bps = choose_back_part_size(backsize_mode, backsize, valid_node, valid_len)
        part_pointer, num_parts, v2 = capi.split_back_part(node_degs[k], e, bps)
        assert v2 == valid_len
        width = widths[min(k, len(widths) - 1)]
        # a heavily pruned path gathers from few distinct rows, which stay cached in any order: its
        # plan keeps the groups in one block
        path_plan = (capi.build_plan(part_pointer, edge_list, num_parts, valid_len, n, width, ids=ids,
                                     block_shift=0 if 2 * valid_len >= e else 31)
                     if plan and num_parts > 0 else None)
        # the pre-scaling pass of the gradient only has to cover the rows the path reads
        bitmap, distinct = capi.mark_gathered_rows(edge_list, valid_len, n)
        paths.append(BackwardPath(k + 1, ids, edge_list, part_pointer, node_degs[k], bps, num_parts,
                                  valid_len, valid_node, path_plan, bitmap if 2 * distinct < n else None))
    # one plan of the forward groups serves every width (the column block is sized for the widest)
    plans = {}
    if plan and part2node.numel() > 0:
        shared = capi.build_plan(part_ptr, g.column_index, part2node.numel(), e, n, max(widths), part2node=part2node)
        plans = {w: shared for w in set(widths)}
    return Workload(g, ps, part_ptr, part2node, train_mask, ngh_masks, paths, plans)


# ------------------------------------------------------------------ algorithmic bytes (4-byte elements)
def bytes_forward(num_nodes: int, num_edges: int, dim: int) -> int:
    """Gather model: per edge its column id, the neighbour's scale and one dim-wide row; per
    vertex one output row, its row pointer and its own scale."""
    return num_edges * (4 + 4 + 4 * dim) + num_nodes * (4 * dim + 4 + 4)


def bytes_pruned_backward(num_nodes: int, valid_len: int, num_parts: int, dim: int) -> int:
    """Per kept edge its column id, the neighbour's scale and one gradient row; the full [N, dim]
    output written once; per group its pointer and its row id."""
    return valid_len * (4 + 4 + 4 * dim) + num_nodes * 4 * dim + num_parts * 8


def bytes_compulsory(num_nodes: int, num_edges: int, dim: int) -> int:
    """Lower bound with perfect reuse: every input row read once."""
    return 4 * num_edges + 8 * num_nodes + 8 * num_nodes * dim


def bytes_mask(num_nodes: int, num_edges: int) -> int:
    return num_edges * (4 + 1) + num_edges * 4 + num_nodes * 4


def bytes_compact(num_edges: int, valid_len: int) -> int:
    return num_edges * 4 + valid_len * 4 + valid_len * 8


def bytes_split(num_nodes: int, num_parts: int) -> int:
    return num_nodes * 4 + num_parts * 12
