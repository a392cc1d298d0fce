"""Vectorised numpy closed forms of the path-preparation functions and dense /
sparse algebra for the aggregations.  Test infrastructure only.

These are written independently of ``eppgcn_oracle.c`` (no loops over groups,
no shared code) so that agreement between the two pins both: a dropped term,
an off-by-one group boundary or a swapped row/column shows up as a mismatch.
Notation: ``row = repeat(arange(N), diff(indptr))``, ``col = column_index``.
"""
from __future__ import annotations

import numpy as np


def row_index(indptr) -> np.ndarray:
    indptr = np.asarray(indptr, np.int64)
    return np.repeat(np.arange(indptr.size - 1, dtype=np.int64), np.diff(indptr))


def build_part(part_size: int, indptr):
    """Groups of <= part_size consecutive CSR slots, never crossing a row.
    (what EPPGCN/GCNConv/EPPGCN.cpp:186-227 computes)"""
    indptr = np.asarray(indptr, np.int64)
    deg = np.diff(indptr)
    q = -(-deg // part_size)                       # ceil
    part2node = np.repeat(np.arange(deg.size, dtype=np.int64), q)
    first_group_of_row = np.cumsum(q) - q          # index of the row's first group
    rank_in_row = np.arange(part2node.size, dtype=np.int64) - first_group_of_row[part2node]
    part_ptr = indptr[part2node] + part_size * rank_in_row
    part_ptr = np.concatenate([part_ptr, indptr[-1:]])
    return part_ptr.astype(np.int32), part2node.astype(np.int32)


def mask_forward(indptr, col, src_mask, ngh_mask, back_edge_mask, node_degs, is_last: bool):
    """Returns the updated (ngh_mask, back_edge_mask, node_degs); inputs untouched.
    (what EPPGCN/GCNConv/EPPGCN_kernel.cu:351-388 computes for any forward partition)"""
    row = row_index(indptr)
    col = np.asarray(col, np.int64)
    src_mask = np.asarray(src_mask, bool)
    keep = src_mask[col]
    bem = np.array(back_edge_mask, np.int32, copy=True)
    bem[keep] = row[keep]
    degs = np.array(node_degs, np.int32, copy=True)
    degs += np.bincount(row[keep], minlength=degs.size).astype(np.int32)
    ngh = None if ngh_mask is None else np.array(ngh_mask, bool, copy=True)
    if not is_last:
        sel = src_mask[row]
        ngh[row[sel]] = True
        ngh[col[sel]] = True
    return ngh, bem, degs


def compact_mask(edge_mask, col):
    """(what EPPGCN/GCNConv/cuCompactor.cu:328-465 computes)"""
    edge_mask = np.asarray(edge_mask, np.int32)
    idx = np.flatnonzero(edge_mask != -1)
    out_id = np.zeros_like(edge_mask)
    out_edge = np.zeros_like(edge_mask)
    out_id[: idx.size] = edge_mask[idx]
    out_edge[: idx.size] = np.asarray(col, np.int32)[idx]
    return out_id, out_edge, int(idx.size)


def compact_count(node_degs) -> int:
    return int(np.count_nonzero(np.asarray(node_degs)))


def split_back_part(node_degs, num_edges: int, part_size: int):
    """part_pointer[:P+1] = [0, cumsum(counts)] where the counts of a vertex with
    g > 0 kept edges are ps,...,ps,g-(q-1)ps.  Length num_edges+1, tail zero.
    (EPPGCN/GCNConv/EPPGCN.cpp:327-346 over cuCompactor.cu:467-621 and :42-48)"""
    g = np.asarray(node_degs, np.int64)
    g = g[g > 0]
    q = -(-g // part_size)
    p = int(q.sum())
    owner = np.repeat(np.arange(g.size), q)
    rank = np.arange(p) - (np.cumsum(q) - q)[owner]
    start_of_vertex = np.cumsum(g) - g
    part_pointer = np.zeros(num_edges + 1, np.int32)
    part_pointer[:p] = (start_of_vertex[owner] + rank * part_size).astype(np.int32)
    part_pointer[p] = int(g.sum())
    return part_pointer, p


def c_round(x: float) -> int:
    """C round(): half away from zero."""
    return int(np.floor(x + 0.5)) if x >= 0 else int(-np.floor(-x + 0.5))


def map_back_part_size(valid_node: int, valid_len: int) -> int:
    """(EPPGCN/GCNConv/EPPGCN.cpp:303-310)"""
    vd = valid_len / valid_node
    return c_round(0.65538 + 1.67431e-5 * valid_node - 2.24342e-6 * valid_len + 0.63641 * vd)


def threshold_back_part_size(valid_node: int, valid_len: int) -> int:
    """(EPPGCN/GCNConv/EPPGCN.cpp:246-258)"""
    vd = valid_len // valid_node
    for bound, size in ((4, 4), (16, 8), (64, 16), (256, 32), (512, 64)):
        if vd < bound:
            return size
    return 0


def get_ginfo(node_degs, valid_len: int) -> np.ndarray:
    """(EPPGCN/GCNConv/EPPGCN.cpp:348-386)"""
    d = np.asarray(node_degs, np.int64)
    valid = int(np.count_nonzero(d))
    edges = [1, 5, 10, 20, 40, 80, 160]
    hist = [int(((d >= lo) & (d < hi)).sum()) for lo, hi in zip(edges[:-1], edges[1:])]
    rest = d.size - sum(hist)
    re = np.zeros(10, np.float64)
    re[0] = valid / 10000
    re[1] = valid_len / 10000
    re[2] = valid_len / valid
    re[3:9] = np.array(hist) / valid
    re[9] = rest / valid
    return re.astype(np.float32)


def edge_weights32(indptr, col, scale) -> np.ndarray:
    """fl32(s_row * s_col) per CSR slot."""
    s = np.asarray(scale, np.float32)
    return (s[row_index(indptr)] * s[np.asarray(col, np.int64)]).astype(np.float32)


def aggregate_csr64(indptr, col, scale, feats) -> np.ndarray:
    """Textbook CSR product (scipy) in float64 with fp32 edge weights."""
    import scipy.sparse as sp
    n = len(indptr) - 1
    w = edge_weights32(indptr, col, scale).astype(np.float64)
    a = sp.csr_matrix((w, np.asarray(col, np.int64), np.asarray(indptr, np.int64)), shape=(n, n))
    return a @ np.asarray(feats, np.float64)


def aggregate_dense64(indptr, col, scale, feats) -> np.ndarray:
    """diag(s) A diag(s) T with a dense 0/1 adjacency; tiny graphs only."""
    n = len(indptr) - 1
    a = np.zeros((n, n), np.float64)
    a[row_index(indptr), np.asarray(col, np.int64)] = 1.0
    s = np.asarray(scale, np.float32)
    w = (s[:, None] * s[None, :]).astype(np.float32).astype(np.float64)
    return (a * w) @ np.asarray(feats, np.float64)


def abs_sum_bound(indptr, col, scale, feats) -> np.ndarray:
    """sum_j |w_ij x_j| per output element: the magnitude fp32 summation error scales with."""
    import scipy.sparse as sp
    n = len(indptr) - 1
    w = np.abs(edge_weights32(indptr, col, scale).astype(np.float64))
    a = sp.csr_matrix((w, np.asarray(col, np.int64), np.asarray(indptr, np.int64)), shape=(n, n))
    return a @ np.abs(np.asarray(feats, np.float64))


def pruned_path(indptr, col, src_mask, part_size: int):
    """End-to-end closed form of one layer's backward path from a source mask:
    (id, edge_list, part_pointer, valid_len, num_parts, node_degs)."""
    n = len(indptr) - 1
    e = len(col)
    _, bem, degs = mask_forward(indptr, col, src_mask, None, np.full(e, -1, np.int32),
                                np.zeros(n, np.int32), True)
    out_id, out_edge, v = compact_mask(bem, col)
    pp, p = split_back_part(degs, e, part_size)
    return out_id, out_edge, pp, v, p, degs
