"""ctypes front-end of the C restatement (``eppgcn_oracle.c``).  Test infrastructure only.

All functions take and return numpy arrays (int32 indices, float32 features,
uint8/bool masks).  ``load()`` uses the prebuilt ``_build/liboracle.so`` and
builds it with ``make`` when it is absent.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None

_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def load():
    global _lib
    if _lib is not None:
        return _lib
    lib = C.CDLL(build())
    lib.oracle_build_part.restype = C.c_int64
    lib.oracle_build_part.argtypes = [C.c_int, _i32p, C.c_int, C.c_void_p, C.c_void_p]
    for name in ("oracle_spmm_groups", "oracle_spmm_groups_mt"):
        fn = getattr(lib, name)
        fn.restype = None
        fn.argtypes = [_f32p, _f32p, _i32p, _f32p, _i32p, _i32p, C.c_int64, C.c_int, C.c_int]
    lib.oracle_spmm_f64.restype = None
    lib.oracle_spmm_f64.argtypes = [_f64p, _f32p, _i32p, _i32p, _f32p, C.c_int, C.c_int]
    lib.oracle_mask_forward.restype = None
    lib.oracle_mask_forward.argtypes = [_i32p, _i32p, _i32p, _u8p, _u8p, _i32p, _i32p, C.c_int64, C.c_int]
    lib.oracle_compact_mask.restype = C.c_int64
    lib.oracle_compact_mask.argtypes = [_i32p, _i32p, _i32p, _i32p, C.c_int64]
    lib.oracle_compact_count.restype = C.c_int64
    lib.oracle_compact_count.argtypes = [_i32p, C.c_int64]
    lib.oracle_compact_part.restype = C.c_int64
    lib.oracle_compact_part.argtypes = [_i32p, _i32p, C.c_int64, C.c_int]
    lib.oracle_exclusive_scan.restype = None
    lib.oracle_exclusive_scan.argtypes = [_i32p, _i32p, C.c_int64]
    for name in ("oracle_ours_backward", "oracle_ours_backward_mt"):
        fn = getattr(lib, name)
        fn.restype = None
        fn.argtypes = [_f32p, _f32p, _i32p, _i32p, _i32p, _f32p, C.c_int64, C.c_int, C.c_int]
    lib.oracle_map_back_part_size.restype = C.c_int
    lib.oracle_map_back_part_size.argtypes = [C.c_int, C.c_int]
    lib.oracle_threshold_back_part_size.restype = C.c_int
    lib.oracle_threshold_back_part_size.argtypes = [C.c_int, C.c_int]
    lib.oracle_get_ginfo.restype = None
    lib.oracle_get_ginfo.argtypes = [_i32p, C.c_int, C.c_int, _f32p]
    lib.oracle_update_forward.restype = None
    lib.oracle_update_forward.argtypes = [_f32p, C.c_int, _f32p, _f32p, C.c_void_p, C.c_int, C.c_int64, C.c_int, C.c_int]
    lib.oracle_update_backward_input.restype = None
    lib.oracle_update_backward_input.argtypes = [_f32p, _f32p, _f32p, C.c_void_p, C.c_int64, C.c_int, C.c_int]
    lib.oracle_update_backward_weight.restype = None
    lib.oracle_update_backward_weight.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int64, C.c_int, C.c_int]
    lib.oracle_num_threads.restype = C.c_int
    _lib = lib
    return lib


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return np.ascontiguousarray(np.asarray(a).astype(np.uint8))


def num_threads() -> int:
    return int(load().oracle_num_threads())


def build_part(part_size: int, indptr):
    """-> (part_ptr int32[P+1], part2node int32[P])"""
    lib = load()
    indptr = _i32(indptr)
    n = indptr.size - 1
    p = lib.oracle_build_part(part_size, indptr, n, None, None)
    part_ptr = np.zeros(p + 1, np.int32)
    part2node = np.zeros(p, np.int32)
    lib.oracle_build_part(part_size, indptr, n, part_ptr.ctypes.data, part2node.ctypes.data)
    return part_ptr, part2node


def spmm_groups(inp, col, scale, part_ptr, part2node, num_nodes: int, threads: bool = False):
    """fp32 neighbour-group aggregation -> float32 [N, D]."""
    lib = load()
    inp = _f32(inp)
    dim = inp.shape[1]
    out = np.empty((num_nodes, dim), np.float32)
    fn = lib.oracle_spmm_groups_mt if threads else lib.oracle_spmm_groups
    part2node = _i32(part2node)
    fn(out, inp, _i32(col), _f32(scale), _i32(part_ptr), part2node, part2node.size, num_nodes, dim)
    return out


def spmm_f64(inp, indptr, col, scale):
    """float64 accumulation of the same sum (fp32 edge weights) -> float64 [N, D]."""
    lib = load()
    inp = _f32(inp)
    indptr = _i32(indptr)
    n = indptr.size - 1
    out = np.empty((n, inp.shape[1]), np.float64)
    lib.oracle_spmm_f64(out, inp, indptr, _i32(col), _f32(scale), n, inp.shape[1])
    return out


def mask_forward(part2node, part_ptr, col, src_mask, ngh_mask, back_edge_mask, node_degs, is_last: bool):
    """In-place on ngh_mask (uint8 view), back_edge_mask, node_degs (numpy, contiguous)."""
    lib = load()
    part2node = _i32(part2node)
    assert back_edge_mask.dtype == np.int32 and node_degs.dtype == np.int32
    if ngh_mask is None or ngh_mask.size == 0:
        assert is_last, "an empty ngh_mask is only legal on the last layer"
        ngh_u8 = np.zeros(1, np.uint8)
    else:
        ngh_u8 = ngh_mask.view(np.uint8)
    lib.oracle_mask_forward(part2node, _i32(part_ptr), _i32(col), _u8(src_mask), ngh_u8,
                            back_edge_mask, node_degs, part2node.size, int(is_last))


def compact_mask(edge_mask, column_index):
    """-> (id int32[E], edge_list int32[E], valid_len); tails zero."""
    lib = load()
    edge_mask = _i32(edge_mask)
    out_id = np.zeros_like(edge_mask)
    out_edge = np.zeros_like(edge_mask)
    v = lib.oracle_compact_mask(edge_mask, out_id, _i32(column_index), out_edge, edge_mask.size)
    return out_id, out_edge, int(v)


def compact_count(node_deg) -> int:
    node_deg = _i32(node_deg)
    return int(load().oracle_compact_count(node_deg, node_deg.size))


def split_back_part(node_deg, num_edges: int, part_size: int):
    """compact_part + exclusive_scan as split_back_part composes them
    (EPPGCN/GCNConv/EPPGCN.cpp:327-346) -> (part_pointer int32[num_edges+1], num_parts)."""
    lib = load()
    node_deg = _i32(node_deg)
    part_count = np.zeros(num_edges + 1, np.int32)
    part_pointer = np.zeros(num_edges + 1, np.int32)
    p = lib.oracle_compact_part(node_deg, part_count, node_deg.size, part_size)
    lib.oracle_exclusive_scan(part_count, part_pointer, p)
    return part_pointer, int(p)


def ours_backward(d_out, ids, part_pointer, edge_list, scale, num_parts: int, threads: bool = False):
    lib = load()
    d_out = _f32(d_out)
    n, dim = d_out.shape
    d_in = np.empty_like(d_out)
    fn = lib.oracle_ours_backward_mt if threads else lib.oracle_ours_backward
    fn(d_in, d_out, _i32(ids), _i32(part_pointer), _i32(edge_list), _f32(scale), num_parts, n, dim)
    return d_in


def map_back_part_size(valid_node: int, valid_len: int) -> int:
    return int(load().oracle_map_back_part_size(valid_node, valid_len))


def threshold_back_part_size(valid_node: int, valid_len: int) -> int:
    return int(load().oracle_threshold_back_part_size(valid_node, valid_len))


def get_ginfo(node_deg, valid_len: int):
    node_deg = _i32(node_deg)
    re = np.zeros(10, np.float32)
    load().oracle_get_ginfo(node_deg, node_deg.size, valid_len, re)
    return re


def update_forward(x, w, scale=None, relu_input: bool = False, ld_out: int = None):
    """scale[r] * act(x) @ w with rows ld_out floats apart (zero padded) -> float32 [N, ld_out]."""
    lib = load()
    x, w = _f32(x), _f32(w)
    n, k = x.shape
    m = w.shape[1]
    ld = ld_out or m
    out = np.empty((n, ld), np.float32)
    sc = _f32(scale) if scale is not None else None
    lib.oracle_update_forward(out, ld, x, w, sc.ctypes.data if sc is not None else None, int(relu_input), n, k, m)
    return out


def update_backward_input(g, w, relu_ref=None):
    """(g @ w.T) masked where relu_ref <= 0 -> float32 [N, in_dim]."""
    lib = load()
    g, w = _f32(g), _f32(w)
    n, m = g.shape
    k = w.shape[0]
    d_x = np.empty((n, k), np.float32)
    ref = _f32(relu_ref) if relu_ref is not None else None
    lib.oracle_update_backward_input(d_x, g, w, ref.ctypes.data if ref is not None else None, n, k, m)
    return d_x


def update_backward_weight(x, g, relu_input: bool = False):
    """act(x).T @ g -> float32 [in_dim, out_dim]."""
    lib = load()
    x, g = _f32(x), _f32(g)
    n, k = x.shape
    m = g.shape[1]
    d_w = np.empty((k, m), np.float32)
    lib.oracle_update_backward_weight(d_w, x, g, int(relu_input), n, k, m)
    return d_w
