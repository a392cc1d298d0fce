"""ctypes access to the C ABI of ``libeppgcn_hip.so`` with torch tensors as device memory.

This is the thinnest possible host layer: torch only provides allocations and the
current HIP stream; every computation happens in the library.  Loading fails loudly
when the library has not been built - there is no fallback implementation.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("EPPGCN_HIP_LIB") or os.path.join(_HERE, "lib", "libeppgcn_hip.so")

EXPORTS = [
    "eppgcn_last_error", "eppgcn_abi_version", "eppgcn_feature_workspace_floats", "eppgcn_plan_recommended", "eppgcn_plan_bytes",
    "eppgcn_plan_workspace_bytes", "eppgcn_build_plan", "eppgcn_spmm_forward", "eppgcn_spmm_backward",
    "eppgcn_ours_backward", "eppgcn_mask_forward", "eppgcn_compact_workspace_bytes",
    "eppgcn_split_workspace_bytes", "eppgcn_compact_back_edge", "eppgcn_count_nonzero",
    "eppgcn_map_back_part_size", "eppgcn_threshold_back_part_size", "eppgcn_split_back_part",
    "eppgcn_build_part", "eppgcn_get_ginfo", "eppgcn_set_timing", "eppgcn_print_time",
    "eppgcn_clear_time", "eppgcn_get_time_ms", "eppgcn_set_team_size", "eppgcn_set_rounds", "eppgcn_set_plan_shift", "eppgcn_set_plan_keep_rows",
    "eppgcn_feature_workspace_pitch", "eppgcn_update_forward", "eppgcn_update_backward_input",
    "eppgcn_update_workspace_bytes", "eppgcn_update_backward_weight", "eppgcn_update_supported", "eppgcn_update_backward",
    "eppgcn_mark_compact_workspace_bytes", "eppgcn_mark_compact", "eppgcn_set_plan_length_classes",
    "eppgcn_mark_gathered_rows", "eppgcn_set_wide_index", "eppgcn_wave64_back_part_size",
    "eppgcn_compact_back_edge_static", "eppgcn_compact_back_edge_static_max_length",
    "eppgcn_auto_back_part_size", "eppgcn_scan_status", "eppgcn_plan_status", "eppgcn_set_scan_test_mode",
    "eppgcn_plan_workspace_floats", "eppgcn_set_stream_mode", "eppgcn_last_call_used_stream",
    "eppgcn_update_forward_table", "eppgcn_feature_workspace_row", "eppgcn_plan_release", "eppgcn_aggregation_status",
    "eppgcn_ours_backward_rows", "eppgcn_update_backward_rows",
]

ABI_VERSION = 16      # what eppgcn_abi_version() of a matching library returns

_lib = None


class EppgcnError(RuntimeError):
    pass


def load():
    """Loads the shared library (once).  Raises if it is missing: build it with
    ``python -m eppgcn_amd.build``."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise EppgcnError(f"{LIB_PATH} is missing; run `python -m eppgcn_amd.build` (needs hipcc)")
    lib = C.CDLL(LIB_PATH)
    p, i, i64, sz = C.c_void_p, C.c_int, C.c_int64, C.c_size_t
    lib.eppgcn_last_error.restype = C.c_char_p
    lib.eppgcn_abi_version.restype = i
    if lib.eppgcn_abi_version() != ABI_VERSION:
        raise EppgcnError(f"{LIB_PATH} has ABI version {lib.eppgcn_abi_version()}, this package expects "
                          f"{ABI_VERSION}; rebuild it with `python -m eppgcn_amd.build`")
    lib.eppgcn_feature_workspace_floats.argtypes = [i64, i]
    lib.eppgcn_feature_workspace_floats.restype = sz
    lib.eppgcn_plan_recommended.argtypes = [i64, i]
    lib.eppgcn_plan_recommended.restype = i
    lib.eppgcn_plan_bytes.argtypes = [i64, i64, i64]
    lib.eppgcn_plan_bytes.restype = sz
    lib.eppgcn_plan_workspace_bytes.argtypes = [i64, i64]
    lib.eppgcn_plan_workspace_bytes.restype = sz
    lib.eppgcn_build_plan.argtypes = [p, p, p, p, i, i64, i, i, i, p, sz, p, sz, p]
    lib.eppgcn_build_plan.restype = i
    lib.eppgcn_spmm_forward.argtypes = [p, p, p, p, p, p, p, i, i, i, i, i, i, p, sz, p, p]
    lib.eppgcn_spmm_backward.argtypes = [p, p, p, p, p, p, p, i, i, i, i, i, i, p, sz, p, p]
    lib.eppgcn_ours_backward.argtypes = [p, p, p, p, p, p, i, i, i, i, i, i, i, p, sz, p, p, p]
    lib.eppgcn_mark_gathered_rows.argtypes = [p, i64, i, p, p, C.POINTER(i64), p]
    lib.eppgcn_mark_gathered_rows.restype = i
    lib.eppgcn_mask_forward.argtypes = [p, p, p, p, p, p, p, i, i64, i, i, i, p]
    lib.eppgcn_compact_workspace_bytes.argtypes = [i64]
    lib.eppgcn_compact_workspace_bytes.restype = sz
    lib.eppgcn_split_workspace_bytes.argtypes = [i64]
    lib.eppgcn_split_workspace_bytes.restype = sz
    lib.eppgcn_compact_back_edge.argtypes = [p, p, p, p, i64, p, sz, p, C.POINTER(i64), p]
    lib.eppgcn_compact_back_edge_static.argtypes = [p, p, p, p, i64, p, C.POINTER(i64), p]
    lib.eppgcn_compact_back_edge_static.restype = i
    lib.eppgcn_compact_back_edge_static_max_length.restype = i64
    lib.eppgcn_count_nonzero.argtypes = [p, i64, p, C.POINTER(i64), p]
    lib.eppgcn_map_back_part_size.argtypes = [i64, i64, C.POINTER(i)]
    lib.eppgcn_threshold_back_part_size.argtypes = [i64, i64]
    lib.eppgcn_wave64_back_part_size.argtypes = [i64, i64]
    lib.eppgcn_wave64_back_part_size.restype = i
    lib.eppgcn_auto_back_part_size.argtypes = [i64, i64, C.POINTER(i)]
    lib.eppgcn_auto_back_part_size.restype = i
    lib.eppgcn_scan_status.argtypes = [p, p]
    lib.eppgcn_scan_status.restype = i
    lib.eppgcn_plan_status.argtypes = [p, i, i64, i, C.POINTER(i64), p]
    lib.eppgcn_plan_status.restype = i
    lib.eppgcn_plan_release.argtypes = [p]
    lib.eppgcn_plan_release.restype = None
    lib.eppgcn_aggregation_status.argtypes = [p]
    lib.eppgcn_aggregation_status.restype = i
    lib.eppgcn_plan_workspace_floats.argtypes = [p, i64, i]
    lib.eppgcn_plan_workspace_floats.restype = sz
    lib.eppgcn_set_stream_mode.argtypes = [i]
    lib.eppgcn_set_stream_mode.restype = None
    lib.eppgcn_last_call_used_stream.restype = i
    lib.eppgcn_split_back_part.argtypes = [p, i, i, p, i64, p, sz, p, C.POINTER(i64), C.POINTER(i64), p]
    lib.eppgcn_build_part.argtypes = [p, i, i, p, p, i64, p, sz, p, C.POINTER(i64), p]
    lib.eppgcn_get_ginfo.argtypes = [p, i64, i64, p, C.POINTER(C.c_float), p]
    lib.eppgcn_set_timing.argtypes = [i]
    lib.eppgcn_set_timing.restype = None
    lib.eppgcn_print_time.restype = None
    lib.eppgcn_clear_time.restype = None
    lib.eppgcn_get_time_ms.argtypes = [i]
    lib.eppgcn_get_time_ms.restype = C.c_double
    lib.eppgcn_set_team_size.argtypes = [i]
    lib.eppgcn_set_team_size.restype = None
    lib.eppgcn_set_rounds.argtypes = [i]
    lib.eppgcn_set_rounds.restype = None
    lib.eppgcn_set_scan_test_mode.argtypes = [C.c_uint, i]
    lib.eppgcn_set_scan_test_mode.restype = None
    lib.eppgcn_set_wide_index.argtypes = [i]
    lib.eppgcn_set_wide_index.restype = None
    lib.eppgcn_set_plan_shift.argtypes = [i]
    lib.eppgcn_set_plan_shift.restype = None
    lib.eppgcn_set_plan_length_classes.argtypes = [i]
    lib.eppgcn_set_plan_length_classes.restype = None
    lib.eppgcn_set_plan_keep_rows.argtypes = [i]
    lib.eppgcn_set_plan_keep_rows.restype = None
    lib.eppgcn_mark_compact_workspace_bytes.argtypes = [i64]
    lib.eppgcn_mark_compact_workspace_bytes.restype = sz
    lib.eppgcn_mark_compact.argtypes = [p, p, p, p, p, p, p, p, i, i64, i, p, sz, p, C.POINTER(i64), p]
    lib.eppgcn_mark_compact.restype = i
    lib.eppgcn_feature_workspace_pitch.argtypes = [i]
    lib.eppgcn_feature_workspace_pitch.restype = i
    lib.eppgcn_update_supported.argtypes = [i, i]
    lib.eppgcn_update_supported.restype = i
    lib.eppgcn_update_forward.argtypes = [p, i, p, p, p, i, i64, i, i, p]
    lib.eppgcn_update_forward_table.argtypes = [p, sz, p, p, p, i, i64, i, i, p]
    lib.eppgcn_update_forward_table.restype = i
    lib.eppgcn_feature_workspace_row.argtypes = [i64]
    lib.eppgcn_feature_workspace_row.restype = i64
    lib.eppgcn_update_backward_input.argtypes = [p, p, p, p, i64, i, i, p]
    lib.eppgcn_update_workspace_bytes.argtypes = [i64, i, i]
    lib.eppgcn_update_workspace_bytes.restype = sz
    lib.eppgcn_update_backward_weight.argtypes = [p, p, p, i, i64, i, i, p, sz, p]
    lib.eppgcn_update_backward.argtypes = [p, p, p, p, p, i, i64, i, i, p, sz, p]
    lib.eppgcn_update_backward_rows.argtypes = [p, p, p, p, p, i, p, i64, i, i, p, sz, p]
    lib.eppgcn_ours_backward_rows.argtypes = [p, p, p, p, p, p, i, i, i, i, i, i, i, p, sz, p, p,
                                              C.POINTER(C.c_void_p), C.POINTER(i64), p]
    lib.eppgcn_ours_backward_rows.restype = i
    for name in ("eppgcn_update_forward", "eppgcn_update_backward_input", "eppgcn_update_backward_weight",
                 "eppgcn_update_backward", "eppgcn_update_backward_rows"):
        getattr(lib, name).restype = i
    for name in ("eppgcn_spmm_forward", "eppgcn_spmm_backward", "eppgcn_ours_backward", "eppgcn_mask_forward",
                 "eppgcn_compact_back_edge", "eppgcn_count_nonzero", "eppgcn_map_back_part_size",
                 "eppgcn_threshold_back_part_size", "eppgcn_split_back_part", "eppgcn_build_part",
                 "eppgcn_get_ginfo"):
        getattr(lib, name).restype = i
    _lib = lib
    return lib


def _check(rc: int):
    if rc != 0:
        raise EppgcnError(f"libeppgcn_hip error {rc}: {load().eppgcn_last_error().decode()}")


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, dtype, name):
    if not t.is_cuda:
        raise EppgcnError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise EppgcnError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise EppgcnError(f"{name} must be contiguous")
    return t


def _mask_bytes(t, name):
    if t is None or t.numel() == 0:
        return None
    if t.dtype not in (torch.bool, torch.uint8):
        raise EppgcnError(f"{name} must be bool or uint8")
    if not t.is_cuda or not t.is_contiguous():
        raise EppgcnError(f"{name} must be a contiguous device tensor")
    return t


# --------------------------------------------------------------------------- aggregation
def feature_workspace_pitch(dim: int) -> int:
    """Row pitch (floats) of the pre-scaled feature workspace for `dim`-wide features."""
    return int(load().eppgcn_feature_workspace_pitch(int(dim)))


def update_forward(x, w, scale=None, relu_input=False, ld_out=None, out=None):
    """scale[r] * act(x) @ w as rows ``ld_out`` floats apart (zeros in the padding) -> [N, ld_out]."""
    lib = load()
    _dev(x, torch.float32, "x"); _dev(w, torch.float32, "w")
    n, k = x.shape
    if w.dim() != 2 or w.shape[0] != k:
        raise EppgcnError("w must be [in_dim, out_dim]")
    m = w.shape[1]
    ld = int(ld_out) if ld_out else m
    if scale is not None:
        _dev(scale, torch.float32, "scale")
        if scale.numel() != n:
            raise EppgcnError("scale must have one entry per row")
    if out is None:
        out = torch.empty((n, ld), dtype=torch.float32, device=x.device)
    elif out.numel() < n * ld:
        raise EppgcnError("out is too small")
    _check(lib.eppgcn_update_forward(_ptr(out), ld, _ptr(x), _ptr(w), _ptr(scale), int(bool(relu_input)), n, k, m,
                                     _stream()))
    return out


def update_forward_table(x, w, scale, relu_input=False, table=None, plan=None):
    """scale[r] * act(x) @ w written as the pre-scaled feature workspace of the aggregation calls (their
    ``feats=None`` form): padded rows in the workspace's row order.  ``plan``: leave room for the partial
    sums of that plan's stream form behind the table."""
    lib = load()
    _dev(x, torch.float32, "x"); _dev(w, torch.float32, "w"); _dev(scale, torch.float32, "scale")
    n, k = x.shape
    if w.dim() != 2 or w.shape[0] != k:
        raise EppgcnError("w must be [in_dim, out_dim]")
    m = w.shape[1]
    if scale.numel() != n:
        raise EppgcnError("scale must have one entry per row")
    if table is None:
        table = feature_workspace(n, m, x.device, plan)
    elif table.numel() < lib.eppgcn_feature_workspace_floats(n, m):
        raise EppgcnError("table is too small")
    _check(lib.eppgcn_update_forward_table(_ptr(table), table.numel(), _ptr(x), _ptr(w), _ptr(scale), int(bool(relu_input)), n, k, m,
                                           _stream()))
    return table


def feature_workspace_rows(num_nodes: int, device) -> torch.Tensor:
    """int64[num_nodes]: the row of a separate feature workspace that holds each vertex."""
    r = torch.arange(int(num_nodes), dtype=torch.int64, device=device)
    return r ^ ((r >> 5) & 4095)


def update_backward_input(g, w, relu_ref=None):
    """(g @ w.T), zeroed where relu_ref <= 0 -> [N, in_dim]."""
    lib = load()
    _dev(g, torch.float32, "g"); _dev(w, torch.float32, "w")
    n, m = g.shape
    if w.dim() != 2 or w.shape[1] != m:
        raise EppgcnError("w must be [in_dim, out_dim] with out_dim = g.shape[1]")
    k = w.shape[0]
    if relu_ref is not None:
        _dev(relu_ref, torch.float32, "relu_ref")
        if tuple(relu_ref.shape) != (n, k):
            raise EppgcnError("relu_ref must be [N, in_dim]")
    d_x = torch.empty((n, k), dtype=torch.float32, device=g.device)
    _check(lib.eppgcn_update_backward_input(_ptr(d_x), _ptr(g), _ptr(w), _ptr(relu_ref), n, k, m, _stream()))
    return d_x


def update_backward_weight(x, g, relu_input=False):
    """act(x).T @ g -> [in_dim, out_dim], summed in a fixed order."""
    lib = load()
    _dev(x, torch.float32, "x"); _dev(g, torch.float32, "g")
    n, k = x.shape
    if g.shape[0] != n:
        raise EppgcnError("x and g must have the same number of rows")
    m = g.shape[1]
    d_w = torch.empty((k, m), dtype=torch.float32, device=x.device)
    nbytes = lib.eppgcn_update_workspace_bytes(n, k, m)
    ws = torch.empty(max(1, (nbytes + 3) // 4), dtype=torch.float32, device=x.device)
    _check(lib.eppgcn_update_backward_weight(_ptr(d_w), _ptr(x), _ptr(g), int(bool(relu_input)), n, k, m, _ptr(ws),
                                             nbytes, _stream()))
    return d_w


def update_backward(x, w, g, relu_input=False):
    """Both gradients of a layer ``act(x) @ w`` from the gradient ``g`` of the product, in one call:
    -> (d_x [N, in_dim], d_w [in_dim, out_dim]); the same bits as update_backward_input (with
    ``relu_ref=x`` when ``relu_input``) and update_backward_weight."""
    lib = load()
    _dev(x, torch.float32, "x"); _dev(w, torch.float32, "w"); _dev(g, torch.float32, "g")
    n, k = x.shape
    m = g.shape[1]
    if g.shape[0] != n or tuple(w.shape) != (k, m):
        raise EppgcnError("x [N, in_dim], w [in_dim, out_dim] and g [N, out_dim] are expected")
    d_x = torch.empty((n, k), dtype=torch.float32, device=x.device)
    d_w = torch.empty((k, m), dtype=torch.float32, device=x.device)
    nbytes = lib.eppgcn_update_workspace_bytes(n, k, m)
    ws = torch.empty(max(1, (nbytes + 3) // 4), dtype=torch.float32, device=x.device)
    _check(lib.eppgcn_update_backward(_ptr(d_x), _ptr(d_w), _ptr(x), _ptr(g), _ptr(w), int(bool(relu_input)), n, k, m,
                                      _ptr(ws), nbytes, _stream()))
    return d_x, d_w


def update_backward_rows(x, w, g, rows, relu_input=False, need_dx=True):
    """``update_backward`` for a gradient ``g`` of which only the rows with a set bit in ``rows`` are defined (a
    device int32 bitmap, bit r of word r // 32, or the device address ``ours_backward_rows`` returns, or None for
    all rows): the other rows count as zeros and are not read, nor are their rows of ``x``.
    -> (d_x [N, in_dim] or None when ``need_dx`` is false, d_w [in_dim, out_dim])."""
    lib = load()
    _dev(x, torch.float32, "x"); _dev(g, torch.float32, "g")
    n, k = x.shape
    m = g.shape[1]
    if g.shape[0] != n:
        raise EppgcnError("x and g must have the same number of rows")
    if need_dx:
        _dev(w, torch.float32, "w")
        if tuple(w.shape) != (k, m):
            raise EppgcnError("w must be [in_dim, out_dim]")
    if isinstance(rows, torch.Tensor):
        _dev(rows, torch.int32, "rows")
        if rows.numel() < (n + 31) // 32:
            raise EppgcnError("the row bitmap needs (N + 31) // 32 words")
        rows_ptr = _ptr(rows)
    else:
        rows_ptr = C.c_void_p(rows) if rows else None
    d_x = torch.empty((n, k), dtype=torch.float32, device=x.device) if need_dx else None
    d_w = torch.empty((k, m), dtype=torch.float32, device=x.device)
    nbytes = lib.eppgcn_update_workspace_bytes(n, k, m)
    ws = torch.empty(max(1, (nbytes + 3) // 4), dtype=torch.float32, device=x.device)
    _check(lib.eppgcn_update_backward_rows(_ptr(d_x), _ptr(d_w), _ptr(x), _ptr(g), _ptr(w) if need_dx else None,
                                           int(bool(relu_input)), rows_ptr, n, k, m, _ptr(ws), nbytes, _stream()))
    return d_x, d_w


def _feature_workspace(workspace, feats, plan=None):
    """None -> per-edge scale gather (no scratch); True -> allocate; a tensor -> use it (it may be
    `feats` itself, which is then overwritten with the scaled features)."""
    if workspace is None or workspace is False:
        return None
    if workspace is True:
        return feature_workspace(feats.shape[0], feats.shape[1], feats.device, plan)
    _dev(workspace, torch.float32, "workspace")
    return workspace


def feature_workspace(num_nodes: int, dim: int, device, plan=None):
    """A scratch tensor large enough for the pre-scaled, padded copy of [num_nodes, dim] features and,
    with ``plan``, for the partial sums of a call through the plan's stream form behind it."""
    lib = load()
    floats = lib.eppgcn_feature_workspace_floats(int(num_nodes), int(dim))
    plans = [] if plan is None else [plan] if isinstance(plan, Plan) else list(plan)     # several: room for any of them
    for pl in plans:
        if pl is not None:
            floats = max(floats, lib.eppgcn_plan_workspace_floats(C.c_void_p(pl.base_ptr), int(num_nodes), int(dim)))
    return torch.empty(floats, dtype=torch.float32, device=device)


def last_call_used_stream() -> bool:
    """Whether this thread's last aggregation call ran the stream form of its plan."""
    return bool(load().eppgcn_last_call_used_stream())


def set_stream_mode(on: bool, wide: bool = False):
    """False keeps planned calls on the group kernel (comparisons); True (default) allows the stream form;
    ``wide`` forces the stream kernel's 64-bit addressing variant at any table size (tests)."""
    load().eppgcn_set_stream_mode(2 if (on and wide) else int(bool(on)))


STREAM_WAVE = 512      # slots a wave of the stream kernel takes
STREAM_CHUNK = 32      # piece ends are counted per chunk of this many slots


class Plan:
    """A column-blocked execution plan (device buffer + the sizes it was built for)."""

    def __init__(self, buffer, base_ptr, num_parts, num_slots, num_nodes, partial_rows=0):
        self.buffer, self.base_ptr, self.num_parts, self.num_slots = buffer, base_ptr, num_parts, num_slots
        self.num_nodes = num_nodes
        self.partial_rows = partial_rows      # partial sums of a call through the stream form (0: no stream form)

    def release(self):
        """Tells the library that this plan's memory is given up (it forgets the header it read there)."""
        if self.base_ptr and _lib is not None:
            _lib.eppgcn_plan_release(C.c_void_p(self.base_ptr))
        self.base_ptr = 0

    def __del__(self):
        try:
            self.release()
        except Exception:      # interpreter shutdown
            pass

    @property
    def padded_slots(self):
        return (self.num_slots + STREAM_WAVE - 1) // STREAM_WAVE * STREAM_WAVE

    def _offsets(self):
        def al(x):
            return (x + 255) // 256 * 256
        p = self.num_parts
        off = self.base_ptr - self.buffer.data_ptr()
        o1 = off + al(4 * (p + 1)); o2 = o1 + al(4 * p); o3 = o2 + al(p)
        o4 = o3 + al(4 * ((self.num_nodes + 31) // 32))
        return off, o1, o2, o3, o4

    def view(self, raw_col=False):
        """(ptr, row, flags, col) as torch tensors, for tests.  ``raw_col``: keep bit 31 of the column ids,
        which marks the last slot of every piece."""
        p, s = self.num_parts, self.num_slots
        off, o1, o2, o3, o4 = self._offsets()
        raw = self.buffer.view(torch.uint8)
        col = raw[o4: o4 + 4 * s].view(torch.int32)
        return (raw[off: off + 4 * (p + 1)].view(torch.int32), raw[o1: o1 + 4 * p].view(torch.int32),
                raw[o2: o2 + p], col if raw_col else col & 0x7fffffff)

    def stream_view(self):
        """The stream form as a dict of torch tensors (header, col with padding, erow, cev, wtail, touched, frow,
        fptr), for tests."""
        def al(x):
            return (x + 255) // 256 * 256
        p, n, sp = self.num_parts, self.num_nodes, self.padded_slots
        *_, o4 = self._offsets()
        raw = self.buffer.view(torch.uint8)
        words = (n + 31) // 32
        o = o4 + al(4 * sp)
        out = {"col": raw[o4: o4 + 4 * sp].view(torch.int32), "header": raw[o: o + 64].view(torch.int32)}
        o += al(64)
        for name, count in (("erow", p), ("cev", sp // STREAM_CHUNK + 1), ("wtail", sp // STREAM_WAVE),
                            ("touched", words), ("frow", n), ("fptr", n + 1)):
            out[name] = raw[o: o + 4 * count].view(torch.int32)
            o += al(4 * count)
        return out

    def single_rows(self):
        """bool[num_nodes]: rows recorded as one non-empty group (skipped by the output clear), for tests."""
        _, _, _, o3, _ = self._offsets()
        words = self.buffer.view(torch.uint8)[o3: o3 + 4 * ((self.num_nodes + 31) // 32)].view(torch.int32)
        r = torch.arange(self.num_nodes, device=words.device)
        return ((words[r >> 5] >> (r & 31)) & 1).bool()


def _aligned_buffer(nbytes, device):
    buf = torch.empty(nbytes + 256, dtype=torch.uint8, device=device)
    return buf, (buf.data_ptr() + 255) // 256 * 256


def build_plan(part_ptr, column_index, num_parts: int, num_slots: int, num_nodes: int, dim: int,
               part2node=None, ids=None, block_shift: int = 0):
    """Column-blocked execution plan of the groups; build once per graph and group array and pass it
    as ``plan=`` to the aggregation calls.  Forward groups: give part2node; backward path: give ids.
    ``block_shift``: 0 = blocks sized for the width, n = blocks of 2^n vertices (31: one block)."""
    lib = load()
    _dev(part_ptr, torch.int32, "part_ptr"); _dev(column_index, torch.int32, "column_index")
    if (part2node is None) == (ids is None):
        raise EppgcnError("give exactly one of part2node (forward groups) and ids (backward path)")
    if part_ptr.numel() < num_parts + 1:
        raise EppgcnError("part_ptr needs num_parts + 1 entries")
    if column_index.numel() < num_slots:
        raise EppgcnError("column_index is shorter than num_slots")
    nbytes = lib.eppgcn_plan_bytes(int(num_parts), int(num_slots), int(num_nodes))
    buf, base = _aligned_buffer(nbytes, part_ptr.device)
    wbytes = lib.eppgcn_plan_workspace_bytes(int(num_parts), int(num_slots))
    ws, wbase = _aligned_buffer(wbytes, part_ptr.device)
    _check(lib.eppgcn_build_plan(_ptr(part_ptr), _ptr(column_index), _ptr(part2node), _ptr(ids), int(num_parts),
                                 int(num_slots), int(num_nodes), int(dim), int(block_shift), C.c_void_p(base), nbytes,
                                 C.c_void_p(wbase), wbytes, _stream()))
    # synchronises (the workspace is released on return), refuses a plan whose scan stalled and lets the
    # library know the plan's stream form
    partial = C.c_int64(0)
    _check(lib.eppgcn_plan_status(C.c_void_p(base), int(num_parts), int(num_slots), int(num_nodes), C.byref(partial),
                                  _stream()))
    return Plan(buf, base, int(num_parts), int(num_slots), int(num_nodes), int(partial.value))


def plan_recommended(num_nodes: int, dim: int) -> bool:
    """True when the feature table is too large to stay cached by itself, so a plan pays off."""
    return bool(load().eppgcn_plan_recommended(int(num_nodes), int(dim)))


def _plan_ptr(plan, num_parts, num_nodes):
    if plan is None:
        return None
    if plan.num_parts != num_parts or plan.num_nodes != num_nodes:
        raise EppgcnError("the plan was built for a different number of groups or vertices")
    return C.c_void_p(plan.base_ptr)


def spmm_forward(feats, column_index, degrees, part_ptr, part2node, part_size=32, dim_worker=32,
                 warp_per_block=8, row_pointers=None, out=None, backward=False, workspace=True, plan=None,
                 prescaled_dim=None):
    """out[N, D] = neighbour-group aggregation of feats (``backward=True`` uses the unpruned
    backward entry point; same operator).  ``feats=None`` with ``prescaled_dim=D``: ``workspace``
    already holds the scaled, padded rows (as ``update_forward(..., scale=degrees)`` writes them)."""
    lib = load()
    _dev(column_index, torch.int32, "column_index")
    _dev(degrees, torch.float32, "degrees"); _dev(part_ptr, torch.int32, "part_ptr")
    _dev(part2node, torch.int32, "part2node")
    if feats is None:
        _dev(workspace, torch.float32, "workspace")
        n, dim = degrees.numel(), int(prescaled_dim)
        if out is None:
            out = torch.empty((n, dim), dtype=torch.float32, device=degrees.device)
    else:
        _dev(feats, torch.float32, "feats")
        n, dim = feats.shape
    num_parts = part2node.numel()
    if part_ptr.numel() < num_parts + 1:
        raise EppgcnError("part_ptr needs num_parts + 1 entries")
    if degrees.numel() != n:
        raise EppgcnError("degrees must have one entry per vertex")
    if out is None:
        out = torch.empty_like(feats)
    fn = lib.eppgcn_spmm_backward if backward else lib.eppgcn_spmm_forward
    ws = workspace if feats is None else _feature_workspace(workspace, feats, plan)
    _check(fn(_ptr(out), _ptr(feats), _ptr(row_pointers), _ptr(column_index), _ptr(degrees), _ptr(part_ptr),
              _ptr(part2node), n, dim, num_parts, part_size, dim_worker, warp_per_block, _ptr(ws),
              0 if ws is None else ws.numel(), _plan_ptr(plan, num_parts, n), _stream()))
    return out


def mark_gathered_rows(edge_list, valid_len: int, num_nodes: int):
    """-> (bitmap int32[(N+31)//32] with bit c set for every c in edge_list[:valid_len], number of set bits)."""
    lib = load()
    _dev(edge_list, torch.int32, "edge_list")
    if edge_list.numel() < valid_len:
        raise EppgcnError("edge_list is shorter than valid_len")
    bitmap = torch.empty((int(num_nodes) + 31) // 32 + 1, dtype=torch.int32, device=edge_list.device)
    count = C.c_int64(0)
    _check(lib.eppgcn_mark_gathered_rows(_ptr(edge_list), int(valid_len), int(num_nodes), _ptr(bitmap),
                                         _ptr(bitmap[-1:]), C.byref(count), _stream()))
    return bitmap[:-1], int(count.value)


def ours_backward(d_output, ids, part_pointer, edge_list, degrees, num_parts, part_size=32, layer=1,
                  blockx=4, blocky=16, out=None, workspace=True, plan=None, gathered_rows=None):
    """``gathered_rows``: the bitmap of ``mark_gathered_rows`` for this path, or None."""
    lib = load()
    _dev(d_output, torch.float32, "d_output"); _dev(ids, torch.int32, "ids")
    _dev(part_pointer, torch.int32, "part_pointer"); _dev(edge_list, torch.int32, "edge_list")
    _dev(degrees, torch.float32, "degrees")
    n, dim = d_output.shape
    if part_pointer.numel() < num_parts + 1:
        raise EppgcnError("part_pointer needs num_parts + 1 entries")
    if out is None:
        out = torch.empty_like(d_output)
    ws = _feature_workspace(workspace, d_output, plan)
    _check(lib.eppgcn_ours_backward(_ptr(out), _ptr(d_output), _ptr(ids), _ptr(part_pointer), _ptr(edge_list),
                                    _ptr(degrees), n, dim, int(num_parts), part_size, layer, blockx, blocky,
                                    _ptr(ws), 0 if ws is None else ws.numel(),
                                    _plan_ptr(plan, int(num_parts), n), _ptr(gathered_rows), _stream()))
    return out


def ours_backward_rows(d_output, ids, part_pointer, edge_list, degrees, num_parts, part_size=32, layer=1,
                       blockx=4, blocky=16, out=None, workspace=True, plan=None, gathered_rows=None):
    """``ours_backward`` that leaves the rows without groups as they are when it runs a plan's stream form.
    -> (out, rows, num_written): ``rows`` is the device address of the bitmap of the written rows (inside the
    plan; pass it to ``update_backward_rows``), or None when every row of ``out`` is defined."""
    lib = load()
    _dev(d_output, torch.float32, "d_output"); _dev(ids, torch.int32, "ids")
    _dev(part_pointer, torch.int32, "part_pointer"); _dev(edge_list, torch.int32, "edge_list")
    _dev(degrees, torch.float32, "degrees")
    n, dim = d_output.shape
    if part_pointer.numel() < num_parts + 1:
        raise EppgcnError("part_pointer needs num_parts + 1 entries")
    if out is None:
        out = torch.empty_like(d_output)
    ws = _feature_workspace(workspace, d_output, plan)
    rows, count = C.c_void_p(), C.c_int64()
    _check(lib.eppgcn_ours_backward_rows(_ptr(out), _ptr(d_output), _ptr(ids), _ptr(part_pointer), _ptr(edge_list),
                                         _ptr(degrees), n, dim, int(num_parts), part_size, layer, blockx, blocky,
                                         _ptr(ws), 0 if ws is None else ws.numel(),
                                         _plan_ptr(plan, int(num_parts), n), _ptr(gathered_rows),
                                         C.byref(rows), C.byref(count), _stream()))
    return out, rows.value, count.value


# --------------------------------------------------------------------------- preparation
def mask_forward(part2node, part_ptr, column_index, src_mask, ngh_mask, back_edge_mask, node_degs,
                 is_last_layer: bool, blockx=4, blocky=16):
    lib = load()
    _dev(part2node, torch.int32, "part2node"); _dev(part_ptr, torch.int32, "part_ptr")
    _dev(column_index, torch.int32, "column_index"); _dev(back_edge_mask, torch.int32, "back_edge_mask")
    _dev(node_degs, torch.int32, "node_degs")
    src = _mask_bytes(src_mask, "src_mask")
    ngh = _mask_bytes(ngh_mask, "ngh_mask")
    if src is None:
        raise EppgcnError("src_mask must not be empty")
    _check(lib.eppgcn_mask_forward(_ptr(part2node), _ptr(part_ptr), _ptr(column_index), _ptr(src), _ptr(ngh),
                                   _ptr(back_edge_mask), _ptr(node_degs), part2node.numel(),
                                   column_index.numel(), int(bool(is_last_layer)), blockx, blocky, _stream()))


def _workspace(nbytes: int, device):
    return torch.empty((nbytes + 7) // 8, dtype=torch.int64, device=device)


def compact_back_edge(edge_mask, column_index):
    """-> (id int32[E], edge_list int32[E], valid_len int)"""
    lib = load()
    _dev(edge_mask, torch.int32, "edge_mask"); _dev(column_index, torch.int32, "column_index")
    length = edge_mask.numel()
    if column_index.numel() < length:
        raise EppgcnError("column_index is shorter than edge_mask")
    out_id = torch.empty_like(edge_mask)
    out_edge = torch.empty(length, dtype=torch.int32, device=edge_mask.device)
    nbytes = lib.eppgcn_compact_workspace_bytes(length)
    ws = _workspace(nbytes, edge_mask.device)
    v = C.c_int64(0)
    _check(lib.eppgcn_compact_back_edge(_ptr(edge_mask), _ptr(column_index), _ptr(out_id), _ptr(out_edge), length,
                                        _ptr(ws), nbytes, None, C.byref(v), _stream()))
    return out_id, out_edge, int(v.value)


def compact_back_edge_static_max_length() -> int:
    return int(load().eppgcn_compact_back_edge_static_max_length())


def compact_back_edge_static(edge_mask, column_index, out_id, out_edge, d_valid_len=None, host_count=True):
    """The compaction through the library's static device scratch: the call itself allocates
    nothing, so the caller supplies both output tensors (int32, at least as long as edge_mask).
    -> valid_len (None with ``host_count=False``: the count then only lands in ``d_valid_len``)."""
    lib = load()
    _dev(edge_mask, torch.int32, "edge_mask"); _dev(column_index, torch.int32, "column_index")
    _dev(out_id, torch.int32, "out_id"); _dev(out_edge, torch.int32, "out_edge")
    length = edge_mask.numel()
    if column_index.numel() < length or out_id.numel() < length or out_edge.numel() < length:
        raise EppgcnError("column_index, out_id and out_edge must be at least as long as edge_mask")
    if d_valid_len is not None:
        _dev(d_valid_len, torch.int32, "d_valid_len")
    v = C.c_int64(0)
    _check(lib.eppgcn_compact_back_edge_static(_ptr(edge_mask), _ptr(column_index), _ptr(out_id), _ptr(out_edge), length,
                                               _ptr(d_valid_len), C.byref(v) if host_count else None, _stream()))
    return int(v.value) if host_count else None


def mark_compact(part2node, part_ptr, column_index, src_mask, ngh_mask, node_degs, is_last_layer: bool):
    """Marking and compaction of one layer in one pass -> (id int32[E], edge_list int32[E],
    valid_len); ngh_mask and node_degs are updated in place."""
    lib = load()
    _dev(part2node, torch.int32, "part2node"); _dev(part_ptr, torch.int32, "part_ptr")
    _dev(column_index, torch.int32, "column_index"); _dev(node_degs, torch.int32, "node_degs")
    src = _mask_bytes(src_mask, "src_mask")
    ngh = _mask_bytes(ngh_mask, "ngh_mask")
    if src is None:
        raise EppgcnError("src_mask must not be empty")
    if part_ptr.numel() < part2node.numel() + 1:
        raise EppgcnError("part_ptr needs num_parts + 1 entries")
    length = column_index.numel()
    out_id = torch.empty(length, dtype=torch.int32, device=column_index.device)
    out_edge = torch.empty(length, dtype=torch.int32, device=column_index.device)
    nbytes = lib.eppgcn_mark_compact_workspace_bytes(length)
    ws = _workspace(nbytes, column_index.device)
    v = C.c_int64(0)
    _check(lib.eppgcn_mark_compact(_ptr(part2node), _ptr(part_ptr), _ptr(column_index), _ptr(src), _ptr(ngh),
                                   _ptr(node_degs), _ptr(out_id), _ptr(out_edge), part2node.numel(), length,
                                   int(bool(is_last_layer)), _ptr(ws), nbytes, None, C.byref(v), _stream()))
    return out_id, out_edge, int(v.value)


def count_nonzero(node_deg) -> int:
    lib = load()
    _dev(node_deg, torch.int32, "node_deg")
    d = torch.empty(1, dtype=torch.int32, device=node_deg.device)
    v = C.c_int64(0)
    _check(lib.eppgcn_count_nonzero(_ptr(node_deg), node_deg.numel(), _ptr(d), C.byref(v), _stream()))
    return int(v.value)


def map_back_part_size(valid_node: int, valid_len: int):
    """-> (group size >= 1, clamped flag)"""
    c = C.c_int(0)
    ps = load().eppgcn_map_back_part_size(int(valid_node), int(valid_len), C.byref(c))
    return int(ps), bool(c.value)


def threshold_back_part_size(valid_node: int, valid_len: int) -> int:
    return int(load().eppgcn_threshold_back_part_size(int(valid_node), int(valid_len)))


def wave64_back_part_size(valid_node: int, valid_len: int) -> int:
    """The group-size rule re-fitted for this library's kernels (16 or 32)."""
    return int(load().eppgcn_wave64_back_part_size(int(valid_node), int(valid_len)))


def auto_back_part_size(valid_node: int, valid_len: int):
    """The reference's `map` mode made safe for large paths -> (group size, fell_back): the fitted
    regression while it gives at least 1, the wave64 rule otherwise."""
    c = C.c_int(0)
    ps = load().eppgcn_auto_back_part_size(int(valid_node), int(valid_len), C.byref(c))
    return int(ps), bool(c.value)


def scan_status(workspace) -> None:
    """Raises if the last scan-based call over ``workspace`` stalled or overflowed (synchronises).
    ``None``: the static scratch of ``compact_back_edge_static`` on the current device."""
    _check(load().eppgcn_scan_status(_ptr(workspace), _stream()))


def aggregation_status() -> None:
    """Raises (once) if the stream or fix-up kernel of an aggregation call found a plan header in memory
    that was not the one ``build_plan`` left there (synchronises)."""
    _check(load().eppgcn_aggregation_status(_stream()))


def split_back_part(node_deg, num_edges: int, part_size: int):
    """-> (part_pointer int32[num_edges + 1], num_parts int, valid_len int)"""
    lib = load()
    _dev(node_deg, torch.int32, "node_deg")
    n = node_deg.numel()
    capacity = int(num_edges) + 1
    part_pointer = torch.empty(capacity, dtype=torch.int32, device=node_deg.device)
    nbytes = lib.eppgcn_split_workspace_bytes(n)
    ws = _workspace(nbytes, node_deg.device)
    p, v = C.c_int64(0), C.c_int64(0)
    _check(lib.eppgcn_split_back_part(_ptr(node_deg), n, int(part_size), _ptr(part_pointer), capacity, _ptr(ws),
                                      nbytes, None, C.byref(p), C.byref(v), _stream()))
    return part_pointer, int(p.value), int(v.value)


def build_part(part_size: int, row_pointers, num_edges: int = None):
    """Device build of the forward groups -> (part_ptr int32[P+1], part2node int32[P])"""
    lib = load()
    _dev(row_pointers, torch.int32, "row_pointers")
    n = row_pointers.numel() - 1
    if num_edges is None:
        num_edges = int(row_pointers[-1].item()) - int(row_pointers[0].item())
    capacity = num_edges // int(part_size) + n + 1
    part_ptr = torch.empty(capacity, dtype=torch.int32, device=row_pointers.device)
    part2node = torch.empty(max(capacity - 1, 1), dtype=torch.int32, device=row_pointers.device)
    nbytes = lib.eppgcn_split_workspace_bytes(n)
    ws = _workspace(nbytes, row_pointers.device)
    p = C.c_int64(0)
    _check(lib.eppgcn_build_part(_ptr(row_pointers), n, int(part_size), _ptr(part_ptr), _ptr(part2node), capacity,
                                 _ptr(ws), nbytes, None, C.byref(p), _stream()))
    np_ = int(p.value)
    return part_ptr[: np_ + 1], part2node[:np_]


def get_ginfo(node_deg, valid_len: int):
    lib = load()
    _dev(node_deg, torch.int32, "node_deg")
    hist = torch.empty(10, dtype=torch.int32, device=node_deg.device)
    out = (C.c_float * 10)()
    _check(lib.eppgcn_get_ginfo(_ptr(node_deg), node_deg.numel(), int(valid_len), _ptr(hist), out, _stream()))
    return torch.tensor(list(out), dtype=torch.float32)


# --------------------------------------------------------------------------- timers / tuning
def set_timing(enabled: bool):
    load().eppgcn_set_timing(int(bool(enabled)))


def print_time():
    load().eppgcn_print_time()


def clear_time():
    load().eppgcn_clear_time()


def get_time_ms(which: int) -> float:
    return float(load().eppgcn_get_time_ms(which))


def set_team_size(lanes: int):
    load().eppgcn_set_team_size(int(lanes))


def set_rounds(rounds: int):
    load().eppgcn_set_rounds(int(rounds))


def set_wide_index(on: bool):
    """Forces the 64-bit instantiations of the clear and pre-scaling kernels (for tests)."""
    load().eppgcn_set_wide_index(int(bool(on)))


def set_scan_test_mode(spin_limit: int = 0, mute_first_tile: bool = False):
    """Test knob: bounded look-back waits that are certain to give up (see the header); (0, False) = normal."""
    load().eppgcn_set_scan_test_mode(int(spin_limit), int(bool(mute_first_tile)))


def set_plan_length_classes(on):
    """True / False, or None: chosen per build from the kernel that will run over the plan (the default)."""
    load().eppgcn_set_plan_length_classes(-1 if on is None else int(bool(on)))


def set_plan_shift(shift: int):
    load().eppgcn_set_plan_shift(int(shift))


def set_plan_keep_rows(groups):
    """Rows of up to 32 * groups slots stay together; None: chosen per build (the default)."""
    load().eppgcn_set_plan_keep_rows(-1 if groups is None else int(groups))
