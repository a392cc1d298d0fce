"""The allocation-free compaction entry point (static device scratch inside the library) against
the workspace-based entry point it is a variant of, through the C ABI.  Integer work: bit-exact."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("needs the MI355X")
    from eppgcn_amd import capi
    capi.load()
    # the documented first call on the device: looks up the static scratch's address (what it reports is the
    # status of whichever call used the scratch last, possibly another test's forced stall: not looked at here)
    capi.load().eppgcn_scan_status(None, None)
    return capi, torch


def _inputs(torch, length, density, seed):
    rng = np.random.default_rng(seed)
    keep = rng.random(length) < density
    rows = np.sort(rng.integers(0, max(length // 7, 1), length)).astype(np.int32)
    mask = np.where(keep, rows, -1).astype(np.int32)
    col = rng.integers(0, 1 << 30, length).astype(np.int32)
    dev = torch.device("cuda:0")
    return torch.from_numpy(mask).to(dev), torch.from_numpy(col).to(dev), int(keep.sum())


def _compare(capi, torch, length, density, seed, out_id, out_edge, d_count):
    mask, col, kept = _inputs(torch, length, density, seed)
    want_id, want_edge, want_v = capi.compact_back_edge(mask, col)        # caller workspace
    out_id.fill_(-7)
    out_edge.fill_(-7)
    d_count.fill_(-7)
    torch.cuda.synchronize()
    free_before, held_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    got_v = capi.compact_back_edge_static(mask, col, out_id, out_edge, d_valid_len=d_count)
    # the call allocates nothing: neither from the device (hipMemGetInfo) nor from torch's pool
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_allocated() == held_before
    assert got_v == want_v == kept
    assert int(d_count.item()) == kept
    assert torch.equal(out_id[:length], want_id), "row ids differ (zero tail included)"
    assert torch.equal(out_edge[:length], want_edge), "column ids differ (zero tail included)"
    # entries beyond the input length are not the call's to touch
    assert bool((out_id[length:] == -7).all()) and bool((out_edge[length:] == -7).all())


def test_static_scratch_compaction_two_calls_in_a_row_second_one_smaller(api):
    capi, torch = api
    dev = torch.device("cuda:0")
    big, small = (1 << 22) + 12345, 70001         # 1027 tiles, then 18 tiles of the same scratch
    out_id = torch.empty(big + 64, dtype=torch.int32, device=dev)
    out_edge = torch.empty(big + 64, dtype=torch.int32, device=dev)
    d_count = torch.empty(1, dtype=torch.int32, device=dev)
    _compare(capi, torch, big, 0.37, 11, out_id, out_edge, d_count)
    _compare(capi, torch, small, 0.81, 12, out_id, out_edge, d_count)
    # and further sizes over the same array, including empty, all kept, none kept, one tile exactly
    for length, density, seed in [(0, 0.5, 13), (1, 1.0, 14), (4096, 1.0, 15), (4097, 0.0, 16), (300000, 0.05, 17),
                                  (big, 0.9, 18), (63, 0.5, 19)]:
        _compare(capi, torch, length, density, seed, out_id, out_edge, d_count)


def test_static_scratch_compaction_without_a_host_count(api):
    """The asynchronous form: the count only lands in device memory; nothing synchronises."""
    capi, torch = api
    dev = torch.device("cuda:0")
    length = 123457
    mask, col, kept = _inputs(torch, length, 0.25, 21)
    out_id = torch.empty(length, dtype=torch.int32, device=dev)
    out_edge = torch.empty(length, dtype=torch.int32, device=dev)
    d_count = torch.zeros(1, dtype=torch.int32, device=dev)
    assert capi.compact_back_edge_static(mask, col, out_id, out_edge, d_valid_len=d_count, host_count=False) is None
    want_id, want_edge, want_v = capi.compact_back_edge(mask, col)
    capi.scan_status(None)           # the status of the static scratch: no stall, nothing raised
    assert int(d_count.item()) == kept == want_v
    assert torch.equal(out_id, want_id) and torch.equal(out_edge, want_edge)


def test_static_scratch_compaction_rejects_what_the_scratch_cannot_hold(api):
    capi, torch = api
    lib = capi.load()
    limit = capi.compact_back_edge_static_max_length()
    assert limit == 1 << 30
    one = ctypes.c_void_p(256)       # non-null, never dereferenced: the size check comes first
    rc = lib.eppgcn_compact_back_edge_static(one, one, one, one, limit + 1, None, None, None)
    assert rc == -4 and b"exceeds the static scratch" in lib.eppgcn_last_error()
    assert lib.eppgcn_compact_back_edge_static(one, one, one, one, -1, None, None, None) == -1
    assert lib.eppgcn_compact_back_edge_static(None, one, one, one, 5, None, None, None) == -1
