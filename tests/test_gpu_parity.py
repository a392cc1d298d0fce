"""GPU parity: every entry point of the C ABI (through ctypes) against the CPU checker.

Bars: integer outputs (group pointers, path marking, compacted lists, counts) bit-exact;
aggregation outputs within rel. tol. 1e-5 of the float64 sum, the tolerance being taken
relative to sum_j |w_ij x_j| per output element (summation-order differences only)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import closed_forms as cf
from tests.helpers import hub_csr, random_symmetric_csr, scale_inv_sqrt, scale_sqrt

pytestmark = pytest.mark.gpu
RTOL = 1e-5


@pytest.fixture(scope="module")
def api():
    from eppgcn_amd import capi
    capi.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return capi


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def assert_close(got, want64, bound, what=""):
    err = np.abs(got.astype(np.float64) - want64)
    lim = RTOL * bound + 1e-30
    worst = float(np.max(err / lim)) if err.size else 0.0
    assert worst <= 1.0, f"{what}: max err/limit = {worst:.3f}"


GRAPHS = {
    "single": lambda: random_symmetric_csr(1, 0, 0),
    "tiny": lambda: random_symmetric_csr(7, 9, 2),
    "small": lambda: random_symmetric_csr(130, 260, 5),
    "isolated": lambda: random_symmetric_csr(3000, 9000, 11, isolated=0.3),
    "hub": lambda: hub_csr(5000, 4000, 7),
    "medium": lambda: random_symmetric_csr(20000, 150000, 13),
}


# ----------------------------------------------------------------------------- build_part
@pytest.mark.parametrize("name", list(GRAPHS))
@pytest.mark.parametrize("ps", [1, 3, 8, 32, 5000])
def test_build_part_bit_exact(api, name, ps):
    indptr, col = GRAPHS[name]()
    want_pp, want_p2n = co.build_part(ps, indptr)
    pp, p2n = api.build_part(ps, dev(indptr), col.size)
    assert np.array_equal(pp.cpu().numpy(), want_pp)
    assert np.array_equal(p2n.cpu().numpy(), want_p2n)


# ----------------------------------------------------------------------------- mask_forward
@pytest.mark.parametrize("name", ["tiny", "small", "isolated", "hub", "medium"])
@pytest.mark.parametrize("ratio", [0.0, 0.1, 0.5, 1.0])
@pytest.mark.parametrize("ps", [1, 5, 32, 200])
def test_mask_forward_bit_exact(api, name, ratio, ps):
    indptr, col = GRAPHS[name]()
    n, e = indptr.size - 1, col.size
    rng = np.random.default_rng(int(ratio * 100) + ps)
    src = rng.random(n) < ratio
    pre_ngh = rng.random(n) < 0.02
    pre_degs = rng.integers(0, 3, n).astype(np.int32)
    pp, p2n = co.build_part(ps, indptr)
    for is_last in (False, True):
        want = cf.mask_forward(indptr, col, src, pre_ngh, np.full(e, -1, np.int32), pre_degs, is_last)
        ngh = dev(pre_ngh)
        bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
        degs = dev(pre_degs)
        api.mask_forward(dev(p2n), dev(pp), dev(col), dev(src), None if is_last else ngh, bem, degs, is_last)
        assert np.array_equal(bem.cpu().numpy(), want[1])
        assert np.array_equal(degs.cpu().numpy(), want[2])
        assert np.array_equal(ngh.cpu().numpy(), want[0] if not is_last else pre_ngh)


# ----------------------------------------------------------------------------- compaction
@pytest.mark.parametrize("length", [0, 1, 63, 64, 65, 4095, 4096, 4097, 100000, 1 << 20, (1 << 22) + 12345])
@pytest.mark.parametrize("density", [0.0, 0.1, 0.5, 1.0])
def test_compact_back_edge_bit_exact(api, length, density):
    rng = np.random.default_rng(length % 9973 + int(density * 10))
    em = np.where(rng.random(length) < density, rng.integers(0, 1 << 20, length), -1).astype(np.int32)
    col = rng.integers(0, 1 << 20, length).astype(np.int32)
    want_id, want_edge, want_v = cf.compact_mask(em, col)
    oid, oedge, v = api.compact_back_edge(dev(em), dev(col))
    assert v == want_v
    assert np.array_equal(oid.cpu().numpy(), want_id)
    assert np.array_equal(oedge.cpu().numpy(), want_edge)


@pytest.mark.parametrize("shift", [1, 2, 3])
@pytest.mark.parametrize("length", [1, 4095, 16384, 16385, 70001])
def test_compact_back_edge_unaligned_arrays(api, length, shift):
    """Arrays that start at any 4-byte boundary (views into larger buffers); lengths around the kernel's tile of
    16384 items."""
    rng = np.random.default_rng(length + shift)
    em = np.where(rng.random(length + shift) < 0.4, rng.integers(0, 1 << 20, length + shift), -1).astype(np.int32)
    col = rng.integers(0, 1 << 20, length + shift).astype(np.int32)
    want_id, want_edge, want_v = cf.compact_mask(em[shift:], col[shift:])
    for a, b in ((dev(em)[shift:], dev(col)[shift:]), (dev(em[shift:]), dev(col)[shift:]), (dev(em)[shift:], dev(col[shift:]))):
        oid, oedge, v = api.compact_back_edge(a, b)
        assert v == want_v
        assert np.array_equal(oid.cpu().numpy(), want_id) and np.array_equal(oedge.cpu().numpy(), want_edge)


def test_compact_is_deterministic_across_runs(api):
    rng = np.random.default_rng(5)
    length = 3_000_000
    em = np.where(rng.random(length) < 0.3, rng.integers(0, 1000, length), -1).astype(np.int32)
    col = rng.integers(0, 1000, length).astype(np.int32)
    dem, dcol = dev(em), dev(col)
    first = api.compact_back_edge(dem, dcol)
    for _ in range(5):
        again = api.compact_back_edge(dem, dcol)
        assert again[2] == first[2]
        assert torch.equal(again[0], first[0]) and torch.equal(again[1], first[1])


# ----------------------------------------------------------------------------- split / counts
@pytest.mark.parametrize("n", [1, 5, 2047, 2048, 2049, 100000, 1 << 20])
@pytest.mark.parametrize("ps", [1, 2, 8, 32, 64])
def test_split_back_part_bit_exact(api, n, ps):
    rng = np.random.default_rng(n % 1000 + ps)
    degs = (rng.integers(0, 40, n) * (rng.random(n) < 0.6)).astype(np.int32)
    if n > 10:
        degs[n // 3] = 70000          # far more than 1023 groups for one vertex
    e = int(degs.sum()) + 17
    want_pp, want_p = cf.split_back_part(degs, e, ps)
    pp, p, v = api.split_back_part(dev(degs), e, ps)
    assert p == want_p and v == int(degs.sum())
    assert np.array_equal(pp.cpu().numpy(), want_pp)
    assert api.count_nonzero(dev(degs)) == cf.compact_count(degs)


def test_split_all_zero_and_capacity_error(api):
    degs = np.zeros(5000, np.int32)
    pp, p, v = api.split_back_part(dev(degs), 100, 8)
    assert p == 0 and v == 0 and not pp.cpu().numpy().any()
    degs[:] = 3
    with pytest.raises(api.EppgcnError):
        api.split_back_part(dev(degs), 100, 1)     # 15000 groups cannot fit 101 entries


def test_scan_status_reports_what_asynchronous_calls_cannot(api):
    """With every count taken on the device (no h_* argument) the scan-based calls return before the
    device has run; eppgcn_scan_status is how such a caller learns of a capacity overflow."""
    import ctypes as C
    lib = api.load()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: C.c_void_p(t.data_ptr())
    n = 50000
    degs = torch.full((n,), 3, dtype=torch.int32, device="cuda")
    nbytes = lib.eppgcn_split_workspace_bytes(n)
    ws = torch.empty((nbytes + 7) // 8, dtype=torch.int64, device="cuda")
    counts = torch.zeros(2, dtype=torch.int32, device="cuda")
    roomy = torch.empty(3 * n + 1, dtype=torch.int32, device="cuda")
    assert lib.eppgcn_split_back_part(ptr(degs), n, 1, ptr(roomy), roomy.numel(), ptr(ws), nbytes, ptr(counts),
                                      None, None, stream) == 0
    assert lib.eppgcn_scan_status(ptr(ws), stream) == 0
    assert counts.tolist() == [3 * n, 3 * n] and int(roomy[-1]) == 3 * n
    tight = torch.empty(n, dtype=torch.int32, device="cuda")             # 3n + 1 entries are needed
    assert lib.eppgcn_split_back_part(ptr(degs), n, 1, ptr(tight), tight.numel(), ptr(ws), nbytes, ptr(counts),
                                      None, None, stream) == 0
    assert lib.eppgcn_scan_status(ptr(ws), stream) == -4 and b"capacity" in lib.eppgcn_last_error()
    # a compaction that took its count on the device only
    mask = torch.where(torch.arange(100000, device="cuda") % 3 == 0, 7, -1).int()
    col = torch.arange(100000, dtype=torch.int32, device="cuda")
    oid, oedge = torch.empty_like(mask), torch.empty_like(col)
    cbytes = lib.eppgcn_compact_workspace_bytes(mask.numel())
    cws = torch.empty((cbytes + 7) // 8, dtype=torch.int64, device="cuda")
    kept = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert lib.eppgcn_compact_back_edge(ptr(mask), ptr(col), ptr(oid), ptr(oedge), mask.numel(), ptr(cws), cbytes,
                                        ptr(kept), None, stream) == 0
    assert lib.eppgcn_scan_status(ptr(cws), stream) == 0 and int(kept) == 33334
    assert torch.equal(oedge[:33334], col[::3])


def test_stalled_scans_are_reported_and_the_kernels_still_finish(api):
    """Failure handling of the look-back scans, forced from the host: tile 0 keeps its result to itself and
    the spin limit is tiny, so every waiting tile gives up after a few polls, flags the stall and goes on -
    no kernel hangs, and every call that reads the status reports EPPGCN_ERR_SCAN_STALLED (-3)."""
    import ctypes as C
    lib = api.load()
    n = 300000
    mask = torch.where(torch.arange(n, device="cuda") % 3 == 0, 5, -1).int()
    col = torch.arange(n, dtype=torch.int32, device="cuda")
    degs = torch.full((n,), 2, dtype=torch.int32, device="cuda")
    indptr, cols = GRAPHS["medium"]()
    pp, p2n = co.build_part(4, indptr)
    api.set_scan_test_mode(8, True)
    try:
        for call in (lambda: api.compact_back_edge(mask, col), lambda: api.split_back_part(degs, 2 * n, 1),
                     lambda: api.build_part(2, dev(indptr)),
                     lambda: api.build_plan(dev(pp), dev(cols), p2n.size, cols.size, indptr.size - 1, 16, part2node=dev(p2n)),
                     lambda: api.compact_back_edge_static(mask, col, torch.empty_like(mask), torch.empty_like(col))):
            with pytest.raises(api.EppgcnError, match="-3"):
                call()
        # the asynchronous form returns 0; the status call tells
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        nbytes = lib.eppgcn_compact_workspace_bytes(n)
        ws = torch.empty((nbytes + 7) // 8, dtype=torch.int64, device="cuda")
        oid, oedge = torch.empty_like(mask), torch.empty_like(col)
        kept = torch.zeros(1, dtype=torch.int32, device="cuda")
        p = lambda t: C.c_void_p(t.data_ptr())
        assert lib.eppgcn_compact_back_edge(p(mask), p(col), p(oid), p(oedge), n, p(ws), nbytes, p(kept), None, stream) == 0
        assert lib.eppgcn_scan_status(p(ws), stream) == -3 and b"stalled" in lib.eppgcn_last_error()
    finally:
        api.set_scan_test_mode(0, False)
    oid, oedge, v = api.compact_back_edge(mask, col)          # and normal operation is back
    assert v == 100000 and torch.equal(oedge[:v], col[::3])


def test_heuristics_and_ginfo(api):
    for vn, vl in [(1000, 5000), (100000, 1000000), (419000, 13_400_000), (7, 7)]:
        ps, clamped = api.map_back_part_size(vn, vl)
        raw = cf.map_back_part_size(vn, vl)
        assert ps == max(raw, 1) and clamped == (raw < 1)
        assert api.threshold_back_part_size(vn, vl) == cf.threshold_back_part_size(vn, vl)
    assert api.map_back_part_size(1_000_000, 100_000_000) == (1, True)   # raw value is negative
    rng = np.random.default_rng(1)
    degs = (rng.integers(0, 300, 100000) * (rng.random(100000) < 0.7)).astype(np.int32)
    got = api.get_ginfo(dev(degs), 12345).numpy()
    assert np.allclose(got, cf.get_ginfo(degs, 12345), rtol=1e-6)


# ----------------------------------------------------------------------------- aggregation
def _forward_case(api, indptr, col, s, x, ps, what):
    n = indptr.size - 1
    pp, p2n = co.build_part(ps, indptr)
    want = co.spmm_f64(x, indptr, col, s)
    bound = cf.abs_sum_bound(indptr, col, s, x)
    dx = dev(x)
    # three scale modes: per-edge gather (no scratch), scratch workspace, workspace aliasing the input
    plain = api.spmm_forward(dx, dev(col), dev(s), dev(pp), dev(p2n), part_size=ps, workspace=None).cpu().numpy()
    assert_close(plain, want, bound, what + " [no workspace]")
    got = api.spmm_forward(dx, dev(col), dev(s), dev(pp), dev(p2n), part_size=ps, workspace=True).cpu().numpy()
    assert_close(got, want, bound, what + " [workspace]")
    assert np.array_equal(dx.cpu().numpy(), x), "a separate workspace must leave the input untouched"
    alias = api.spmm_forward(dx, dev(col), dev(s), dev(pp), dev(p2n), part_size=ps, workspace=dx).cpu().numpy()
    assert_close(alias, want, bound, what + " [aliased workspace]")
    assert np.array_equal(dx.cpu().numpy(), (s[:, None] * x).astype(np.float32)), "aliased input holds s*x"
    return got


@pytest.mark.parametrize("name", list(GRAPHS))
@pytest.mark.parametrize("dim", [16, 22])
@pytest.mark.parametrize("ps", [1, 4, 32, 700])
def test_forward_aggregation_headline_widths(api, name, dim, ps):
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    rng = np.random.default_rng(dim + ps)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    for scale_fn in (scale_inv_sqrt, scale_sqrt):
        s = scale_fn(indptr)
        got = _forward_case(api, indptr, col, s, x, ps, f"{name} D={dim} ps={ps}")
        # the fp32 restatement of the reference's rounding model agrees to the same tolerance
        pp, p2n = co.build_part(ps, indptr)
        ref32 = co.spmm_groups(x, col, s, pp, p2n, n)
        assert_close(got, ref32.astype(np.float64), 2 * cf.abs_sum_bound(indptr, col, s, x), "vs fp32 restatement")


@pytest.mark.parametrize("dim", [1, 2, 3, 4, 6, 8, 12, 31, 32, 64, 96, 100, 128, 250, 256, 300, 512, 1030, 1100])
def test_forward_aggregation_every_width_class(api, dim):
    indptr, col = hub_csr(1500, 1200, 3)
    n = indptr.size - 1
    x = np.random.default_rng(dim).standard_normal((n, dim)).astype(np.float32)
    s = scale_inv_sqrt(indptr)
    for ps in (7, 64):
        _forward_case(api, indptr, col, s, x, ps, f"D={dim} ps={ps}")


@pytest.mark.parametrize("team", [4, 8, 16, 32, 64])
@pytest.mark.parametrize("dim", [16, 22, 64])
def test_forward_aggregation_forced_team_sizes(api, team, dim):
    indptr, col = hub_csr(4000, 3000, 9)
    n = indptr.size - 1
    x = np.random.default_rng(team + dim).standard_normal((n, dim)).astype(np.float32)
    s = scale_inv_sqrt(indptr)
    try:
        api.set_team_size(team)
        for ps in (3, 32):
            _forward_case(api, indptr, col, s, x, ps, f"team={team} D={dim} ps={ps}")
    finally:
        api.set_team_size(0)


@pytest.mark.parametrize("rounds", [1, 2, 3, 7, 64])
@pytest.mark.parametrize("dim", [16, 22, 64, 256])
def test_forward_and_pruned_forced_rounds_exact_integer_sums(api, rounds, dim):
    """Waves that process several consecutive group rounds carry a row's partial sum from one
    round to the next: with s == 1 and small integer features the result must still be exactly
    the neighbour sum, for rows shorter than a group and rows spanning many rounds and waves."""
    indptr, col = hub_csr(3000, 2500, 17)
    n = indptr.size - 1
    x = np.random.default_rng(rounds).integers(-8, 9, (n, dim)).astype(np.float32)
    s = np.ones(n, np.float32)
    want = np.zeros((n, dim), np.float64)
    np.add.at(want, cf.row_index(indptr), x[col].astype(np.float64))
    src = np.random.default_rng(3).random(n) < 0.4
    want_b = np.zeros((n, dim), np.float64)
    keep = src[col]
    np.add.at(want_b, cf.row_index(indptr)[keep], (x * src[:, None])[col[keep]].astype(np.float64))
    try:
        api.set_rounds(rounds)
        for ps in (1, 2, 9, 32):
            pp, p2n = co.build_part(ps, indptr)
            for ws in (None, True):
                got = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=ps, workspace=ws)
                assert np.array_equal(got.cpu().numpy().astype(np.float64), want), f"ps={ps} ws={ws}"
            oid, oedge, bpp, p = _gpu_path(api, indptr, col, src, 5, ps)
            dy = dev((x * src[:, None]).astype(np.float32))
            gb = api.ours_backward(dy, oid, bpp, oedge, dev(s), p, part_size=ps)
            assert np.array_equal(gb.cpu().numpy().astype(np.float64), want_b), f"pruned ps={ps}"
    finally:
        api.set_rounds(0)


@pytest.mark.parametrize("name", ["tiny", "small", "isolated", "hub", "medium"])
@pytest.mark.parametrize("ps", [1, 5, 32])
def test_plan_is_a_stable_column_block_reordering(api, name, ps):
    """The execution plan must hold every group exactly once, ordered by the column block of its
    first slot with the original order kept inside a block, with rows, column ids and adjacency
    flags that describe the original groups."""
    indptr, col = GRAPHS[name]()
    # default block sizes (one block for these small graphs at width 16) and forced small blocks; blocks of
    # 4 vertices make sort keys of up to 15 bits, i.e. two passes of the radix sort
    _check_plan_order(api, indptr, col, ps, ((16, 0), (256, 0), (16, 9), (16, 12), (16, 2)))


def test_plan_sort_with_three_radix_passes(api):
    """300 000 vertices in blocks of 2: 18 block bits + 2 class bits = three 8-bit passes, the last of
    which has to land in the final buffer; ties must stay in group order."""
    indptr, col = random_symmetric_csr(300000, 500000, 29)
    _check_plan_order(api, indptr, col, 16, ((16, 1), (16, 5)))


def _check_plan_order(api, indptr, col, ps, cases):
    # the defaults (rows of up to 64 slots together, no length classes: the stream form's optimum) and the
    # group kernel's optimum (256 slots, length classes)
    for keep, classes in ((2, False), (8, True)):
        api.set_plan_keep_rows(keep)
        api.set_plan_length_classes(classes)
        try:
            _check_plan_order_with(api, indptr, col, ps, cases, 32 * keep, classes)
        finally:
            api.set_plan_keep_rows(None)
            api.set_plan_length_classes(None)


def _check_plan_order_with(api, indptr, col, ps, cases, keep_slots, classes):
    n = indptr.size - 1
    pp, p2n = co.build_part(ps, indptr)
    P = p2n.size
    for dim, forced in cases:
        api.set_plan_shift(forced)
        try:
            plan = api.build_plan(dev(pp), dev(col), P, col.size, n, dim, part2node=dev(p2n))
        finally:
            api.set_plan_shift(0)
        ptr, row, flags, pcol = [t.cpu().numpy() for t in plan.view()]
        assert ptr[0] == 0 and ptr[-1] == col.size and np.all(np.diff(ptr) >= 1)
        # identify every plan entry with its original group: same row, same size, same columns;
        # the first column and the row identify a group uniquely
        first = {(int(p2n[p]), int(col[pp[p]])): p for p in range(P)}
        order = np.array([first[(int(row[q]), int(pcol[ptr[q]]))] for q in range(P)])
        assert np.array_equal(np.sort(order), np.arange(P))
        for q in (0, P // 3, P // 2, P - 1):
            p = order[q]
            assert np.array_equal(pcol[ptr[q]:ptr[q + 1]], col[pp[p]:pp[p + 1]])
        sizes = np.diff(pp)[order]
        assert np.array_equal(np.diff(ptr), sizes)
        # sort key: column block of the group's first slot; rows of at most keep_slots slots (in at most 64
        # groups) use the key of their first group so that they stay together
        groups_per_row = np.bincount(p2n, minlength=n)
        row_first_group = np.concatenate([[0], np.cumsum(groups_per_row)[:-1]])
        short = (groups_per_row <= 64) & (np.diff(indptr) <= keep_slots)
        key_col = np.where(short[p2n], col[pp[row_first_group[p2n]]], col[pp[:-1]])[order]
        # second key (optional): length class (steps of 8 slots) of short rows that are a single group, 3 for the rest
        cls = np.where((groups_per_row[p2n] == 1) & short[p2n], np.minimum(3, (np.diff(pp) - 1) >> 3), 3)[order]
        if not classes:
            cls = np.zeros_like(cls)
        ok = False
        for shift in ([forced] if forced else range(8, 18)):
            keys = ((key_col >> shift) << 2) | cls
            if np.all(np.diff(keys) >= 0) and np.all((np.diff(keys) > 0) | (np.diff(order) > 0)):
                ok = True
        assert ok, "not ordered by (power-of-two column block, length class) with stable ties"
        prev = np.concatenate([[False], p2n[1:] == p2n[:-1]])[order]
        nxt = np.concatenate([p2n[1:] == p2n[:-1], [False]])[order]
        jl = prev & np.concatenate([[False], order[1:] == order[:-1] + 1])
        jr = nxt & np.concatenate([order[1:] == order[:-1] + 1, [False]])
        assert np.array_equal(flags & 1, prev) and np.array_equal((flags >> 1) & 1, nxt)
        assert np.array_equal((flags >> 2) & 1, jl) and np.array_equal((flags >> 3) & 1, jr)
        # rows made of one group are recorded for the output clear to skip
        assert np.array_equal(plan.single_rows().cpu().numpy(), groups_per_row == 1)


def test_plan_block_shift_argument(api):
    """The per-call block size equals the tuning knob's, and 31 leaves one block: the groups keep
    their order (apart from the length classes of single-group rows when those are switched on)."""
    indptr, col = GRAPHS["hub"]()
    n = indptr.size - 1
    pp, p2n = co.build_part(5, indptr)
    args = (dev(pp), dev(col), p2n.size, col.size, n, 16)
    api.set_plan_shift(9)
    try:
        knob = api.build_plan(*args, part2node=dev(p2n))
    finally:
        api.set_plan_shift(0)
    call = api.build_plan(*args, part2node=dev(p2n), block_shift=9)
    for a, b in zip(knob.view(), call.view()):
        assert torch.equal(a, b)
    one = api.build_plan(*args, part2node=dev(p2n), block_shift=31)
    ptr, row, flags, pcol = [t.cpu().numpy() for t in one.view()]
    assert np.array_equal(row, p2n) and np.array_equal(ptr, pp) and np.array_equal(pcol, col)
    api.set_plan_length_classes(True)
    try:
        one = api.build_plan(*args, part2node=dev(p2n), block_shift=31)
    finally:
        api.set_plan_length_classes(None)
    ptr, row, flags, pcol = [t.cpu().numpy() for t in one.view()]
    groups_per_row = np.bincount(p2n, minlength=n)
    cls = np.where(groups_per_row[p2n] == 1, np.minimum(3, (np.diff(pp) - 1) >> 3), 3)
    order = np.argsort(cls, kind="stable")
    assert np.array_equal(row, p2n[order]) and np.array_equal(np.diff(ptr), np.diff(pp)[order])
    with pytest.raises(api.EppgcnError):
        api.build_plan(*args, part2node=dev(p2n), block_shift=32)


def test_plan_policy_follows_the_kernel_that_will_run(api):
    """With the policy left automatic a plan is ordered for the kernel that will run over it: the stream form's
    order (rows of up to 64 slots together, no length classes) when the launch shape is one the stream kernel
    covers, the group kernel's (256 slots, length classes) when the stream mode is off at build time or the rows
    are wider than the stream kernel takes (more than 1024 bytes)."""
    indptr, col = GRAPHS["medium"]()
    n = indptr.size - 1
    pp, p2n = co.build_part(31, indptr)       # single-group rows of 1 ... 31 slots: all four length classes

    def build(dim, keep=None, classes=None):
        api.set_plan_keep_rows(keep)
        api.set_plan_length_classes(classes)
        try:
            return api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n), block_shift=8)
        finally:
            api.set_plan_keep_rows(None)
            api.set_plan_length_classes(None)

    def same(a, b):
        return all(torch.equal(x, y) for x, y in zip(a.view(), b.view()))

    stream_order, group_order = build(16, 2, False), build(16, 8, True)
    assert not same(stream_order, group_order), "the two policies must differ on this graph for the test to mean anything"
    assert same(build(16), stream_order)
    api.set_stream_mode(False)
    try:
        assert same(build(16), group_order)
    finally:
        api.set_stream_mode(True)
    assert same(build(260), build(260, 8, True))          # 1040-byte rows: group kernel
    assert same(build(256), build(256, 2, False))         # 1024-byte rows: stream kernel


@pytest.mark.parametrize("rounds", [0, 1, 3])
@pytest.mark.parametrize("dim", [16, 22, 64, 256])
@pytest.mark.parametrize("shift", [0, 3, 20])
def test_planned_aggregation_exact_integer_sums(api, rounds, dim, shift):
    """A plan only changes which groups run together.  With s == 1 and small integer features the
    result must be exactly the neighbour sums, for tiny column blocks (every group alone in its
    block order), the default, and one block (the original order)."""
    indptr, col = hub_csr(3000, 2500, 23)
    n = indptr.size - 1
    x = np.random.default_rng(dim).integers(-8, 9, (n, dim)).astype(np.float32)
    s = np.ones(n, np.float32)
    want = np.zeros((n, dim), np.float64)
    np.add.at(want, cf.row_index(indptr), x[col].astype(np.float64))
    src = np.random.default_rng(5).random(n) < 0.4
    keep = src[col]
    want_b = np.zeros((n, dim), np.float64)
    np.add.at(want_b, cf.row_index(indptr)[keep], (x * src[:, None])[col[keep]].astype(np.float64))
    try:
        api.set_rounds(rounds)
        api.set_plan_shift(shift)
        for ps in (1, 3, 32):
            pp, p2n = co.build_part(ps, indptr)
            dpp, dcol, dp2n = dev(pp), dev(col), dev(p2n)
            plan = api.build_plan(dpp, dcol, p2n.size, col.size, n, dim, part2node=dp2n)
            # the output buffer arrives full of NaN: rows the clear skips must be written whole
            got = api.spmm_forward(dev(x), dcol, dev(s), dpp, dp2n, part_size=ps, plan=plan,
                                   out=torch.full((n, dim), float("nan"), device="cuda"))
            assert np.array_equal(got.cpu().numpy().astype(np.float64), want), f"forward ps={ps}"
            # a plan also serves calls without a feature workspace (per-edge scale gather)
            got = api.spmm_forward(dev(x), dcol, dev(s), dpp, dp2n, part_size=ps, plan=plan, workspace=None,
                                   out=torch.full((n, dim), float("nan"), device="cuda"))
            assert np.array_equal(got.cpu().numpy().astype(np.float64), want), f"forward ps={ps}, no workspace"
            oid, oedge, bpp, p = _gpu_path(api, indptr, col, src, 5, ps)
            if p == 0:
                continue
            bplan = api.build_plan(bpp, oedge, p, int(keep.sum()), n, dim, ids=oid)
            dy = dev((x * src[:, None]).astype(np.float32))
            kept_per_row = np.bincount(cf.row_index(indptr)[keep], minlength=n)
            assert np.array_equal(bplan.single_rows().cpu().numpy(), (kept_per_row >= 1) & (kept_per_row <= ps))
            gb = api.ours_backward(dy, oid, bpp, oedge, dev(s), p, part_size=ps, plan=bplan,
                                   out=torch.full((n, dim), float("nan"), device="cuda"))
            assert np.array_equal(gb.cpu().numpy().astype(np.float64), want_b), f"pruned ps={ps}"
            gb = api.ours_backward(dy, oid, bpp, oedge, dev(s), p, part_size=ps, plan=bplan, workspace=None,
                                   out=torch.full((n, dim), float("nan"), device="cuda"))
            assert np.array_equal(gb.cpu().numpy().astype(np.float64), want_b), f"pruned ps={ps}, no workspace"
    finally:
        api.set_rounds(0)
        api.set_plan_shift(0)


@pytest.mark.parametrize("name", ["isolated", "hub", "medium"])
@pytest.mark.parametrize("dim", [16, 22, 100, 7, 5, 3])
def test_planned_aggregation_within_tolerance(api, name, dim):
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    x = np.random.default_rng(dim).standard_normal((n, dim)).astype(np.float32)
    s = scale_inv_sqrt(indptr)
    want = co.spmm_f64(x, indptr, col, s)
    bound = cf.abs_sum_bound(indptr, col, s, x)
    for ps in (4, 32):
        pp, p2n = co.build_part(ps, indptr)
        plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
        got = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=ps, plan=plan,
                               out=torch.full((n, dim), float("nan"), device="cuda"))
        assert_close(got.cpu().numpy(), want, bound, f"{name} D={dim} ps={ps} planned")
        got = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=ps, plan=plan, workspace=None,
                               out=torch.full((n, dim), float("nan"), device="cuda"))
        assert_close(got.cpu().numpy(), want, bound, f"{name} D={dim} ps={ps} planned, no workspace")


def test_forward_unit_scale_integer_features_bit_exact(api):
    """With s == 1 and small integer features every partial sum is exact in fp32, so any
    grouping, lane mapping or atomic order must give exactly the neighbour sum."""
    indptr, col = hub_csr(6000, 5000, 4)
    n = indptr.size - 1
    x = np.random.default_rng(0).integers(-8, 9, (n, 22)).astype(np.float32)
    s = np.ones(n, np.float32)
    want = np.zeros((n, 22), np.float64)
    np.add.at(want, cf.row_index(indptr), x[col].astype(np.float64))
    for ps in (1, 5, 32, 100):
        pp, p2n = co.build_part(ps, indptr)
        got = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=ps).cpu().numpy()
        assert np.array_equal(got.astype(np.float64), want)
        back = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=ps, backward=True)
        assert np.array_equal(back.cpu().numpy(), got)


def test_forward_zero_groups_and_argument_errors(api):
    x = torch.randn(10, 16, device="cuda")
    empty = torch.zeros(0, dtype=torch.int32, device="cuda")
    pp = torch.zeros(1, dtype=torch.int32, device="cuda")
    out = api.spmm_forward(x, empty, torch.ones(10, device="cuda"), pp, empty)
    assert not out.any()
    with pytest.raises(api.EppgcnError):
        api.spmm_forward(x.double(), empty, torch.ones(10, device="cuda"), pp, empty)
    with pytest.raises(api.EppgcnError):
        api.spmm_forward(x, empty, torch.ones(10, device="cuda"), pp, empty, part_size=0)
    with pytest.raises(api.EppgcnError):
        api.spmm_forward(x.cpu(), empty, torch.ones(10, device="cuda"), pp, empty)


# ----------------------------------------------------------------------------- pruned backward
def _gpu_path(api, indptr, col, src, ps_fwd, ps_back):
    """mask -> compact -> split on the GPU, checked bit-exact against the closed form."""
    n, e = indptr.size - 1, col.size
    pp, p2n = co.build_part(ps_fwd, indptr)
    bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mask_forward(dev(p2n), dev(pp), dev(col), dev(src), None, bem, degs, True)
    oid, oedge, v = api.compact_back_edge(bem, dev(col))
    bpp, p, v2 = api.split_back_part(degs, e, ps_back)
    w_id, w_edge, w_pp, w_v, w_p, w_degs = cf.pruned_path(indptr, col, src, ps_back)
    assert v == v2 == w_v and p == w_p
    assert np.array_equal(oid.cpu().numpy(), w_id) and np.array_equal(oedge.cpu().numpy(), w_edge)
    assert np.array_equal(bpp.cpu().numpy(), w_pp) and np.array_equal(degs.cpu().numpy(), w_degs)
    return oid, oedge, bpp, p


@pytest.mark.parametrize("name", ["tiny", "small", "isolated", "hub", "medium"])
@pytest.mark.parametrize("dim", [16, 22, 64])
@pytest.mark.parametrize("ratio", [0.0, 0.01, 0.1, 0.5, 1.0])
def test_pruned_backward_vs_checker_and_unpruned(api, name, dim, ratio):
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    rng = np.random.default_rng(dim + int(ratio * 100))
    src = rng.random(n) < ratio
    s = scale_inv_sqrt(indptr)
    dy = (rng.standard_normal((n, dim)) * src[:, None]).astype(np.float32)
    want = co.spmm_f64(dy, indptr, col, s)
    bound = cf.abs_sum_bound(indptr, col, s, dy)
    for ps_back in (1, 8, 64):
        oid, oedge, bpp, p = _gpu_path(api, indptr, col, src, 5, ps_back)
        got = api.ours_backward(dev(dy), oid, bpp, oedge, dev(s), p, part_size=ps_back).cpu().numpy()
        assert_close(got, want, bound, f"{name} D={dim} r={ratio} ps={ps_back}")
        plain = api.ours_backward(dev(dy), oid, bpp, oedge, dev(s), p, part_size=ps_back, workspace=None)
        assert_close(plain.cpu().numpy(), want, bound, f"{name} D={dim} r={ratio} ps={ps_back} [no workspace]")
        ref32 = co.ours_backward(dy, oid.cpu().numpy(), bpp.cpu().numpy(), oedge.cpu().numpy(), s, p)
        assert_close(got, ref32.astype(np.float64), 2 * bound, "vs fp32 restatement")
        # pruning really ignores gradient rows outside the mask
        noisy = (dy + (~src)[:, None] * 50.0).astype(np.float32)
        got2 = api.ours_backward(dev(noisy), oid, bpp, oedge, dev(s), p, part_size=ps_back).cpu().numpy()
        assert_close(got2, want, bound, "noise outside the mask")


@pytest.mark.parametrize("name", ["tiny", "isolated", "hub", "medium"])
@pytest.mark.parametrize("ratio", [0.0, 0.02, 0.3, 1.0])
def test_gathered_rows_bitmap_and_restricted_prescaling(api, name, ratio):
    """The bitmap of the rows a path gathers is exactly the set of its column ids; with it the
    pre-scaling pass leaves every other row of the workspace alone (here: NaN, as are the gradient
    rows outside the set), and the result is the same as without it."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    rng = np.random.default_rng(int(ratio * 100) + n)
    src = rng.random(n) < ratio
    s = scale_inv_sqrt(indptr)
    oid, oedge, bpp, p = _gpu_path(api, indptr, col, src, 5, 8)
    v = int(src[col].sum())
    bitmap, distinct = api.mark_gathered_rows(oedge, v, n)
    want_rows = np.zeros(n, bool)
    want_rows[col[src[col]]] = True
    words = bitmap.cpu().numpy().view(np.uint32)
    got_rows = ((words[np.arange(n) >> 5] >> (np.arange(n) & 31).astype(np.uint32)) & 1).astype(bool)
    assert np.array_equal(got_rows, want_rows) and distinct == int(want_rows.sum())
    assert words.size == (n + 31) // 32 and (n % 32 == 0 or words[-1] >> (n % 32) == 0)
    if p == 0:
        return
    for dim in (16, 22, 7, 40):
        dy = (rng.standard_normal((n, dim)) * src[:, None]).astype(np.float32)
        want = co.spmm_f64(dy, indptr, col, s)
        bound = cf.abs_sum_bound(indptr, col, s, dy)
        poisoned = dy.copy()
        poisoned[~want_rows] = np.nan
        for alias in (False, True):
            d_in = dev(poisoned)
            ws = d_in if alias else torch.full((api.feature_workspace(n, dim, "cuda").numel(),), float("nan"), device="cuda")
            got = api.ours_backward(d_in, oid, bpp, oedge, dev(s), p, part_size=8, workspace=ws,
                                    gathered_rows=bitmap)
            assert_close(got.cpu().numpy(), want, bound, f"{name} r={ratio} D={dim} alias={alias}")
            if not alias:     # rows outside the set were not written
                pitch = api.feature_workspace_pitch(dim)
                rows = api.feature_workspace_rows(n, "cuda")       # where the workspace keeps each vertex
                assert torch.isnan(ws.view(-1, pitch)[rows[dev(~want_rows)]]).all()
                assert not torch.isnan(ws.view(-1, pitch)[rows[dev(want_rows)]][:, :dim]).any()
        plan = api.build_plan(bpp, oedge, p, v, n, dim, ids=oid)
        got = api.ours_backward(dev(poisoned), oid, bpp, oedge, dev(s), p, part_size=8, plan=plan,
                                gathered_rows=bitmap, out=torch.full((n, dim), float("nan"), device="cuda"))
        assert_close(got.cpu().numpy(), want, bound, f"{name} r={ratio} D={dim} planned")


def test_two_layer_mask_chain_on_gpu(api):
    """The wiring of the reference's driver for 2 layers (EPPGCN/gcn_main.py:130-139)."""
    indptr, col = GRAPHS["medium"]()
    n, e = indptr.size - 1, col.size
    rng = np.random.default_rng(2)
    train = rng.random(n) < 0.1
    pp, p2n = co.build_part(8, indptr)
    dpp, dp2n, dcol = dev(pp), dev(p2n), dev(col)
    ngh0 = torch.zeros(n, dtype=torch.bool, device="cuda")
    em = [torch.full((e,), -1, dtype=torch.int32, device="cuda") for _ in range(2)]
    nd = [torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(2)]
    api.mask_forward(dp2n, dpp, dcol, dev(train), ngh0, em[1], nd[1], False)          # conv 0's forward
    api.mask_forward(dp2n, dpp, dcol, ngh0, torch.zeros(0, dtype=torch.bool, device="cuda"), em[0], nd[0], True)
    row = cf.row_index(indptr)
    closure = train.copy()
    closure[col[train[row]]] = True
    assert np.array_equal(ngh0.cpu().numpy(), closure)
    assert np.array_equal(em[1].cpu().numpy() != -1, train[col])
    assert np.array_equal(em[0].cpu().numpy() != -1, closure[col])


# ----------------------------------------------------------------------------- full-size properties
@pytest.fixture(scope="module")
def rmat20():
    from eppgcn_amd import graphs
    return graphs.make_graph("cfg3_rmat20", device="cuda")


def test_rmat20_exact_integer_sums_and_path_invariants(api, rmat20):
    """Size-independent properties at a benchmark size (R-MAT scale 20): exact integer neighbour
    sums against torch index_add in int64; compacted-path invariants; pruned == unpruned."""
    from eppgcn_amd import graphs
    g = rmat20
    n, e = g.num_nodes, g.num_edges
    ps = int(g.avg_degree)
    pp, p2n = api.build_part(ps, g.row_pointers, e)
    assert int(pp[-1]) == e and int((pp[1:] - pp[:-1]).max()) <= ps and int((pp[1:] - pp[:-1]).min()) >= 1
    row = g.row_index()
    xi = (graphs.uniform32(5, torch.arange(n * 16, device="cuda")) % 17 - 8).reshape(n, 16)
    ones = torch.ones(n, device="cuda")
    got = api.spmm_forward(xi.float(), g.column_index, ones, pp, p2n, part_size=ps)
    want = torch.zeros(n, 16, dtype=torch.int64, device="cuda").index_add_(0, row, xi[g.column_index.long()])
    assert torch.equal(got.long(), want)
    plan = api.build_plan(pp, g.column_index, p2n.numel(), e, n, 16, part2node=p2n)
    got_p = api.spmm_forward(xi.float(), g.column_index, ones, pp, p2n, part_size=ps, plan=plan)
    assert torch.equal(got_p.long(), want)

    train = graphs.bernoulli_mask(n, 0.1, 2, "cuda")
    bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mask_forward(p2n, pp, g.column_index, train, None, bem, degs, True)
    keep = train[g.column_index.long()]
    assert torch.equal(bem != -1, keep)
    oid, oedge, v = api.compact_back_edge(bem, g.column_index)
    assert v == int(keep.sum())
    assert torch.equal(oid[:v].long(), row[keep]) and torch.equal(oedge[:v], g.column_index[keep])
    assert not oid[v:].any() and not oedge[v:].any()
    assert torch.equal(torch.bincount(oid[:v].long(), minlength=n).int(), degs)
    for ps_b in (8, 32):
        bpp, p, v2 = api.split_back_part(degs, e, ps_b)
        assert v2 == v and int(bpp[p]) == v
        sizes = bpp[1: p + 1] - bpp[:p]
        assert int(sizes.min()) >= 1 and int(sizes.max()) <= ps_b
        assert torch.equal(oid[bpp[:p].long()], oid[(bpp[1: p + 1] - 1).long()])   # a group never spans two rows
        dy = xi.float() * train[:, None]
        pruned = api.ours_backward(dy, oid, bpp, oedge, ones, p, part_size=ps_b)
        unpruned = api.spmm_forward(dy, g.column_index, ones, pp, p2n, part_size=ps, backward=True)
        assert torch.equal(pruned, unpruned)


def test_rmat20_linearity_and_tolerance(api, rmat20):
    from eppgcn_amd import graphs
    g = rmat20
    n, e = g.num_nodes, g.num_edges
    ps = int(g.avg_degree)
    pp, p2n = api.build_part(ps, g.row_pointers, e)
    for dim in (16, 22):
        x = graphs.normal32(1, (n, dim), "cuda")
        got = api.spmm_forward(x, g.column_index, g.degrees, pp, p2n, part_size=ps)
        row = g.row_index()
        w = (g.degrees[row] * g.degrees[g.column_index.long()]).double()
        want = torch.zeros(n, dim, dtype=torch.float64, device="cuda").index_add_(
            0, row, w[:, None] * x[g.column_index.long()].double())
        bound = torch.zeros(n, dim, dtype=torch.float64, device="cuda").index_add_(
            0, row, w.abs()[:, None] * x[g.column_index.long()].double().abs())
        worst = ((got.double() - want).abs() / (RTOL * bound + 1e-30)).max().item()
        assert worst <= 1.0, f"D={dim}: max err/limit {worst:.3f}"


def test_rmat20_against_the_reference_order_restatement(api, rmat20):
    """R-MAT 20 at its own size against the checker's fp32 restatement of the reference's loops (one group after the
    other, `w = fl(s_r s_c)`, the reference's roundings per term; EPPGCN_kernel.cu:263-293, :642-668), not only
    against a float64 sum: forward at both widths through the path without workspace (the reference's rounding
    model, groups in CSR order) and through the benchmark's path (plan, pre-scaled table, stream form); pruned
    backward over a 10 % mask both ways.  What remains is the order in which the groups of a row are combined and,
    on the pre-scaled path, one rounding more per term and one less per row: 2e-5 of the absolute sum."""
    from eppgcn_amd import graphs
    g = rmat20
    n, e = g.num_nodes, g.num_edges
    ps = max(16, int(g.avg_degree))
    pp, p2n = api.build_part(ps, g.row_pointers, e)
    col_h, s_h = g.column_index.cpu().numpy(), g.degrees.cpu().numpy()
    pp_h, p2n_h = pp.cpu().numpy(), p2n.cpu().numpy()
    row = g.row_index()
    w_abs = (g.degrees[row] * g.degrees[g.column_index.long()]).abs()

    def bound_of(x):
        return torch.zeros(n, x.shape[1], device="cuda").index_add_(0, row, w_abs[:, None] * x[g.column_index.long()].abs())

    def check(got, want_h, bound, what):
        worst = ((got - torch.from_numpy(want_h).cuda()).abs() / (2e-5 * bound + 1e-30)).max().item()
        assert worst <= 1.0, f"{what}: max err/limit {worst:.3f}"

    plan = api.build_plan(pp, g.column_index, p2n.numel(), e, n, 22, part2node=p2n)
    for dim in (16, 22):
        x = graphs.normal32(1, (n, dim), "cuda", dim)
        want = co.spmm_groups(x.cpu().numpy(), col_h, s_h, pp_h, p2n_h, n, threads=True)
        bound = bound_of(x)
        check(api.spmm_forward(x, g.column_index, g.degrees, pp, p2n, part_size=ps, workspace=None), want, bound,
              f"forward D={dim}, reference rounding model")
        ws = api.feature_workspace(n, dim, "cuda", plan)
        check(api.spmm_forward(x, g.column_index, g.degrees, pp, p2n, part_size=ps, workspace=ws, plan=plan), want, bound,
              f"forward D={dim}, benchmark path")
        assert api.last_call_used_stream()
    # pruned backward over the last layer's path of a 10 % mask
    mask = graphs.bernoulli_mask(n, 0.1, 2, "cuda")
    bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mask_forward(p2n, pp, g.column_index, mask, None, bem, degs, True)
    ids, edge_list, v = api.compact_back_edge(bem, g.column_index)
    part_pointer, num_parts, _ = api.split_back_part(degs, e, 32)
    dy = graphs.normal32(5, (n, 22), "cuda") * mask[:, None]
    want = co.ours_backward(dy.cpu().numpy(), ids.cpu().numpy(), part_pointer.cpu().numpy(), edge_list.cpu().numpy(), s_h,
                            num_parts, threads=True)
    bound = bound_of(dy)
    check(api.ours_backward(dy, ids, part_pointer, edge_list, g.degrees, num_parts, 32, workspace=None), want, bound,
          "pruned backward, reference rounding model")
    path_plan = api.build_plan(part_pointer, edge_list, num_parts, v, n, 22, ids=ids, block_shift=31)
    ws = api.feature_workspace(n, 22, "cuda", path_plan)
    check(api.ours_backward(dy, ids, part_pointer, edge_list, g.degrees, num_parts, 32, 1, 4, 16, None, ws, plan=path_plan),
          want, bound, "pruned backward, benchmark path")
    assert api.last_call_used_stream()


# ----------------------------------------------------------------------------- fused marking + compaction
@pytest.mark.parametrize("name", list(GRAPHS))
@pytest.mark.parametrize("ratio", [0.0, 0.1, 0.6, 1.0])
@pytest.mark.parametrize("ps", [1, 3, 32, 5000])
def test_mark_compact_equals_marking_then_compaction(api, name, ratio, ps):
    """One pass must leave exactly what the checker's mask_forward followed by its compaction
    leave: compacted rows and columns with zero tails, kept length, kept degrees (added to what
    node_degs held), neighbour mask (or-ed into what it held); for a middle and a last layer."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    rng = np.random.default_rng(5)
    src = rng.random(n) < ratio
    pp, p2n = co.build_part(ps, indptr)
    for is_last in (False, True):
        ngh0 = rng.random(n) < 0.05
        degs0 = rng.integers(0, 3, n).astype(np.int32)
        want_ngh = ngh0.copy()
        want_bem = np.full(col.size, -1, np.int32)
        want_degs = degs0.copy()
        co.mask_forward(p2n, pp, col, src, None if is_last else want_ngh, want_bem, want_degs, is_last)
        want_id, want_edge, want_v = co.compact_mask(want_bem, col)
        ngh = None if is_last else dev(ngh0)
        degs = dev(degs0)
        out_id, out_edge, v = api.mark_compact(dev(p2n), dev(pp), dev(col), dev(src), ngh, degs, is_last)
        assert v == want_v
        assert np.array_equal(out_id.cpu().numpy(), want_id) and np.array_equal(out_edge.cpu().numpy(), want_edge)
        assert np.array_equal(degs.cpu().numpy(), want_degs)
        if not is_last:
            assert np.array_equal(ngh.cpu().numpy(), want_ngh)


def test_fused_and_stepwise_path_preparation_agree_at_scale(api):
    """R-MAT scale 20: the whole mask chain and both layers' backward paths, fused versus the
    reference's separate steps, bit for bit."""
    from eppgcn_amd import graphs, workload
    g = graphs.make_graph("cfg3_rmat20", device="cuda")
    a = workload.prepare(g, 2, 0.1, 2, fused=True, plan=False)
    b = workload.prepare(g, 2, 0.1, 2, fused=False, plan=False)
    assert torch.equal(a.ngh_masks[0], b.ngh_masks[0])
    for pa, pb in zip(a.paths, b.paths):
        assert (pa.valid_len, pa.num_parts, pa.valid_node) == (pb.valid_len, pb.num_parts, pb.valid_node)
        assert torch.equal(pa.ids, pb.ids) and torch.equal(pa.edge_list, pb.edge_list)
        assert torch.equal(pa.part_pointer, pb.part_pointer) and torch.equal(pa.node_degs, pb.node_degs)


# ----------------------------------------------------------------------------- HIP graph capture
@pytest.mark.parametrize("stream_form", [False, True])
def test_aggregation_calls_replay_from_a_hip_graph(api, stream_form):
    """The library allocates nothing and clears its outputs with a fill kernel (no memset nodes),
    so a caller can capture the calls into a HIP graph.  Every replay, with eager work and
    synchronisations in between and fresh inputs each time, must equal the eager result - through the
    group kernel (workspace without room for partial sums) and through the plans' stream form (pre-scaling
    pass, stream kernel, fix-up kernel and the clear of rows without slots all recorded), where replay and
    eager run must agree bit for bit."""
    indptr, col = random_symmetric_csr(6000, 40000, 77)
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(8)
    src = rng.random(n) < 0.3
    pp, p2n = api.build_part(8, dev(indptr), col.size)
    d_col, d_s = dev(col), dev(s)
    ids, edge_list, v = api.mark_compact(p2n, pp, d_col, dev(src), None, torch.zeros(n, dtype=torch.int32, device="cuda"), True)
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mark_compact(p2n, pp, d_col, dev(src), None, degs, True)
    part_pointer, num_parts, _ = api.split_back_part(degs, col.size, 8)
    x = torch.zeros((n, 22), device="cuda")
    y_fwd, y_bwd = torch.empty_like(x), torch.empty_like(x)
    # with a plan (selective output clear) and the gathered-rows bitmap (restricted pre-scaling)
    plan = api.build_plan(pp, d_col, p2n.numel(), col.size, n, 22, part2node=p2n)
    bplan = api.build_plan(part_pointer, edge_list, num_parts, v, n, 22, ids=ids) if stream_form else None
    ws = api.feature_workspace(n, 22, "cuda", (plan, bplan) if stream_form else None)
    bitmap, _ = api.mark_gathered_rows(edge_list, v, n)
    used = []

    def both():
        api.spmm_forward(x, d_col, d_s, pp, p2n, 8, out=y_fwd, workspace=ws, plan=plan)
        used.append(api.last_call_used_stream())
        api.ours_backward(x, ids, part_pointer, edge_list, d_s, num_parts, 8, out=y_bwd, workspace=ws,
                          plan=bplan, gathered_rows=bitmap)
        used.append(api.last_call_used_stream())

    both()                                    # warm-up outside the capture
    assert used == [stream_form, stream_form]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        both()
    for rep in range(4):
        x.copy_(dev(rng.standard_normal((n, 22)).astype(np.float32)))
        y_fwd.fill_(7.0); y_bwd.fill_(7.0)    # stale contents the replay has to clear itself
        graph.replay()
        torch.cuda.synchronize()
        got_f, got_b = y_fwd.clone(), y_bwd.clone()
        both()                                # eager, same inputs
        torch.cuda.synchronize()
        xn = x.cpu().numpy()
        bound = co.spmm_f64(np.abs(xn), indptr, col, s) + 1e-30
        assert_close(got_f.cpu().numpy(), y_fwd.cpu().numpy().astype(np.float64), 2 * bound, f"forward replay {rep}")
        assert_close(got_b.cpu().numpy(), y_bwd.cpu().numpy().astype(np.float64), 2 * bound, f"backward replay {rep}")
        assert_close(got_f.cpu().numpy(), co.spmm_f64(xn, indptr, col, s), bound, f"forward replay {rep} vs checker")
        if stream_form:
            assert torch.equal(got_f, y_fwd) and torch.equal(got_b, y_bwd), "the stream form sums in a fixed order"


# ----------------------------------------------------------------------------- headline size
def test_rmat22_headline_size_exact_integer_sums_with_plans(api):
    """The benchmark's own configuration (R-MAT scale 22, 132 M slots), where execution plans,
    128-byte padded rows and multi-round waves are what runs by default.  Integer-valued inputs
    with unit scale make every partial sum exact in fp32 (|sum| <= 8 * max degree < 2^24), so the
    results must equal torch's index_add bit for bit whatever the summation order; the pruned
    backward must equal the unpruned backward of the masked gradient."""
    from eppgcn_amd import graphs, workload
    g = graphs.make_graph("cfg4_rmat22", device="cuda")
    n, e = g.num_nodes, g.num_edges
    wl = workload.prepare(g, 2, 0.1, 2)
    assert wl.plans and wl.paths[0].plan is not None, "plans are expected at this size"
    assert int(g.row_pointers[1:].sub(g.row_pointers[:-1]).max()) * 8 < (1 << 24)
    ones = torch.ones(n, device="cuda")
    row = g.row_index()
    col = g.column_index.long()
    for dim in (16, 22):
        xi = (graphs.uniform32(6, torch.arange(n * dim, device="cuda")) % 17 - 8).reshape(n, dim).float()
        want = torch.zeros(n, dim, device="cuda").index_add_(0, row, xi[col])
        got = api.spmm_forward(xi, g.column_index, ones, wl.part_ptr, wl.part2node, wl.part_size, plan=wl.plans[dim])
        assert torch.equal(got, want), f"planned forward, width {dim}"
        del want
        path = wl.paths[0] if dim == 16 else wl.paths[1]
        src = wl.ngh_masks[0] if dim == 16 else wl.train_mask
        dy = xi * src[:, None]
        pruned = api.ours_backward(dy, path.ids, path.part_pointer, path.edge_list, ones, path.num_parts,
                                   path.part_size, plan=path.plan)
        unpruned = api.spmm_forward(dy, g.column_index, ones, wl.part_ptr, wl.part2node, wl.part_size, backward=True,
                                    plan=wl.plans[dim])
        assert torch.equal(pruned, unpruned), f"pruned vs unpruned backward, width {dim}"
        # the kept path is exactly the slots whose column is in the source mask, in CSR order
        keep = src[col]
        assert path.valid_len == int(keep.sum())
        assert torch.equal(path.edge_list[:path.valid_len], g.column_index[keep])
        assert torch.equal(path.ids[:path.valid_len].long(), row[keep])
        del keep, dy, pruned, unpruned, xi


@pytest.mark.parametrize("name", ["small", "hub", "medium"])
def test_marking_with_empty_groups_in_the_group_arrays(api, name):
    """Caller-made group arrays may hold empty groups (two groups starting at the same slot);
    build_part never makes them, so this is the only test of the owner search both marking kernels
    fall back to.  Empty groups carry arbitrary rows, which must not be marked or counted."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    rng = np.random.default_rng(12)
    pp, p2n = co.build_part(6, indptr)
    where = np.sort(rng.integers(0, p2n.size + 1, size=max(3, p2n.size // 7)))
    pp2 = np.insert(pp, where, pp[where]).astype(np.int32)            # duplicate starts = empty groups
    p2n2 = np.insert(p2n, where, rng.integers(0, n, where.size)).astype(np.int32)
    assert np.all(np.diff(pp2) >= 0) and (np.diff(pp2) == 0).sum() == where.size
    src = rng.random(n) < 0.3
    for is_last in (False, True):
        want_ngh = np.zeros(n, bool)
        want_bem = np.full(col.size, -1, np.int32)
        want_degs = np.zeros(n, np.int32)
        co.mask_forward(p2n2, pp2, col, src, None if is_last else want_ngh, want_bem, want_degs, is_last)
        want_id, want_edge, want_v = co.compact_mask(want_bem, col)
        ngh = torch.zeros(n, dtype=torch.bool, device="cuda")
        bem = torch.full((col.size,), -1, dtype=torch.int32, device="cuda")
        degs = torch.zeros(n, dtype=torch.int32, device="cuda")
        api.mask_forward(dev(p2n2), dev(pp2), dev(col), dev(src), None if is_last else ngh, bem, degs, is_last)
        assert np.array_equal(bem.cpu().numpy(), want_bem) and np.array_equal(degs.cpu().numpy(), want_degs)
        assert np.array_equal(ngh.cpu().numpy(), want_ngh)
        ngh2 = torch.zeros(n, dtype=torch.bool, device="cuda")
        degs2 = torch.zeros(n, dtype=torch.int32, device="cuda")
        oid, oedge, v = api.mark_compact(dev(p2n2), dev(pp2), dev(col), dev(src), None if is_last else ngh2, degs2, is_last)
        assert v == want_v and np.array_equal(oid.cpu().numpy(), want_id) and np.array_equal(oedge.cpu().numpy(), want_edge)
        assert np.array_equal(degs2.cpu().numpy(), want_degs) and np.array_equal(ngh2.cpu().numpy(), want_ngh)


@pytest.mark.parametrize("name", ["small", "hub", "medium"])
@pytest.mark.parametrize("dim", [16, 22, 70])
def test_aggregation_with_empty_groups(api, name, dim):
    """Empty groups (two groups starting at the same slot) that name the row of the group after
    them keep a row's groups consecutive, which is all the aggregation requires; they add nothing."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(14)
    pp, p2n = co.build_part(5, indptr)
    where = np.sort(rng.integers(0, p2n.size, size=max(3, p2n.size // 5)))
    pp2 = np.insert(pp, where, pp[where]).astype(np.int32)
    p2n2 = np.insert(p2n, where, p2n[where]).astype(np.int32)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    want = co.spmm_f64(x, indptr, col, s)
    bound = co.spmm_f64(np.abs(x), indptr, col, s) + 1e-30
    for workspace in (True, None):
        got = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp2), dev(p2n2), part_size=5, workspace=workspace)
        assert_close(got.cpu().numpy(), want, bound, f"empty groups, workspace={workspace}")
    plan = api.build_plan(dev(pp2), dev(col), p2n2.size, col.size, n, dim, part2node=dev(p2n2))
    api.set_plan_shift(9)
    try:
        plan = api.build_plan(dev(pp2), dev(col), p2n2.size, col.size, n, dim, part2node=dev(p2n2))
    finally:
        api.set_plan_shift(0)
    got = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp2), dev(p2n2), part_size=5, plan=plan,
                           out=torch.full((n, dim), float("nan"), device="cuda"))
    assert_close(got.cpu().numpy(), want, bound, "empty groups with a plan")
    groups = np.bincount(p2n2, minlength=n)
    filled = np.bincount(p2n2[np.diff(pp2) > 0], minlength=n)
    assert np.array_equal(plan.single_rows().cpu().numpy(), (groups == 1) & (filled == 1))


@pytest.mark.parametrize("dim", [16, 22, 7, 64])
@pytest.mark.parametrize("shift_in,shift_out", [(1, 0), (0, 1), (1, 1), (2, 3)])
def test_aggregation_with_misaligned_feature_buffers(api, dim, shift_in, shift_out):
    """Feature and output matrices that start 4, 8 or 12 bytes into an allocation (views of larger
    tensors) take the narrower vector paths; with and without a workspace, forward and pruned."""
    indptr, col = GRAPHS["medium"]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(16)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    want = co.spmm_f64(x, indptr, col, s)
    bound = co.spmm_f64(np.abs(x), indptr, col, s) + 1e-30
    pp, p2n = api.build_part(8, dev(indptr), col.size)
    xin = torch.empty(n * dim + 4, device="cuda")[shift_in: shift_in + n * dim].view(n, dim)
    xin.copy_(dev(x))
    out = torch.empty(n * dim + 4, device="cuda")[shift_out: shift_out + n * dim].view(n, dim)
    assert xin.data_ptr() % 16 == 4 * shift_in and out.data_ptr() % 16 == 4 * shift_out
    for workspace in (True, None):
        out.fill_(3.0)
        api.spmm_forward(xin, dev(col), dev(s), pp, p2n, part_size=8, out=out, workspace=workspace)
        assert_close(out.cpu().numpy(), want, bound, f"forward, workspace={workspace}")
    # with a plan the output clear skips single-group rows: the narrower clears must do the same
    plan = api.build_plan(pp, dev(col), p2n.numel(), col.size, n, dim, part2node=p2n)
    out.fill_(float("nan"))
    api.spmm_forward(xin, dev(col), dev(s), pp, p2n, part_size=8, out=out, plan=plan)
    assert_close(out.cpu().numpy(), want, bound, "forward with a plan")
    src = rng.random(n) < 0.4
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    ids, edge_list, v = api.mark_compact(p2n, pp, dev(col), dev(src), None, degs, True)
    bpp, p, _ = api.split_back_part(degs, col.size, 8)
    xm = x * src[:, None]
    xin.copy_(dev(xm))
    want_b = co.spmm_f64(xm, indptr, col, s)
    for workspace in (True, None):
        out.fill_(3.0)
        api.ours_backward(xin, ids, bpp, edge_list, dev(s), p, 8, out=out, workspace=workspace)
        assert_close(out.cpu().numpy(), want_b, bound, f"pruned backward, workspace={workspace}")


@pytest.mark.parametrize("dim", [16, 22, 7, 3])
def test_wide_index_instantiations_of_the_streaming_kernels(api, dim):
    """The clear and pre-scaling kernels have a 32-bit and a 64-bit index instantiation; the
    second is only chosen by itself for matrices of 2^32 elements and more, so it is forced here:
    padded, flat and aliased pre-scaling, restricted to gathered rows or not, full and selective
    clear must give the results of the default instantiation bit for bit."""
    indptr, col = GRAPHS["medium"]()
    n = indptr.size - 1
    rng = np.random.default_rng(dim)
    s = scale_inv_sqrt(indptr)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    src = rng.random(n) < 0.2
    pp, p2n = co.build_part(6, indptr)
    oid, oedge, bpp, p = _gpu_path(api, indptr, col, src, 6, 8)
    bitmap, _ = api.mark_gathered_rows(oedge, int(src[col].sum()), n)
    plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
    dy = (x * src[:, None]).astype(np.float32)

    def run_all():
        nan = lambda: torch.full((n, dim), float("nan"), device="cuda")
        res = [api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=6, out=nan()),
               api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=6, plan=plan, out=nan())]
        alias = dev(x)
        res.append(api.spmm_forward(alias, dev(col), dev(s), dev(pp), dev(p2n), part_size=6, workspace=alias, out=nan()))
        res.append(api.ours_backward(dev(dy), oid, bpp, oedge, dev(s), p, part_size=8, gathered_rows=bitmap, out=nan()))
        alias = dev(dy)
        res.append(api.ours_backward(alias, oid, bpp, oedge, dev(s), p, part_size=8, workspace=alias,
                                     gathered_rows=bitmap, out=nan()))
        return [r.cpu().numpy() for r in res]

    narrow = run_all()
    api.set_wide_index(True)
    try:
        wide = run_all()
    finally:
        api.set_wide_index(False)
    want = co.spmm_f64(x, indptr, col, s)
    assert_close(narrow[1], want, cf.abs_sum_bound(indptr, col, s, x), "planned forward")
    for k, (a, b) in enumerate(zip(narrow, wide)):
        # float atomics make the order of a row's partial sums vary between runs: compare to rounding
        assert np.allclose(a, b, rtol=1e-5, atol=1e-6), f"case {k}"
        assert not np.isnan(b).any()


def test_element_offsets_beyond_int32(api):
    """[N, 256] matrices of more than 2^31 elements (8.6 GB each): every row offset has to be
    formed in 64 bits.  Ring graph with self-loops, unit scale, small integer features, so the
    result is exactly x[i-1] + x[i] + x[i+1] whatever the order of summation; the pruned backward
    over a mask that keeps the last rows must equal the unpruned one on the masked gradient, and
    the dense update must reach the last rows too."""
    n, dim = (1 << 23) + 5, 256
    assert n * dim > (1 << 31)
    idx = torch.arange(n, device="cuda")
    col = torch.stack([(idx - 1) % n, idx, (idx + 1) % n], 1).sort(dim=1).values.to(torch.int32).reshape(-1)
    indptr = (torch.arange(n + 1, device="cuda") * 3).to(torch.int32)
    ones = torch.ones(n, device="cuda")
    pp, p2n = api.build_part(2, indptr)
    from eppgcn_amd import graphs
    x = torch.empty(n, dim, device="cuda")
    step = 1 << 20
    for r0 in range(0, n, step):                       # in pieces: the generator works in int64
        r1 = min(n, r0 + step)
        x[r0:r1] = (graphs.uniform32(11, torch.arange(r0 * dim, r1 * dim, device="cuda")) % 17 - 8).reshape(-1, dim)
    want = x + torch.roll(x, 1, 0)
    want += torch.roll(x, -1, 0)
    got = api.spmm_forward(x, col, ones, pp, p2n, part_size=2)
    assert torch.equal(got[-4096:], want[-4096:]) and torch.equal(got[:4096], want[:4096])
    assert torch.equal(got, want)
    del got
    # pruned backward: mask = the last 3000 vertices and every 1000th one
    src = (idx >= n - 3000) | (idx % 1000 == 0)
    e = col.numel()
    bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mask_forward(p2n, pp, col, src, None, bem, degs, True)
    oid, oedge, v = api.compact_back_edge(bem, col)
    bpp, p, v2 = api.split_back_part(degs, e, 2)
    assert v == v2 == int(src[col.long()].sum())
    x *= src[:, None]
    want = x + torch.roll(x, 1, 0)
    want += torch.roll(x, -1, 0)
    got = api.ours_backward(x, oid, bpp, oedge, ones, p, part_size=2)
    assert torch.equal(got, want)
    del got, want
    # dense update of the last rows: [n, 256] x [256, 16] with integer operands is exact in fp32
    w = (graphs.uniform32(12, torch.arange(dim * 16, device="cuda")) % 5 - 2).reshape(dim, 16).float()
    y = api.update_forward(x, w, ones)
    tail = slice(n - 3000, n)
    assert torch.equal(y[tail, :16], x[tail] @ w)
    # input gradient and weight gradient with the non-zero rows at the end of the matrices
    g = torch.zeros(n, 16, device="cuda")
    g[tail] = (graphs.uniform32(13, torch.arange(3000 * 16, device="cuda")) % 7 - 3).reshape(3000, 16).float()
    dx = api.update_backward_input(g, w)
    assert torch.equal(dx[tail], g[tail] @ w.t()) and not dx[: n - 3000].any()
    del dx
    dw = api.update_backward_weight(x, g)
    assert torch.equal(dw, x[tail].t() @ g[tail])


# ----------------------------------------------------------------------------- ragged random inputs
def test_ragged_random_graphs_whole_path(api):
    """Property-based: randomly drawn ragged graphs (empty rows, rows of several groups, no
    edges at all), any mask density, group sizes from 1: every integer result of the device
    path equals the closed forms bit for bit, both ways of preparing the path agree, and the
    aggregations (plain, planned, pruned with the gathered-rows bitmap) stay within tolerance."""
    from hypothesis import HealthCheck, given, settings
    from hypothesis import strategies as st
    from tests.test_oracle_fuzz import ragged_graph

    import os
    examples = int(os.environ.get("EPPGCN_FUZZ_EXAMPLES", "150"))       # raise it for a longer hunt

    @settings(max_examples=examples, deadline=None, derandomize=examples == 150, database=None,
              suppress_health_check=list(HealthCheck))
    @given(ragged_graph(), st.integers(1, 9), st.integers(1, 9), st.sampled_from([0.0, 0.1, 0.5, 1.0]),
           st.sampled_from([1, 3, 4, 16, 22]))
    def check(graph, ps_fwd, ps_back, ratio, dim):
        indptr, col, rng = graph
        n, e = indptr.size - 1, col.size
        d_col = dev(col) if e else torch.zeros(0, dtype=torch.int32, device="cuda")
        pp, p2n = api.build_part(ps_fwd, dev(indptr), e)
        w_pp, w_p2n = cf.build_part(ps_fwd, indptr)
        assert np.array_equal(pp.cpu().numpy(), w_pp) and np.array_equal(p2n.cpu().numpy(), w_p2n)
        src = rng.random(n) < ratio
        w_id, w_edge, w_bpp, w_v, w_p, w_degs = cf.pruned_path(indptr, col, src, ps_back)
        # marking then compaction
        bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
        degs = torch.zeros(n, dtype=torch.int32, device="cuda")
        if p2n.numel():
            api.mask_forward(p2n, pp, d_col, dev(src), None, bem, degs, True)
        oid, oedge, v = api.compact_back_edge(bem, d_col)
        assert v == w_v and np.array_equal(degs.cpu().numpy(), w_degs)
        assert np.array_equal(oid.cpu().numpy(), w_id) and np.array_equal(oedge.cpu().numpy(), w_edge)
        # the fused pass
        if p2n.numel():
            degs2 = torch.zeros(n, dtype=torch.int32, device="cuda")
            fid, fedge, fv = api.mark_compact(p2n, pp, d_col, dev(src), None, degs2, True)
            assert fv == w_v and torch.equal(degs2, degs)
            assert np.array_equal(fid.cpu().numpy()[:w_v], w_id[:w_v])
            assert np.array_equal(fedge.cpu().numpy()[:w_v], w_edge[:w_v])
        bpp, p, v2 = api.split_back_part(degs, e, ps_back)
        assert (p, v2) == (w_p, w_v) and np.array_equal(bpp.cpu().numpy(), w_bpp)
        # aggregation
        s = rng.uniform(0.2, 1.5, n).astype(np.float32)
        x = rng.standard_normal((n, dim)).astype(np.float32)
        want = co.spmm_f64(x, indptr, col, s)
        bound = cf.abs_sum_bound(indptr, col, s, x) if e else np.zeros((n, dim))
        nan = lambda: torch.full((n, dim), float("nan"), device="cuda")
        got = api.spmm_forward(dev(x), d_col, dev(s), pp, p2n, part_size=ps_fwd, out=nan())
        assert_close(got.cpu().numpy(), want, bound, "forward")
        if p2n.numel():
            plan = api.build_plan(pp, d_col, p2n.numel(), e, n, dim, part2node=p2n)
            got = api.spmm_forward(dev(x), d_col, dev(s), pp, p2n, part_size=ps_fwd, plan=plan, out=nan())
            assert_close(got.cpu().numpy(), want, bound, "planned forward")
        dy = (x * src[:, None]).astype(np.float32)
        want_b = co.spmm_f64(dy, indptr, col, s)
        bitmap, _ = api.mark_gathered_rows(oedge, v, n)
        got_b = api.ours_backward(dev(dy), oid, bpp, oedge, dev(s), p, part_size=ps_back, gathered_rows=bitmap,
                                  out=nan())
        assert_close(got_b.cpu().numpy(), want_b, bound, "pruned backward")

    check()


def test_calls_run_on_the_callers_stream(api):
    """Work is issued on the stream the caller passes (torch's current stream here), not on the
    default stream: two side streams (default priority) run the forward and the pruned backward
    of different inputs at the same time with their own buffers; each result is complete after
    synchronising its own stream only, and the path preparation on a side stream returns its counts
    (it synchronises that stream itself)."""
    indptr, col = GRAPHS["medium"]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(21)
    src = rng.random(n) < 0.3
    d_col, d_s, d_indptr = dev(col), dev(s), dev(indptr)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        pp, p2n = api.build_part(8, d_indptr, col.size)
        degs = torch.zeros(n, dtype=torch.int32, device="cuda")
        ids, edge_list, v = api.mark_compact(p2n, pp, d_col, dev(src), None, degs, True)
        bpp, p, v2 = api.split_back_part(degs, col.size, 8)
    s1.synchronize()
    assert v == v2 == int(src[col].sum())
    xs = [rng.standard_normal((n, 22)).astype(np.float32) for _ in range(2)]
    outs = []
    for x, stream in zip(xs, (s1, s2)):
        with torch.cuda.stream(stream):
            dx = dev(x)
            fwd = api.spmm_forward(dx, d_col, d_s, pp, p2n, part_size=8)
            bwd = api.ours_backward(dev((x * src[:, None]).astype(np.float32)), ids, bpp, edge_list, d_s, p, part_size=8)
            outs.append((fwd, bwd))
    for (fwd, bwd), x, stream in zip(outs, xs, (s1, s2)):
        stream.synchronize()
        bound = cf.abs_sum_bound(indptr, col, s, x)
        assert_close(fwd.cpu().numpy(), co.spmm_f64(x, indptr, col, s), bound, "forward on a side stream")
        assert_close(bwd.cpu().numpy(), co.spmm_f64((x * src[:, None]).astype(np.float32), indptr, col, s), bound,
                     "pruned backward on a side stream")
    torch.cuda.synchronize()
