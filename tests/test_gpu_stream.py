"""GPU tests of the stream form of an execution plan and of the aggregation through it.

No counterpart in the reference (its kernels walk one group per warp, EPPGCN_kernel.cu:204-295, :626-670);
the contract is the same operator, so the results are held against the same float64 checker as the group
kernel, the integer cases bit-exactly, and the stream arrays against a numpy construction from the plan's
group arrays."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import closed_forms as cf
from tests.helpers import hub_csr, random_symmetric_csr, scale_inv_sqrt

pytestmark = pytest.mark.gpu
RTOL = 1e-5
WAVE, CHUNK, FLAG = 512, 32, -2 ** 31


@pytest.fixture(scope="module")
def api():
    from eppgcn_amd import capi
    capi.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return capi


@pytest.fixture(autouse=True)
def _stream_mode_on(api):
    api.set_stream_mode(True)
    yield
    api.set_stream_mode(True)
    api.set_plan_shift(0)


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
    "small": lambda: random_symmetric_csr(130, 260, 5),
    "isolated": lambda: random_symmetric_csr(3000, 9000, 11, isolated=0.3),
    "hub": lambda: hub_csr(5000, 4000, 7),                      # one row of 4000 slots: pieces across waves
    "medium": lambda: random_symmetric_csr(20000, 150000, 13),
    "two hubs": lambda: hub_csr(9000, 8500, 3),
}


def host_stream(ptr, row, flags, col, n):
    """The stream form from the plan's group arrays, written the slow and obvious way."""
    P = row.size
    S = int(ptr[P])
    spad = (S + WAVE - 1) // WAVE * WAVE
    pad_id = (n + 4095) // 4096 * 4096
    scol = np.full(spad, pad_id, np.int64)
    scol[:S] = col[:S]
    pieces = []                      # (first slot, last slot, row, whole)
    q = 0
    while q < P:
        assert ptr[q + 1] > ptr[q], "no empty groups in these tests"
        start = q
        while flags[q] & 8:          # the next entry continues this one
            q += 1
            assert flags[q] & 4
        pieces.append((int(ptr[start]), int(ptr[q + 1]) - 1, int(row[q]), not (flags[start] & 1) and not (flags[q] & 2)))
        q += 1
    ends = np.array([p[1] for p in pieces], np.int64)
    is_end = np.zeros(spad + 1, bool)
    is_end[ends] = True
    scol[ends] |= 1 << 31
    cev = np.zeros(spad // CHUNK + 1, np.int64)
    for c in range(cev.size):
        pos = c * CHUNK
        before = int(np.searchsorted(ends, pos, "left")) if pos < S else len(pieces)
        inside = 0 < pos < S and not is_end[pos - 1]
        cev[c] = before | ((1 << 31) if inside else 0)
    partial = [(not whole) or first < last // WAVE * WAVE for first, last, _, whole in pieces]
    cands = [(pieces[e][2], e) for e in range(len(pieces)) if partial[e]]          # (row, source) in stream order
    nw = spad // WAVE
    for w in range(nw):
        at = (w + 1) * WAVE - 1
        if at < S and not is_end[at]:
            e = int(np.searchsorted(ends, at, "left"))
            cands.append((pieces[e][2], P + w))
    order = sorted(range(len(cands)), key=lambda k: cands[k][0])                   # stable: stream order inside a row
    erow = np.array([p[2] for p in pieces], np.int64)
    wtail = np.full(nw, -1, np.int64)
    for k, j in enumerate(order):
        src = cands[j][1]
        if src < P:
            erow[src] = (1 << 31) | k
        else:
            wtail[src - P] = k
    rows_sorted = [cands[j][0] for j in order]
    frow = sorted(set(rows_sorted))
    fptr = [rows_sorted.index(r) for r in frow] + [len(order)]
    touched = np.zeros(n, bool)
    touched[[p[2] for p in pieces]] = True
    as32 = lambda a: (np.asarray(a, np.int64) & 0xffffffff).astype(np.uint32).view(np.int32)
    return dict(col=as32(scol), erow=as32(erow), cev=as32(cev), wtail=as32(wtail), frow=as32(frow), fptr=as32(fptr),
                touched=touched, header=[1, len(pieces), len(order), len(frow), int((~touched).sum()), 0, 0])


def check_stream_form(api, plan, n):
    ptr, row, flags, col = [t.cpu().numpy() for t in plan.view()]
    want = host_stream(ptr, row, flags, col, n)
    got = {k: v.cpu().numpy() for k, v in plan.stream_view().items()}
    assert got["header"][:7].tolist() == want["header"]
    ne, npart, nf = want["header"][1:4]
    assert plan.partial_rows == npart
    assert np.array_equal(got["col"], want["col"]), "column ids, piece ends and padding"
    assert np.array_equal(got["erow"][:ne], want["erow"]), "piece targets"
    assert np.array_equal(got["cev"], want["cev"]), "piece ends per chunk"
    assert np.array_equal(got["wtail"], want["wtail"]), "wave tails"
    assert np.array_equal(got["frow"][:nf], want["frow"]) and np.array_equal(got["fptr"][:nf + 1], want["fptr"])
    r = np.arange(n)
    assert np.array_equal(((got["touched"][r >> 5] >> (r & 31)) & 1).astype(bool), want["touched"])
    return want


@pytest.mark.parametrize("name,ps,shift", [("small", 4, 0), ("isolated", 3, 9), ("hub", 16, 0), ("hub", 31, 10),
                                           ("medium", 8, 12), ("medium", 32, 0), ("two hubs", 5, 11)])
def test_stream_form_of_forward_plans(api, name, ps, shift):
    """Every array of the stream form equals the host construction: piece ends, targets (row or partial sum),
    counts per 32 slots, wave tails, the partial sums numbered row by row in stream order, touched rows."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    pp, p2n = co.build_part(ps, indptr)
    api.set_plan_shift(shift)
    plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, 16, part2node=dev(p2n))
    want = check_stream_form(api, plan, n)
    if name in ("hub", "two hubs"):
        assert want["header"][2] > 0 and (want["wtail"] >= 0).any(), "the hub row has to cross waves"


@pytest.mark.parametrize("name,ratio,ps", [("hub", 0.5, 8), ("medium", 0.1, 32), ("isolated", 0.3, 2)])
def test_stream_form_of_backward_path_plans(api, name, ratio, ps):
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    rng = np.random.default_rng(5)
    src = rng.random(n) < ratio
    fpp, fp2n = co.build_part(8, indptr)
    mask = torch.full((col.size,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mask_forward(dev(fp2n), dev(fpp), dev(col), dev(src), None, mask, degs, True)
    oid, oedge, v = api.compact_back_edge(mask, dev(col))
    bpp, p, _ = api.split_back_part(degs, col.size, ps)
    for shift in (0, 31):
        plan = api.build_plan(bpp, oedge, p, v, n, 22, ids=oid, block_shift=shift)
        check_stream_form(api, plan, n)


@pytest.mark.parametrize("dim", [1, 3, 4, 8, 16, 22, 32, 40, 64, 100, 200, 256, 260])
def test_stream_aggregation_vs_checker_all_team_sizes(api, dim):
    """Widths that map to teams of 4 ... 64 lanes through the stream kernel; rows wider than 1024 bytes fall back
    to the group kernel.  Results within tolerance of the float64 sum, untouched rows zero, and the call reports
    which kernel ran."""
    indptr, col = GRAPHS["hub"]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(dim)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    want = co.spmm_f64(x, indptr, col, s)
    bound = cf.abs_sum_bound(indptr, col, s, x)
    pp, p2n = co.build_part(7, indptr)
    api.set_plan_shift(10)
    plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
    out = torch.full((n, dim), float("nan"), device="cuda")
    api.spmm_forward(dev(x), dev(col), dev(s), dev(pp), dev(p2n), part_size=7, plan=plan, out=out)
    assert api.last_call_used_stream() == (dim <= 256)
    assert_close(out.cpu().numpy(), want, bound, f"D={dim}")


@pytest.mark.parametrize("name", ["hub", "medium", "isolated", "two hubs"])
def test_stream_aggregation_exact_and_reproducible(api, name):
    """Integer features and unit scales: every sum is exact in fp32, so the stream kernel, its partial sums and the
    fix-up must reproduce the checker bit for bit; with float data two runs give the same bits (fixed summation
    order), which the group kernel with its float atomics does not promise."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    rng = np.random.default_rng(3)
    for dim, ps in ((16, 8), (22, 31), (64, 3)):
        x = rng.integers(-4, 5, (n, dim)).astype(np.float32)
        ones = np.ones(n, np.float32)
        pp, p2n = co.build_part(ps, indptr)
        api.set_plan_shift(11)
        plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
        out = torch.full((n, dim), float("nan"), device="cuda")
        api.spmm_forward(dev(x), dev(col), dev(ones), dev(pp), dev(p2n), part_size=ps, plan=plan, out=out)
        assert api.last_call_used_stream()
        assert np.array_equal(out.cpu().numpy(), co.spmm_f64(x, indptr, col, ones).astype(np.float32)), f"{name} D={dim}"
        xf = dev(rng.standard_normal((n, dim)).astype(np.float32))
        s = dev(scale_inv_sqrt(indptr))
        a = api.spmm_forward(xf, dev(col), s, dev(pp), dev(p2n), part_size=ps, plan=plan)
        for _ in range(3):
            b = api.spmm_forward(xf, dev(col), s, dev(pp), dev(p2n), part_size=ps, plan=plan)
            assert torch.equal(a, b), "same bits on every run"


def test_stream_path_selection_and_fallbacks(api):
    """The group kernel runs, with the same results, when the stream form cannot: stream mode off, a workspace
    without room for the partial sums, the input scaled in place, no workspace at all, a plan the library has not
    seen at that address, a plan with empty groups."""
    indptr, col = GRAPHS["hub"]()
    n = indptr.size - 1
    dim = 16
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(8)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    want = co.spmm_f64(x, indptr, col, s)
    bound = cf.abs_sum_bound(indptr, col, s, x)
    pp, p2n = co.build_part(8, indptr)
    args = (dev(col), dev(s), dev(pp), dev(p2n))
    plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
    assert plan.partial_rows > 0
    lib = api.load()
    assert lib.eppgcn_plan_workspace_floats(plan.base_ptr, n, dim) == \
        lib.eppgcn_feature_workspace_floats(n, dim) + plan.partial_rows * api.feature_workspace_pitch(dim)

    def run(expect_stream, **kw):
        out = torch.full((n, dim), float("nan"), device="cuda")
        feats = kw.pop("feats", None)
        api.spmm_forward(dev(x) if feats is None else feats, *args, part_size=8, out=out, **kw)
        assert api.last_call_used_stream() == expect_stream, kw
        assert_close(out.cpu().numpy(), want, bound, str(kw))

    run(True, plan=plan)
    api.set_stream_mode(False)
    run(False, plan=plan)
    api.set_stream_mode(True)
    run(False, plan=plan, workspace=api.feature_workspace(n, dim, "cuda"))       # table only: no room for partial sums
    run(True, plan=plan, workspace=api.feature_workspace(n, dim, "cuda", plan))
    xin = dev(x)
    run(False, plan=plan, feats=xin, workspace=xin)                               # scaled in place
    run(False, plan=plan, workspace=None)
    run(False, plan=None)
    # the same plan bytes at another address: unknown to the library until eppgcn_plan_status is asked about it
    copy = api.Plan(plan.buffer.clone(), 0, plan.num_parts, plan.num_slots, plan.num_nodes, plan.partial_rows)
    copy.base_ptr = copy.buffer.data_ptr() + (plan.base_ptr - plan.buffer.data_ptr())
    if copy.base_ptr % 256 == 0:
        run(False, plan=copy, workspace=api.feature_workspace(n, dim, "cuda", plan))
    # empty groups: no stream form, the group kernel copes with them
    pp2 = np.repeat(pp, 2)[1:]                     # every second group is empty
    p2n2 = np.repeat(p2n, 2)
    plan2 = api.build_plan(dev(pp2), dev(col), p2n2.size, col.size, n, dim, part2node=dev(p2n2))
    assert plan2.partial_rows == 0 and plan2.stream_view()["header"][0].item() == 0
    out = api.spmm_forward(dev(x), dev(col), dev(s), dev(pp2), dev(p2n2), part_size=8, plan=plan2)
    assert not api.last_call_used_stream()
    assert_close(out.cpu().numpy(), want, bound, "empty groups")


@pytest.mark.parametrize("name,ratio", [("hub", 0.5), ("medium", 0.05), ("isolated", 0.3)])
def test_stream_pruned_backward_with_gathered_rows(api, name, ratio):
    """The pruned backward through the stream form: rows outside the path are zero, the restricted pre-scaling
    (gathered-rows bitmap, NaN everywhere else) feeds the swizzled table, one-block and column-blocked plans."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(2)
    src = rng.random(n) < ratio
    fpp, fp2n = co.build_part(8, indptr)
    mask = torch.full((col.size,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mask_forward(dev(fp2n), dev(fpp), dev(col), dev(src), None, mask, degs, True)
    oid, oedge, v = api.compact_back_edge(mask, dev(col))
    bitmap, _ = api.mark_gathered_rows(oedge, v, n)
    for dim, ps in ((16, 32), (22, 4)):
        bpp, p, _ = api.split_back_part(degs, col.size, ps)
        dy = (rng.standard_normal((n, dim)) * src[:, None]).astype(np.float32)
        want = co.spmm_f64(dy, indptr, col, s)
        bound = cf.abs_sum_bound(indptr, col, s, dy)
        poisoned = dy.copy()
        poisoned[~src] = np.nan                      # rows the path never gathers
        for shift in (0, 31):
            plan = api.build_plan(bpp, oedge, p, v, n, dim, ids=oid, block_shift=shift)
            out = torch.full((n, dim), float("nan"), device="cuda")
            api.ours_backward(dev(poisoned), oid, bpp, oedge, dev(s), p, part_size=ps, plan=plan, gathered_rows=bitmap,
                              out=out)
            assert api.last_call_used_stream()
            assert_close(out.cpu().numpy(), want, bound, f"{name} D={dim} shift={shift}")


@pytest.mark.parametrize("name,ratio", [("hub", 0.5), ("medium", 0.05), ("isolated", 0.3)])
def test_pruned_backward_that_leaves_unwritten_rows_alone(api, name, ratio):
    """eppgcn_ours_backward_rows (no counterpart in the reference): through a plan's stream form the rows without
    groups keep what they held (NaN here), the written rows hold the bits eppgcn_ours_backward writes, the bitmap it
    hands out marks exactly the rows with kept slots and is the one inside the plan; the dense products over that
    bitmap equal the products over the cleared gradient bit for bit.  Without a plan the call clears like
    eppgcn_ours_backward and hands out no bitmap."""
    indptr, col = GRAPHS[name]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(3)
    src = rng.random(n) < ratio
    fpp, fp2n = co.build_part(8, indptr)
    mask = torch.full((col.size,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    api.mask_forward(dev(fp2n), dev(fpp), dev(col), dev(src), None, mask, degs, True)
    oid, oedge, v = api.compact_back_edge(mask, dev(col))
    has_slots = degs.cpu().numpy() > 0
    for dim, ps, k in ((16, 32, 96), (22, 4, 16)):
        bpp, p, _ = api.split_back_part(degs, col.size, ps)
        dy = dev((rng.standard_normal((n, dim)) * src[:, None]).astype(np.float32))
        plan = api.build_plan(bpp, oedge, p, v, n, dim, ids=oid)
        want = api.ours_backward(dy, oid, bpp, oedge, dev(s), p, part_size=ps, plan=plan)
        assert api.last_call_used_stream()
        out = torch.full((n, dim), float("nan"), device="cuda")
        got, rows, count = api.ours_backward_rows(dy, oid, bpp, oedge, dev(s), p, part_size=ps, plan=plan, out=out)
        assert api.last_call_used_stream() and rows is not None and count == int(has_slots.sum())
        assert rows == plan.stream_view()["touched"].data_ptr()
        g = got.cpu().numpy()
        assert np.array_equal(g[has_slots], want.cpu().numpy()[has_slots]) and np.isnan(g[~has_slots]).all()
        # the layer's two dense products over the bitmap, from the uncleared gradient
        x = dev(rng.standard_normal((n, k)).astype(np.float32))
        w = dev(rng.uniform(-0.5, 0.5, (k, dim)).astype(np.float32))
        want_dx, want_dw = api.update_backward(x, w, want, relu_input=True)
        dx, dw = api.update_backward_rows(x, w, got, rows, relu_input=True)
        assert torch.equal(dx, want_dx) and torch.equal(dw, want_dw)
        # no plan: the group kernel clears, every row is defined
        out.fill_(float("nan"))
        got, rows, count = api.ours_backward_rows(dy, oid, bpp, oedge, dev(s), p, part_size=ps, out=out)
        assert rows is None and count == n and not api.last_call_used_stream()
        assert not torch.isnan(got).any() and not got.cpu().numpy()[~has_slots].any()


def test_stream_from_a_table_written_by_the_dense_update(api):
    """eppgcn_update_forward_table leaves the table in the workspace's row order with room for the partial sums;
    the aggregation with a NULL input then runs the stream form on it."""
    indptr, col = GRAPHS["medium"]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((n, 24)).astype(np.float32)
    w = rng.standard_normal((24, 22)).astype(np.float32)
    pp, p2n = co.build_part(8, indptr)
    plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, 22, part2node=dev(p2n))
    table = api.update_forward_table(dev(x), dev(w), dev(s), plan=plan)
    got = api.spmm_forward(None, dev(col), dev(s), dev(pp), dev(p2n), part_size=8, workspace=table, plan=plan,
                           prescaled_dim=22)
    assert api.last_call_used_stream()
    t = co.update_forward(x, w)
    want = co.spmm_f64(t, indptr, col, s)
    bound = co.spmm_f64(np.abs(x) @ np.abs(w), indptr, col, s) + 1e-30
    assert_close(got.cpu().numpy(), want, 2 * bound, "product then aggregation")


def _ragged_csr(rng, n):
    """Rows of very different lengths: a share of empty rows, mostly short ones, a few hubs of up to thousands of
    slots (longer than a wave's 512 slots, cut into many column blocks)."""
    deg = rng.geometric(rng.uniform(0.05, 0.6), n).astype(np.int64)
    deg[rng.random(n) < rng.uniform(0.0, 0.5)] = 0
    hubs = rng.integers(0, n, rng.integers(0, 4))
    deg[hubs] = rng.integers(300, 4000, hubs.size)
    deg = np.minimum(deg, n)
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(deg, out=indptr[1:])
    col = np.concatenate([np.sort(rng.choice(n, d, replace=False)) for d in deg] or [np.zeros(0, np.int64)])
    return indptr.astype(np.int32), col.astype(np.int32)


@pytest.mark.parametrize("seed", range(24))
def test_stream_random_ragged_graphs_exact(api, seed):
    """Random ragged graphs, group sizes, column-block sizes, keep-together bounds and widths: the stream arrays
    against the host construction, and with integer features and unit scales the forward sums and the pruned
    backward sums exactly (every partial sum and every order of adding them is exact in fp32)."""
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(1, 6000))
    indptr, col = _ragged_csr(rng, n)
    if col.size == 0:
        indptr, col = np.array([0] * n + [1], np.int32), np.zeros(1, np.int32)
    ps = int(rng.choice([1, 2, 3, 5, 8, 16, 31, 32, 64]))
    shift = int(rng.choice([3, 5, 8, 11, 14, 31]))
    dim = int(rng.choice([1, 2, 4, 6, 16, 22, 33, 64, 130]))
    api.set_plan_keep_rows(int(rng.choice([0, 1, 2, 8])))
    api.set_plan_length_classes(bool(rng.integers(0, 2)))
    try:
        ones = np.ones(n, np.float32)
        x = rng.integers(-4, 5, (n, dim)).astype(np.float32)
        pp, p2n = co.build_part(ps, indptr)
        plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n), block_shift=shift)
        check_stream_form(api, plan, n)
        out = torch.full((n, dim), float("nan"), device="cuda")
        api.spmm_forward(dev(x), dev(col), dev(ones), dev(pp), dev(p2n), part_size=ps, plan=plan, out=out)
        assert api.last_call_used_stream()
        what = f"seed {seed}: n {n}, slots {col.size}, group size {ps}, shift {shift}, width {dim}"
        assert np.array_equal(out.cpu().numpy(), co.spmm_f64(x, indptr, col, ones).astype(np.float32)), what

        # the pruned backward over the path of a random source mask
        src = rng.random(n) < rng.uniform(0.02, 0.9)
        mask = torch.full((col.size,), -1, dtype=torch.int32, device="cuda")
        degs = torch.zeros(n, dtype=torch.int32, device="cuda")
        api.mask_forward(dev(p2n), dev(pp), dev(col), dev(src), None, mask, degs, True)
        oid, oedge, v = api.compact_back_edge(mask, dev(col))
        if v == 0:
            return
        bps = int(rng.choice([1, 4, 16, 32]))
        bpp, p, _ = api.split_back_part(degs, col.size, bps)
        bitmap, _ = api.mark_gathered_rows(oedge, v, n)
        dy = x * src[:, None]
        poisoned = dy.copy()
        poisoned[~src] = np.nan
        bplan = api.build_plan(bpp, oedge, p, v, n, dim, ids=oid, block_shift=shift)
        check_stream_form(api, bplan, n)
        out.fill_(float("nan"))
        api.ours_backward(dev(poisoned), oid, bpp, oedge, dev(ones), p, part_size=bps, plan=bplan, gathered_rows=bitmap,
                          out=out)
        assert api.last_call_used_stream()
        assert np.array_equal(out.cpu().numpy(), co.spmm_f64(dy, indptr, col, ones).astype(np.float32)), what + " (backward)"
    finally:
        api.set_plan_keep_rows(None)
        api.set_plan_length_classes(None)


def test_replaced_plan_header_is_reported_not_silent(api):
    """A plan whose header in memory is no longer the one the library read there: the stream and fix-up kernels
    write nothing, leave a mark, and eppgcn_aggregation_status reports it once (-5); eppgcn_plan_status refuses
    bytes that are not a finished build's header; after a rebuild everything works again.  Every kernel exits
    normally throughout."""
    indptr, col = GRAPHS["hub"]()
    n = indptr.size - 1
    dim = 16
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(21)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    want = co.spmm_f64(x, indptr, col, s)
    bound = cf.abs_sum_bound(indptr, col, s, x)
    pp, p2n = co.build_part(8, indptr)
    args = (dev(col), dev(s), dev(pp), dev(p2n))
    lib = api.load()

    def call(plan, ws):
        out = torch.full((n, dim), -123.0, device="cuda")
        api.spmm_forward(dev(x), *args, part_size=8, out=out, plan=plan, workspace=ws)
        return out

    plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
    ws = api.feature_workspace(n, dim, "cuda", plan)
    out = call(plan, ws)
    assert api.last_call_used_stream()
    assert_close(out.cpu().numpy(), want, bound, "intact plan")
    api.aggregation_status()                                     # nothing to report

    header = plan.stream_view()["header"]
    saved = header.clone()
    for word, what in ((2, "num_partials"), (8, "generation"), (0, "valid"), (7, "magic")):
        header[word] += 1                                        # the plan's bytes change behind the library's back
        out = call(plan, ws)
        assert api.last_call_used_stream()                       # the host still believes in the plan it remembers
        assert bool((out == -123.0).all()), f"{what}: the kernels must not write through a header they do not know"
        with pytest.raises(api.EppgcnError, match="-5.*plan"):
            api.aggregation_status()
        api.aggregation_status()                                 # reported once
        header.copy_(saved)
        assert_close(call(plan, ws).cpu().numpy(), want, bound, f"{what} restored")
        api.aggregation_status()

    # plan_status takes on only the header of a finished build with these sizes
    status = lambda: lib.eppgcn_plan_status(plan.base_ptr, plan.num_parts, plan.num_slots, plan.num_nodes, None, None)
    header[7] = 0
    assert status() == -5 and b"does not hold a plan" in lib.eppgcn_last_error()
    header.copy_(saved)
    header[9] += 1                                               # another group count than the caller states
    assert status() == -5
    header.copy_(saved)
    # the plan is forgotten after a refused status: the group kernel runs over the (intact) group arrays
    out = call(plan, ws)
    assert not api.last_call_used_stream()
    assert_close(out.cpu().numpy(), want, bound, "forgotten plan")
    assert status() == 0
    assert_close(call(plan, ws).cpu().numpy(), want, bound, "known again")
    assert api.last_call_used_stream()

    # released: unknown to the library again; a rebuild into the same memory gets a new build number
    plan.release()
    plan2 = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
    assert plan2.stream_view()["header"][8].item() > int(saved[8])
    assert_close(call(plan2, api.feature_workspace(n, dim, "cuda", plan2)).cpu().numpy(), want, bound, "rebuilt")
    assert api.last_call_used_stream()
    api.aggregation_status()


@pytest.mark.parametrize("dim", [3, 16, 22, 40, 64, 100, 256])
def test_stream_kernel_with_64_bit_addressing_gives_the_same_bits(api, dim):
    """The variant for tables of 4 GB and more (64-bit global loads; lanes that a buffer load sends out of range
    load row 0 and count as zeros), forced at small size: the same bits as the 32-bit variant, every team size,
    padding slots and unused lanes included; and within tolerance of the checker."""
    indptr, col = GRAPHS["two hubs"]()
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(dim)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    pp, p2n = co.build_part(5, indptr)
    args = (dev(x), dev(col), dev(s), dev(pp), dev(p2n))
    api.set_plan_shift(11)
    plan = api.build_plan(dev(pp), dev(col), p2n.size, col.size, n, dim, part2node=dev(p2n))
    ws = api.feature_workspace(n, dim, "cuda", plan)
    ws.fill_(float("nan"))                       # row 0 and everything else the masked lanes may touch
    narrow = api.spmm_forward(*args, part_size=5, plan=plan, workspace=ws)
    assert api.last_call_used_stream()
    try:
        api.set_stream_mode(True, wide=True)
        out = torch.full((n, dim), float("nan"), device="cuda")
        api.spmm_forward(*args, part_size=5, plan=plan, workspace=ws, out=out)
        assert api.last_call_used_stream()
    finally:
        api.set_stream_mode(True)
    assert torch.equal(out, narrow), "64-bit and 32-bit addressing must agree bit for bit"
    assert_close(out.cpu().numpy(), co.spmm_f64(x, indptr, col, s), cf.abs_sum_bound(indptr, col, s, x), f"D={dim}")
