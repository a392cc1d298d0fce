"""GPU parity at the benchmark's own configurations, set up the way the benchmark sets its launches up.

* Backward-path stress (R-MAT scale 20; train-mask ratio {0.01, 0.1, 0.5} x aggregation width
  {16, 64, 256} x backward group size {8, 16, 32, 64}): all 36 cells, with the execution plans
  (column-blocked, or one block for heavily pruned paths) and the gathered-rows bitmap that
  ``eppgcn_amd.sweep`` and the extension module use.  Per cell: the compacted path against its closed
  form (bit-exact), integer data pruned == unpruned == int64 ``index_add_`` (bit-exact), float data
  with the symmetric normalisation within rel. tol. 1e-5 of a float64 sparse product on the device.
* Headline configuration (R-MAT scale 22): s = deg^-1/2, N(0,1) features, both forward widths and
  both pruned paths through the pre-scaled feature workspace (128-byte rows at width 22) with plans and
  the gathered-rows bitmap - i.e. exactly what ``bench.py`` times - against a float64 sparse product.

Tolerance: |got - want| <= 1e-5 * sum_j |w_ij x_j| per output element (a forward error bound of the
sum, the right yardstick for sums that cancel), written out in ``_assert_within``.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
RTOL = 1e-5

RATIOS = [0.01, 0.1, 0.5]
WIDTHS = [16, 64, 256]
GROUP_SIZES = [8, 16, 32, 64]


@pytest.fixture(scope="module")
def api():
    from eppgcn_amd import capi
    capi.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return capi


# ----------------------------------------------------------------------------- float64 references on the device
def _weighted_sums(row_pointers, col, w, x):
    """(sum_e w_e x[col_e], sum_e |w_e x[col_e]|) per output row in float64: the textbook sparse
    product A @ x of a float64 CSR matrix with the edge weights as values (torch.sparse.mm, i.e. the
    vendor's SpMM - an implementation that shares nothing with the kernels under test)."""
    n = row_pointers.numel() - 1
    crow = row_pointers.long()
    a = torch.sparse_csr_tensor(crow, col, w, size=(n, n))
    want = torch.sparse.mm(a, x.double())
    a_abs = torch.sparse_csr_tensor(crow, col, w.abs(), size=(n, n))
    bound = torch.sparse.mm(a_abs, x.double().abs())
    return want, bound


def _assert_within(got, want, bound, what):
    worst = ((got.double() - want).abs() / (RTOL * bound + 1e-30)).max().item()
    assert worst <= 1.0, f"{what}: max |err| / (1e-5 * sum|w x|) = {worst:.3f}"
    return worst


def _closed_form_part_pointer(degs, group_size, capacity):
    """part_pointer of split_back_part (EPPGCN/GCNConv/EPPGCN.cpp:327-346) from the kept degrees:
    row i with g_i > 0 kept slots starting at G_i yields groups at G_i + j * group_size."""
    g = degs.long()
    q = (g + group_size - 1) // group_size
    num_groups = int(q.sum())
    starts = torch.cumsum(g, 0) - g
    first_group = torch.cumsum(q, 0) - q
    owner = torch.repeat_interleave(torch.arange(g.numel(), device=g.device), q)
    j = torch.arange(num_groups, device=g.device) - first_group[owner]
    out = torch.zeros(capacity, dtype=torch.int32, device=g.device)
    out[:num_groups] = (starts[owner] + j * group_size).int()
    out[num_groups] = int(g.sum())
    return out, num_groups


# ----------------------------------------------------------------------------- backward-path stress, all 36 cells
class _Rmat20:
    """State shared by the cells: the graph, its forward groups and plans, and per mask ratio the marked and
    compacted path (checked once against its closed form)."""

    def __init__(self, api):
        from eppgcn_amd import graphs, param
        self.api, self.graphs = api, graphs
        self.g = graphs.make_graph("cfg3_rmat20", device="cuda")
        g = self.g
        self.n, self.e = g.num_nodes, g.num_edges
        self.ps = max(param.MIN_AUTO_PART_SIZE, int(g.avg_degree))
        self.pp, self.p2n = api.build_part(self.ps, g.row_pointers, self.e)
        self.row = g.row_index()
        self.col = g.column_index.long()
        self.ones = torch.ones(self.n, device="cuda")
        self.w = (g.degrees[self.row] * g.degrees[self.col]).double()
        self.fwd_plans, self.by_ratio, self.refs = {}, {}, {}

    def forward_plan(self, width):
        if not self.api.plan_recommended(self.n, width):
            return None
        if width not in self.fwd_plans:
            self.fwd_plans[width] = self.api.build_plan(self.pp, self.g.column_index, self.p2n.numel(), self.e,
                                                        self.n, width, part2node=self.p2n)
        return self.fwd_plans[width]

    def path(self, ratio):
        if ratio in self.by_ratio:
            return self.by_ratio[ratio]
        api, g, n, e = self.api, self.g, self.n, self.e
        mask = self.graphs.bernoulli_mask(n, ratio, 2, "cuda")
        bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
        degs = torch.zeros(n, dtype=torch.int32, device="cuda")
        api.mask_forward(self.p2n, self.pp, g.column_index, mask, None, bem, degs, True)
        ids, edge_list, v = api.compact_back_edge(bem, g.column_index)
        # closed form of marking + compaction: the slots whose column is in the mask, in CSR order
        keep = mask[self.col]
        assert torch.equal(bem != -1, keep) and torch.equal(bem[keep].long(), self.row[keep])
        assert v == int(keep.sum())
        assert torch.equal(ids[:v].long(), self.row[keep]) and torch.equal(edge_list[:v], g.column_index[keep])
        assert not ids[v:].any() and not edge_list[v:].any()
        assert torch.equal(torch.bincount(self.row[keep], minlength=n).int(), degs)
        # the one-pass preparation leaves the same lists
        degs2 = torch.zeros_like(degs)
        ids2, edge2, v2 = api.mark_compact(self.p2n, self.pp, g.column_index, mask, None, degs2, True)
        assert v2 == v and torch.equal(ids2, ids) and torch.equal(edge2, edge_list) and torch.equal(degs2, degs)
        bitmap, distinct = api.mark_gathered_rows(edge_list, v, n)
        assert distinct == int(torch.unique(edge_list[:v]).numel())
        gathered = bitmap if 2 * distinct < n else None
        self.by_ratio[ratio] = (mask, degs, ids, edge_list, v, api.count_nonzero(degs), gathered)
        return self.by_ratio[ratio]

    def reference(self, ratio, width):
        """float gradient (zero outside the mask) and its float64 aggregate + error yardstick."""
        key = (ratio, width)
        if key not in self.refs:
            self.refs.clear()                     # one (ratio, width) at a time: [N, 256] float64 is 2 GB
            mask = self.path(ratio)[0]
            dy = self.graphs.normal32(7, (self.n, width), "cuda") * mask[:, None]
            want, bound = _weighted_sums(self.g.row_pointers, self.col, self.w, dy)
            self.refs[key] = (dy, want, bound)
        return self.refs[key]


@pytest.fixture(scope="module")
def rmat20(api):
    state = _Rmat20(api)
    yield state
    state.refs.clear()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("group_size", GROUP_SIZES)
@pytest.mark.parametrize("width", WIDTHS)
@pytest.mark.parametrize("ratio", RATIOS)
def test_backward_stress_cell(api, rmat20, ratio, width, group_size):
    st = rmat20
    g, n, e = st.g, st.n, st.e
    mask, degs, ids, edge_list, v, valid_node, gathered = st.path(ratio)

    # ---- split into groups: bit-exact against the closed form, zero tail included
    part_pointer, num_parts, v2 = api.split_back_part(degs, e, group_size)
    want_pp, want_parts = _closed_form_part_pointer(degs, group_size, e + 1)
    assert (num_parts, v2) == (want_parts, v)
    assert torch.equal(part_pointer, want_pp)

    # ---- launch set-up of the sweep / the extension module
    plan = None
    if num_parts > 0 and api.plan_recommended(n, width):
        plan = api.build_plan(part_pointer, edge_list, num_parts, v, n, width, ids=ids,
                              block_shift=0 if 2 * v >= e else 31)
    # room for the partial sums of either plan: the calls run the plans' stream form
    ws = api.feature_workspace(n, width, "cuda", (plan, st.forward_plan(width)))

    def pruned(dy, scale, out=None):
        return api.ours_backward(dy, ids, part_pointer, edge_list, scale, num_parts, group_size, 1, 4, 16, out, ws,
                                 plan=plan, gathered_rows=gathered)

    def unpruned(dy, scale):
        return api.spmm_forward(dy, g.column_index, scale, st.pp, st.p2n, st.ps, 32, 8, None, None, True, ws,
                                plan=st.forward_plan(width))

    # ---- integer data, unit scale: every partial sum is exact, so the order cannot matter
    xi = (st.graphs.uniform32(9, torch.arange(n * width, device="cuda")) % 17 - 8).reshape(n, width).float()
    dyi = xi * mask[:, None]
    out = torch.full((n, width), float("nan"), device="cuda")       # the call must define every element
    got_i = pruned(dyi, st.ones, out)
    assert torch.equal(got_i, unpruned(dyi, st.ones)), "pruned != unpruned on integer data"
    want_i = torch.zeros(n, width, device="cuda")
    for lo in range(0, e, 1 << 23):
        hi = min(e, lo + (1 << 23))
        want_i.index_add_(0, st.row[lo:hi], dyi[st.col[lo:hi]])
    assert torch.equal(got_i, want_i), "pruned backward != index_add on integer data"
    # gradient rows outside the mask must not be read (the bitmap lets the scaling pass skip them)
    noisy = dyi + (~mask)[:, None] * 3.0
    assert torch.equal(pruned(noisy, st.ones), want_i), "rows outside the mask leaked into the result"
    del xi, dyi, noisy, want_i, got_i, out

    # ---- float data, s = deg^-1/2: within tolerance of the float64 sum
    dy, want, bound = st.reference(ratio, width)
    what = f"ratio {ratio} width {width} group size {group_size}"
    _assert_within(pruned(dy, g.degrees), want, bound, "pruned, " + what)
    assert api.last_call_used_stream() == (plan is not None)
    api.set_stream_mode(False)               # the group kernel over the same plan
    try:
        _assert_within(pruned(dy, g.degrees), want, bound, "pruned, group kernel, " + what)
        assert not api.last_call_used_stream()
    finally:
        api.set_stream_mode(True)
    if group_size == GROUP_SIZES[0]:
        _assert_within(unpruned(dy, g.degrees), want, bound, "unpruned, " + what)
        plain = api.ours_backward(dy, ids, part_pointer, edge_list, g.degrees, num_parts, group_size, workspace=None)
        _assert_within(plain, want, bound, "pruned without workspace or plan, " + what)


# ----------------------------------------------------------------------------- headline configuration, benched path
def test_headline_size_benched_numeric_path_within_tolerance(api):
    """R-MAT scale 22 as ``bench.py`` runs it: symmetric normalisation, N(0,1) inputs, feature workspace
    (pre-scaled rows, 128-byte pitch at width 22), column-blocked / one-block plans, gathered-rows bitmap;
    plus the training pipeline's variant in which the dense update writes the scaled table directly."""
    from eppgcn_amd import graphs, workload
    g = graphs.make_graph("cfg4_rmat22", device="cuda")
    n, e = g.num_nodes, g.num_edges
    wl = workload.prepare(g, 2, 0.1, 2)
    assert wl.plans and all(p.plan is not None for p in wl.paths), "plans are expected at this size"
    assert wl.paths[1].gathered_rows is not None, "the last layer's path gathers a tenth of the rows"
    row, col = g.row_index(), g.column_index.long()
    w = (g.degrees[row] * g.degrees[col]).double()
    worst = {}
    for dim, path, src in ((16, wl.paths[0], wl.ngh_masks[0]), (22, wl.paths[1], wl.train_mask)):
        ws = api.feature_workspace(n, dim, "cuda", (wl.plans[dim], path.plan))     # as bench.py sizes it
        x = graphs.normal32(1, (n, dim), "cuda", dim)
        want, bound = _weighted_sums(g.row_pointers, col, w, x)
        out = torch.full((n, dim), float("nan"), device="cuda")
        got = api.spmm_forward(x, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                               g.row_pointers, out, workspace=ws, plan=wl.plans[dim])
        assert api.last_call_used_stream(), "the benchmark's calls run the plans' stream form"
        worst[f"fwd{dim}"] = _assert_within(got, want, bound, f"planned forward, width {dim}")
        again = api.spmm_forward(x, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                                 g.row_pointers, None, workspace=ws, plan=wl.plans[dim])
        assert torch.equal(got, again), "the stream form sums in a fixed order"
        del again
        api.set_stream_mode(False)           # the group kernel over the same plan and workspace
        try:
            out.fill_(float("nan"))
            got = api.spmm_forward(x, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                                   g.row_pointers, out, workspace=ws, plan=wl.plans[dim])
            assert not api.last_call_used_stream()
            worst[f"fwd{dim}_groups"] = _assert_within(got, want, bound, f"planned forward, group kernel, width {dim}")
        finally:
            api.set_stream_mode(True)
        # the same launch fed by a table that is already scaled and padded (what the dense update leaves)
        pitch = api.feature_workspace_pitch(dim)
        table = torch.zeros(api.feature_workspace(n, dim, "cuda", wl.plans[dim]).numel() // pitch, pitch, device="cuda")
        table[api.feature_workspace_rows(n, "cuda"), :dim] = x * g.degrees[:, None]
        out.fill_(float("nan"))
        got = api.spmm_forward(None, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8,
                               g.row_pointers, out, workspace=table.view(-1), plan=wl.plans[dim], prescaled_dim=dim)
        worst[f"fwd{dim}_table"] = _assert_within(got, want, bound, f"forward from a scaled table, width {dim}")
        del table, want, bound

        dy = graphs.normal32(2, (n, dim), "cuda", dim) * src[:, None]
        want, bound = _weighted_sums(g.row_pointers, col, w, dy)
        out.fill_(float("nan"))
        ws.fill_(float("nan"))                   # rows the scaling pass skips must never be gathered
        got = api.ours_backward(dy, path.ids, path.part_pointer, path.edge_list, g.degrees, path.num_parts,
                                path.part_size, path.layer, 4, 16, out, workspace=ws, plan=path.plan,
                                gathered_rows=path.gathered_rows)
        assert api.last_call_used_stream()
        worst[f"bwd{dim}"] = _assert_within(got, want, bound, f"planned pruned backward, width {dim}")
        un = api.spmm_forward(dy, g.column_index, g.degrees, wl.part_ptr, wl.part2node, wl.part_size, 32, 8, None,
                              None, True, ws, plan=wl.plans[dim])
        _assert_within(un, want, bound, f"planned unpruned backward, width {dim}")
        # pruned and unpruned sum the same terms in different orders
        assert ((got - un).abs().double() <= 2 * RTOL * bound + 1e-30).all()
        del dy, want, bound, got, un, out, ws
    print("worst err / limit:", {k: round(v, 4) for k, v in worst.items()})


@pytest.mark.parametrize("ratio", [0.3, 0.8])
def test_mask_ratios_of_the_reference_sweep_at_size(api, rmat20, ratio):
    """The mask ratios the reference's own sweep adds to the benchmark's (EPPGCN/bench_EPPGCN.py:35: 0.1, 0.3, 0.5,
    0.8), on the R-MAT-20 graph at the widths of the 2-layer model: the same cell checks as above."""
    for width in (16, 22):
        test_backward_stress_cell(api, rmat20, ratio, width, 32)


# ----------------------------------------------------------------------------- more than 2^24 vertices
def test_stream_form_with_25_bit_vertex_ids(api):
    """R-MAT scale 25, one generated pair per vertex (33.5 M vertices, many of them isolated): vertex ids and the
    padding id need 25 bits.  At width 16 (64-byte rows, a 2 GB table) the stream form addresses rows with a
    shift; at width 22 the table passes 4 GB and the stream kernel addresses it with 64-bit loads.  Both against
    the float64 sparse product, and both the same bits on a second run."""
    from eppgcn_amd import graphs
    g = graphs.make_graph("rmat:25:1", device="cuda")
    n, e = g.num_nodes, g.num_edges
    assert n == 1 << 25 and int(g.column_index.max()) >= 1 << 24
    ps = 4
    part_ptr, part2node = api.build_part(ps, g.row_pointers, e)
    col = g.column_index.long()
    w = (g.degrees[g.row_index()] * g.degrees[col]).double()
    for dim, streams in ((16, True), (22, True)):
        plan = api.build_plan(part_ptr, g.column_index, part2node.numel(), e, n, dim, part2node=part2node)
        ws = api.feature_workspace(n, dim, "cuda", plan)
        x = graphs.normal32(3, (n, dim), "cuda", dim)
        want, bound = _weighted_sums(g.row_pointers, col, w, x)
        out = torch.full((n, dim), float("nan"), device="cuda")
        got = api.spmm_forward(x, g.column_index, g.degrees, part_ptr, part2node, ps, 32, 8, g.row_pointers, out,
                               workspace=ws, plan=plan)
        assert api.last_call_used_stream() == streams
        _assert_within(got, want, bound, f"planned forward at 2^25 vertices, width {dim}")
        if streams:
            again = api.spmm_forward(x, g.column_index, g.degrees, part_ptr, part2node, ps, 32, 8, g.row_pointers,
                                     None, workspace=ws, plan=plan)
            assert torch.equal(got, again), "the stream form sums in a fixed order"
            del again
        del plan, ws, x, want, bound, out, got
