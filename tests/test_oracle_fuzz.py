"""Property-based pinning of the CPU checker: on randomly drawn ragged graphs (empty rows, rows
longer than several groups, isolated vertices, duplicate-free sorted columns), masks of any
density and group sizes from 1 up, the C restatement must agree bit for bit with the numpy closed
forms on every integer result, and to float64 rounding with a dense matrix product on the
aggregation.  The fixed cases of the other checker tests pin known answers; this one looks for
the ragged shapes nobody thought of."""
import numpy as np
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

from oracle import c_oracle as co
from oracle import closed_forms as cf


@st.composite
def ragged_graph(draw):
    n = draw(st.one_of(st.integers(1, 40), st.integers(41, 700)))     # one wave's worth, or several
    seed = draw(st.integers(0, 2 ** 31 - 1))
    density = draw(st.sampled_from([0.0, 0.02, 0.1, 0.4, 1.0]))
    empty_rows = draw(st.sampled_from([0.0, 0.3, 0.9]))
    rng = np.random.default_rng(seed)
    adj = rng.random((n, n)) < density
    adj[rng.random(n) < empty_rows] = False
    indptr = np.concatenate([[0], np.cumsum(adj.sum(1))]).astype(np.int32)
    col = np.nonzero(adj)[1].astype(np.int32)
    return indptr, col, rng


COMMON = dict(max_examples=200, deadline=None, derandomize=True, database=None,
              suppress_health_check=[HealthCheck.too_slow])


@settings(**COMMON)
@given(ragged_graph(), st.integers(1, 9), st.integers(1, 9), st.sampled_from([0.0, 0.1, 0.5, 1.0]), st.booleans())
def test_integer_path_matches_the_closed_forms(graph, ps_fwd, ps_back, ratio, is_last):
    indptr, col, rng = graph
    n, e = indptr.size - 1, col.size
    pp, p2n = co.build_part(ps_fwd, indptr)
    pp2, p2n2 = cf.build_part(ps_fwd, indptr)
    assert np.array_equal(pp, pp2) and np.array_equal(p2n, p2n2)
    assert pp[-1] == e and (p2n.size == 0 or (np.diff(pp).min() >= 1 and np.diff(pp).max() <= ps_fwd))

    src = rng.random(n) < ratio
    ngh0 = rng.random(n) < 0.2
    degs0 = rng.integers(0, 3, n).astype(np.int32)          # marking adds to what is there
    ngh, bem, degs = (None if is_last else ngh0.copy()), np.full(e, -1, np.int32), degs0.copy()
    co.mask_forward(p2n, pp, col, src, ngh, bem, degs, is_last)
    w_ngh, w_bem, w_degs = cf.mask_forward(indptr, col, src, None if is_last else ngh0, np.full(e, -1, np.int32),
                                           degs0, is_last)
    assert np.array_equal(bem, w_bem) and np.array_equal(degs, w_degs)
    assert is_last or np.array_equal(ngh, w_ngh)

    oid, oedge, v = co.compact_mask(bem, col)
    w_id, w_edge, w_v = cf.compact_mask(bem, col)
    assert v == w_v and np.array_equal(oid, w_id) and np.array_equal(oedge, w_edge)
    assert np.all(np.diff(oid[:v]) >= 0) and not oid[v:].any() and not oedge[v:].any()

    kept = (degs - degs0).astype(np.int32)                    # what this marking pass added
    assert np.array_equal(np.bincount(oid[:v], minlength=n), kept)
    assert co.compact_count(kept) == cf.compact_count(kept) == int(np.count_nonzero(kept))
    bpp, p = co.split_back_part(kept, e, ps_back)
    w_bpp, w_p = cf.split_back_part(kept, e, ps_back)
    assert p == w_p and np.array_equal(bpp, w_bpp)
    assert bpp[p] == v and not bpp[p + 1:].any()
    for q in range(p):                                       # every group lies inside one row of the id list
        seg = oid[bpp[q]:bpp[q + 1]]
        assert 1 <= seg.size <= ps_back and seg.min() == seg.max()


@settings(**COMMON)
@given(ragged_graph(), st.integers(1, 9), st.integers(1, 7), st.sampled_from([0.0, 0.3, 1.0]))
def test_aggregation_matches_a_dense_product(graph, ps, dim, ratio):
    indptr, col, rng = graph
    n = indptr.size - 1
    s = rng.uniform(0.2, 1.5, n).astype(np.float32)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    a = np.zeros((n, n))
    rows = cf.row_index(indptr)
    a[rows, col] = (s[rows] * s[col]).astype(np.float32)     # the weight is rounded to fp32 first
    want = a @ x.astype(np.float64)
    bound = 1e-5 * (np.abs(a) @ np.abs(x).astype(np.float64)) + 1e-30
    pp, p2n = co.build_part(ps, indptr)
    assert np.all(np.abs(co.spmm_groups(x, col, s, pp, p2n, n) - want) <= bound)
    assert np.all(np.abs(co.spmm_f64(x, indptr, col, s) - want) <= 1e-12 * (1 + np.abs(want)))
    # pruned backward == the dense product with the columns outside the mask removed
    src = rng.random(n) < ratio
    oid, oedge, bpp, v, p, _ = cf.pruned_path(indptr, col, src, ps)
    want_b = (a * src[None, :]) @ x.astype(np.float64)
    got_b = co.ours_backward(x, oid, bpp, oedge, s, p)
    assert np.all(np.abs(got_b - want_b) <= bound)
