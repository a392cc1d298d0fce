"""Pins the floating-point half of the CPU checker: neighbour-group aggregation (forward and
unpruned backward share it) and the pruned backward.  No reference fixture exists for them, so
they are pinned by dense float64 algebra on tiny graphs, scipy's CSR product on the benchmark's
small configurations, exact special cases, and the pruned == unpruned-on-masked-gradients
identity the technique rests on.

Tolerance: fp32 results are compared with the float64 sum through
|got - want| <= 1e-5 * sum_j |w_ij x_j|  (the north-star's rel. tol. 1e-5, measured against the
magnitude fp32 summation error scales with, so that cancellation inside a row cannot fail it)."""
import numpy as np
import pytest

from oracle import c_oracle as co
from oracle import closed_forms as cf
from tests.helpers import hub_csr, random_symmetric_csr, scale_inv_sqrt, scale_sqrt

RTOL = 1e-5


def assert_close(got, want64, bound, rtol=RTOL):
    err = np.abs(got.astype(np.float64) - want64)
    lim = rtol * bound + 1e-30
    worst = np.max(err / lim) if err.size else 0.0
    assert worst <= 1.0, f"max err/limit = {worst:.3f}"


@pytest.mark.parametrize("dim", [1, 16, 22, 64])
@pytest.mark.parametrize("scale_fn", [scale_inv_sqrt, scale_sqrt])
def test_group_spmm_vs_dense64(tiny_graphs, dim, scale_fn):
    rng = np.random.default_rng(dim)
    for indptr, col in tiny_graphs:
        n = indptr.size - 1
        s = scale_fn(indptr)
        x = rng.standard_normal((n, dim)).astype(np.float32)
        want = cf.aggregate_dense64(indptr, col, s, x)
        bound = cf.abs_sum_bound(indptr, col, s, x)
        assert np.allclose(co.spmm_f64(x, indptr, col, s), want, rtol=1e-12, atol=1e-12)
        assert np.allclose(cf.aggregate_csr64(indptr, col, s, x), want, rtol=1e-12, atol=1e-12)
        for ps in (1, 3, 32):
            pp, p2n = co.build_part(ps, indptr)
            assert_close(co.spmm_groups(x, col, s, pp, p2n, n), want, bound)
            assert_close(co.spmm_groups(x, col, s, pp, p2n, n, threads=True), want, bound)


def test_group_spmm_unit_scale_integer_features_is_exact_neighbour_sum():
    indptr, col = hub_csr(300, 200, 3)
    n = 300
    x = np.random.default_rng(0).integers(-8, 9, (n, 22)).astype(np.float32)
    s = np.ones(n, np.float32)
    want = np.zeros((n, 22), np.float64)
    np.add.at(want, cf.row_index(indptr), x[col].astype(np.float64))
    for ps in (1, 4, 32):
        pp, p2n = co.build_part(ps, indptr)
        got = co.spmm_groups(x, col, s, pp, p2n, n)
        assert np.array_equal(got.astype(np.float64), want)   # small integers: fp32 sums are exact


def test_group_spmm_identity_graph_is_two_roundings():
    n, dim = 50, 16
    indptr = np.arange(n + 1, dtype=np.int32)
    col = np.arange(n, dtype=np.int32)
    rng = np.random.default_rng(2)
    s = rng.uniform(0.1, 3.0, n).astype(np.float32)
    x = rng.standard_normal((n, dim)).astype(np.float32)
    pp, p2n = co.build_part(4, indptr)
    got = co.spmm_groups(x, col, s, pp, p2n, n)
    want = ((s * s).astype(np.float32)[:, None] * x).astype(np.float32)   # fl(fl(s*s) * x)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("cfg", ["cfg1_uniform", "cfg2_chunglu"])
@pytest.mark.parametrize("dim", [16, 22])
def test_group_spmm_vs_scipy_on_benchmark_graphs(cfg, dim):
    from eppgcn_amd import graphs
    g = graphs.make_graph(cfg)
    indptr, col, s = g.row_pointers.numpy(), g.column_index.numpy(), g.degrees.numpy()
    x = graphs.normal32(1, (g.num_nodes, dim)).numpy()
    want = cf.aggregate_csr64(indptr, col, s, x)
    bound = cf.abs_sum_bound(indptr, col, s, x)
    ps = max(1, int(g.avg_degree))
    pp, p2n = co.build_part(ps, indptr)
    got = co.spmm_groups(x, col, s, pp, p2n, g.num_nodes)
    assert_close(got, want, bound)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel < 1e-6


def _pruned(indptr, col, s, src, dy, ps, threads=False):
    oid, oedge, pp, v, p, degs = cf.pruned_path(indptr, col, src, ps)
    return co.ours_backward(dy, oid, pp, oedge, s, p, threads=threads)


@pytest.mark.parametrize("dim", [16, 22])
@pytest.mark.parametrize("ratio", [0.0, 0.1, 0.5, 1.0])
def test_pruned_backward_equals_unpruned_on_masked_gradients(dim, ratio):
    rng = np.random.default_rng(int(ratio * 10) + dim)
    for indptr, col in [random_symmetric_csr(150, 400, 1), hub_csr(500, 300, 2),
                        random_symmetric_csr(200, 300, 3, isolated=0.3)]:
        n = indptr.size - 1
        s = scale_inv_sqrt(indptr)
        src = rng.random(n) < ratio
        dy = rng.standard_normal((n, dim)).astype(np.float32) * src[:, None]
        want = cf.aggregate_csr64(indptr, col, s, dy)       # full A dY: masked rows of dY are zero
        bound = cf.abs_sum_bound(indptr, col, s, dy)
        for ps in (1, 8, 64):
            assert_close(_pruned(indptr, col, s, src, dy, ps), want, bound)
        assert_close(_pruned(indptr, col, s, src, dy, 8, threads=True), want, bound)
        # and it really prunes: gradient rows outside the mask never reach the output
        noise = dy + (~src)[:, None] * 100.0
        assert np.array_equal(_pruned(indptr, col, s, src, noise.astype(np.float32), 8),
                              _pruned(indptr, col, s, src, dy, 8))


def test_pruned_backward_rows_without_kept_edges_are_zero():
    indptr, col = random_symmetric_csr(100, 150, 8)
    s = scale_sqrt(indptr)
    src = np.zeros(100, bool)
    src[[3, 50]] = True
    dy = np.ones((100, 16), np.float32)
    g = _pruned(indptr, col, s, src, dy, 4)
    touched = np.zeros(100, bool)
    touched[cf.row_index(indptr)[src[col]]] = True
    assert not g[~touched].any() and np.all(g[touched] != 0)
