"""GPU parity of the dense layer update (X*W, G*W^T, X^T*G on the matrix cores) through the
C ABI against the CPU checker.  fp32 bar: |got - want| <= 1e-5 * sum_k |a_k b_k| per output
element (the checker accumulates in float64, so only summation order and product rounding of
the fp32 kernel remain)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from tests.helpers import random_symmetric_csr, scale_inv_sqrt

pytestmark = pytest.mark.gpu
RTOL = 1e-5


@pytest.fixture(scope="module")
def api():
    from eppgcn_amd import capi
    capi.load()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return capi


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(got, want, bound, what=""):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    lim = RTOL * bound + 1e-30
    worst = float(np.max(err / lim)) if err.size else 0.0
    assert worst <= 1.0, f"{what}: max err/limit = {worst:.3f}"


def data(n, k, m, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, k)).astype(np.float32)
    w = rng.uniform(-0.5, 0.5, (k, m)).astype(np.float32)
    g = rng.standard_normal((n, m)).astype(np.float32)
    s = rng.uniform(0.1, 2.0, n).astype(np.float32)
    return x, w, g, s


# rows x reduction length x output columns: tile edges (16 rows, 16 columns, 4*VW reduction
# steps), odd sizes (scalar loads), the benchmark's layer shapes, column slabs (> 128 columns)
SHAPES = [(1, 1, 1), (5, 3, 2), (16, 16, 16), (17, 96, 16), (1000, 16, 22), (1000, 22, 16), (4097, 96, 16),
          (300, 33, 40), (123, 130, 70), (64, 8, 150), (50, 257, 5), (40000, 96, 16)]


@pytest.mark.parametrize("n,k,m", SHAPES)
@pytest.mark.parametrize("relu", [False, True])
def test_update_forward_matches_checker(api, n, k, m, relu):
    x, w, _, s = data(n, k, m, 1)
    xa = np.maximum(x, 0) if relu else x
    bound = np.abs(xa).astype(np.float64) @ np.abs(w).astype(np.float64)
    got = api.update_forward(dev(x), dev(w), relu_input=relu).cpu().numpy()
    assert_close(got, co.update_forward(x, w, relu_input=relu), bound, "plain product")
    ld = api.feature_workspace_pitch(m)
    got = api.update_forward(dev(x), dev(w), scale=dev(s), relu_input=relu, ld_out=ld).cpu().numpy()
    assert got.shape == (n, ld) and not got[:, m:].any()
    assert_close(got[:, :m], co.update_forward(x, w, scale=s, relu_input=relu), bound * s[:, None], "scaled, padded")


@pytest.mark.parametrize("n,k,m", SHAPES)
def test_update_backward_input_matches_checker(api, n, k, m):
    x, w, g, _ = data(n, k, m, 2)
    bound = np.abs(g).astype(np.float64) @ np.abs(w).astype(np.float64).T
    got = api.update_backward_input(dev(g), dev(w)).cpu().numpy()
    assert_close(got, co.update_backward_input(g, w), bound, "no mask")
    got = api.update_backward_input(dev(g), dev(w), relu_ref=dev(x)).cpu().numpy()
    assert_close(got, co.update_backward_input(g, w, relu_ref=x), bound, "relu mask")
    assert not got[x <= 0].any()


@pytest.mark.parametrize("n,k,m", [(1, 1, 1), (5, 3, 2), (63, 16, 16), (1000, 16, 22), (1000, 22, 16),
                                   (4097, 96, 16), (300, 33, 40), (123, 130, 64), (70000, 96, 16), (300000, 16, 22)])
@pytest.mark.parametrize("relu", [False, True])
def test_update_backward_weight_matches_checker(api, n, k, m, relu):
    x, _, g, _ = data(n, k, m, 3)
    xa = np.maximum(x, 0) if relu else x
    bound = np.abs(xa).astype(np.float64).T @ np.abs(g).astype(np.float64)
    a = api.update_backward_weight(dev(x), dev(g), relu_input=relu)
    b = api.update_backward_weight(dev(x), dev(g), relu_input=relu)
    assert torch.equal(a, b), "the weight gradient must be bitwise reproducible"
    assert_close(a.cpu().numpy(), co.update_backward_weight(x, g, relu_input=relu), bound, "weight gradient")


# rows x layer inputs x gradient columns: the benchmark's hidden layer (16 -> 22), a 16 -> 16 hidden layer of the
# deeper models, tile edges and odd widths (every load width of the one-pass kernel), row counts around the 16-row
# steps and the waves' row ranges, and shapes outside the one-pass kernel (in_dim > 16, out_dim > 32)
@pytest.mark.parametrize("n,k,m", [(1, 1, 1), (5, 3, 2), (16, 16, 16), (17, 16, 22), (1000, 16, 22), (4097, 16, 16),
                                   (300, 13, 17), (123, 16, 32), (999, 8, 7), (65536, 16, 22), (300007, 16, 22),
                                   (1000, 96, 16), (500, 16, 40), (200, 33, 33)])
@pytest.mark.parametrize("relu", [False, True])
def test_update_backward_pair_equals_the_two_products(api, n, k, m, relu):
    """eppgcn_update_backward gives both gradients of a layer; for narrow layers from one pass over x and g.  Each
    product is formed exactly as the separate calls form it, so the results are the same bits, and they are held
    against the checker like those."""
    x, w, g, _ = data(n, k, m, 6)
    dx, dw = api.update_backward(dev(x), dev(w), dev(g), relu_input=relu)
    assert torch.equal(dx, api.update_backward_input(dev(g), dev(w), relu_ref=dev(x) if relu else None))
    assert torch.equal(dw, api.update_backward_weight(dev(x), dev(g), relu_input=relu))
    again = api.update_backward(dev(x), dev(w), dev(g), relu_input=relu)
    assert torch.equal(again[0], dx) and torch.equal(again[1], dw), "bitwise reproducible"
    xa = np.maximum(x, 0) if relu else x
    assert_close(dw.cpu().numpy(), co.update_backward_weight(x, g, relu_input=relu),
                 np.abs(xa).astype(np.float64).T @ np.abs(g).astype(np.float64), "weight gradient")
    assert_close(dx.cpu().numpy(), co.update_backward_input(g, w, relu_ref=x if relu else None),
                 np.abs(g).astype(np.float64) @ np.abs(w).astype(np.float64).T, "input gradient")
    if relu:
        assert not dx.cpu().numpy()[x <= 0].any()


def pack_rows(live):
    """bool[n] -> the int32 bitmap the masked products take (bit r of word r // 32)."""
    n = live.size
    padded = np.zeros((n + 31) // 32 * 32, bool)
    padded[:n] = live
    words = np.packbits(padded.reshape(-1, 32), axis=1, bitorder="little").view(np.uint32).reshape(-1)
    return dev(words.view(np.int32))


# the shapes of the pair test (one-pass kernel, the two separate kernels), a first layer (only d_w), and densities of
# the bitmap from "no row" over whole dead tiles to "every row"
@pytest.mark.parametrize("n,k,m", [(1, 1, 1), (5, 3, 2), (16, 16, 16), (17, 16, 22), (1000, 16, 22), (4097, 16, 16),
                                   (300, 13, 17), (999, 8, 7), (65536, 16, 22), (300007, 16, 22), (1000, 96, 16),
                                   (500, 16, 40), (200, 33, 33)])
@pytest.mark.parametrize("density", [0.0, 0.03, 0.4, 1.0])
def test_update_backward_rows_reads_only_the_marked_rows(api, n, k, m, density):
    """eppgcn_update_backward_rows (no counterpart in the reference beyond the sketch in its comments,
    EPPGCN_kernel.cu:607,616): with the gradient zero outside the marked rows the results are those of
    eppgcn_update_backward bit for bit; with NaN in the unmarked rows of the gradient AND of the layer input they
    still are - those rows are not read - and the unmarked rows of d_x are zeros.  Also without d_x."""
    x, w, g, _ = data(n, k, m, 8)
    rng = np.random.default_rng(n + k + m)
    live = rng.random(n) < density
    if density == 0.03 and n > 64:
        live[: n // 2] = False                          # whole tiles and whole wave ranges without a marked row
    g[~live] = 0.0
    rows = pack_rows(live)
    for relu in (False, True):
        want_dx, want_dw = api.update_backward(dev(x), dev(w), dev(g), relu_input=relu)
        dx, dw = api.update_backward_rows(dev(x), dev(w), dev(g), rows, relu_input=relu)
        assert torch.equal(dx, want_dx) and torch.equal(dw, want_dw), "zeros outside the marked rows"
        gp, xp = g.copy(), x.copy()
        gp[~live] = np.nan
        xp[~live] = np.nan
        dx, dw = api.update_backward_rows(dev(xp), dev(w), dev(gp), rows, relu_input=relu)
        assert torch.equal(dx, want_dx) and torch.equal(dw, want_dw), "NaN outside the marked rows"
        assert not dx.cpu().numpy()[~live].any()
        none, dw = api.update_backward_rows(dev(xp), None, dev(gp), rows, relu_input=relu, need_dx=False)
        assert none is None and torch.equal(dw, want_dw), "weight gradient alone"
        dx, dw = api.update_backward_rows(dev(x), dev(w), dev(g), None, relu_input=relu)
        assert torch.equal(dx, want_dx) and torch.equal(dw, want_dw), "no bitmap: every row"


def test_update_backward_pair_on_unaligned_views(api):
    """Gradient and input that start 4 or 8 bytes into an allocation: the one-pass kernel's narrower loads and
    scalar stores."""
    n, k, m = 777, 16, 22
    x, w, g, _ = data(n, k, m, 7)
    for shift in (1, 2):
        gflat = torch.empty(n * m + shift, dtype=torch.float32, device="cuda")
        gv = gflat[shift:].view(n, m)
        gv.copy_(dev(g))
        xflat = torch.empty(n * k + shift, dtype=torch.float32, device="cuda")
        xv = xflat[shift:].view(n, k)
        xv.copy_(dev(x))
        dx, dw = api.update_backward(xv, dev(w), gv, relu_input=True)
        assert torch.equal(dx, api.update_backward_input(gv, dev(w), relu_ref=xv))     # same views: same load widths
        assert torch.equal(dw, api.update_backward_weight(xv, gv, relu_input=True))
        bound = np.abs(g).astype(np.float64) @ np.abs(w).astype(np.float64).T
        assert_close(dx.cpu().numpy(), co.update_backward_input(g, w, relu_ref=x), bound, f"input gradient, shift {shift}")


def test_update_handles_unaligned_views(api):
    """Operands that start 4 bytes into an allocation take the narrower load paths."""
    n, k, m = 777, 22, 16
    x, w, g, _ = data(n, k, m, 4)
    flat = torch.empty(n * k + 1, dtype=torch.float32, device="cuda")
    xv = flat[1:].view(n, k)
    xv.copy_(dev(x))
    bound = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64)
    assert_close(api.update_forward(xv, dev(w)).cpu().numpy(), co.update_forward(x, w), bound, "forward")
    bw = np.abs(x).astype(np.float64).T @ np.abs(g).astype(np.float64)
    assert_close(api.update_backward_weight(xv, dev(g)).cpu().numpy(), co.update_backward_weight(x, g), bw, "weight")


def test_update_rejects_unsupported_shapes(api):
    x = torch.zeros((4, 5000), device="cuda")
    w = torch.zeros((5000, 3), device="cuda")
    with pytest.raises(api.EppgcnError, match="inner dimension"):
        api.update_forward(x, w)
    with pytest.raises(api.EppgcnError, match="64 gradient columns"):
        api.update_backward_weight(torch.zeros((4, 3), device="cuda"), torch.zeros((4, 65), device="cuda"))
    with pytest.raises(api.EppgcnError):
        api.update_forward(torch.zeros((4, 3), device="cuda"), torch.zeros((4, 3), device="cuda"))


@pytest.mark.parametrize("dim", [16, 22, 7, 40])
def test_aggregation_accepts_the_prescaled_product(api, dim):
    """update_forward_table (scaled rows at the workspace's pitch and in its row order) followed by the
    aggregation with a NULL input equals the aggregation of the unscaled product."""
    indptr, col = random_symmetric_csr(5000, 30000, 21)
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    x, w, _, _ = data(n, 24, dim, 6)
    pp, p2n = api.build_part(8, dev(indptr), col.size)
    ws = api.update_forward_table(dev(x), dev(w), dev(s))
    # the table is the plain scaled product, row r at row feature_workspace_rows()[r], zeros in the padding
    pitch = api.feature_workspace_pitch(dim)
    plain = api.update_forward(dev(x), dev(w), scale=dev(s), ld_out=pitch)
    assert torch.equal(ws.view(-1, pitch)[api.feature_workspace_rows(n, "cuda")], plain)
    got = api.spmm_forward(None, dev(col), dev(s), pp, p2n, part_size=8, workspace=ws, prescaled_dim=dim)
    t = co.update_forward(x, w)
    want = co.spmm_f64(t, indptr, col, s)
    bound = co.spmm_f64(np.abs(t), indptr, col, s) + 1e-30
    # two fp32 stages: the product (relative to |x||w|) and the aggregation of its result
    tb = (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64)).astype(np.float32)
    bound = bound + co.spmm_f64(tb, indptr, col, s)
    assert_close(got.cpu().numpy(), want, bound, f"prescaled aggregation, width {dim}")


def test_update_products_on_random_shapes(api):
    """Property-based: any shape the kernels accept (rows 1-400, reduction length 1-1024, 1-150
    result columns, 1-64 for the weight gradient), with and without the ReLU on load, the row
    scale, a padded result pitch and the ReLU mask of the input gradient, stays within tolerance
    of the float64-accumulated checker."""
    from hypothesis import HealthCheck, given, settings
    from hypothesis import strategies as st

    @settings(max_examples=120, deadline=None, derandomize=True, database=None, suppress_health_check=list(HealthCheck))
    @given(st.integers(1, 400), st.one_of(st.integers(1, 40), st.integers(41, 1024)), st.integers(1, 150),
           st.booleans(), st.integers(0, 2 ** 31 - 1))
    def check(n, k, m, relu, seed):
        x, w, g, s = data(n, k, m, seed)
        xa = np.maximum(x, 0) if relu else x
        bound = np.abs(xa).astype(np.float64) @ np.abs(w).astype(np.float64)
        ld = api.feature_workspace_pitch(m)
        got = api.update_forward(dev(x), dev(w), scale=dev(s), relu_input=relu, ld_out=ld).cpu().numpy()
        assert not got[:, m:].any()
        assert_close(got[:, :m], co.update_forward(x, w, scale=s, relu_input=relu), bound * s[:, None], "forward")
        gb = np.abs(g).astype(np.float64) @ np.abs(w).astype(np.float64).T
        got = api.update_backward_input(dev(g), dev(w), relu_ref=dev(x) if relu else None).cpu().numpy()
        assert_close(got, co.update_backward_input(g, w, relu_ref=x if relu else None), gb, "input gradient")
        if m <= 64:
            wb = np.abs(xa).astype(np.float64).T @ np.abs(g).astype(np.float64)
            got = api.update_backward_weight(dev(x), dev(g), relu_input=relu).cpu().numpy()
            assert_close(got, co.update_backward_weight(x, g, relu_input=relu), wb, "weight gradient")

    check()
