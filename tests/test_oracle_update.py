"""Pins the checker's restatement of the dense layer update (the three matrix products around
the aggregation) against numpy's float64 matrix product, a library routine independent of it,
on shapes where a transposed operand, a wrong leading dimension or a forgotten activation
changes the result."""
import numpy as np
import pytest

from oracle import c_oracle as co

def close(got, want, limit):
    err = np.abs(np.asarray(got, np.float64) - want)
    assert np.all(err <= limit), f"max err/limit = {np.max(err / limit):.3f}"


SHAPES = [(1, 1, 1), (5, 3, 2), (33, 96, 16), (40, 16, 22), (17, 22, 16), (9, 7, 40)]


def data(n, k, m, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, k)).astype(np.float32)
    w = rng.uniform(-0.5, 0.5, (k, m)).astype(np.float32)
    g = rng.standard_normal((n, m)).astype(np.float32)
    s = rng.uniform(0.1, 2.0, n).astype(np.float32)
    return x, w, g, s


@pytest.mark.parametrize("n,k,m", SHAPES)
@pytest.mark.parametrize("relu", [False, True])
def test_update_forward_is_the_scaled_matrix_product(n, k, m, relu):
    x, w, _, s = data(n, k, m, 1)
    xa = np.maximum(x, 0) if relu else x
    want = xa.astype(np.float64) @ w.astype(np.float64)
    got = co.update_forward(x, w, relu_input=relu)
    close(got, want, 2e-7 * np.abs(xa).astype(np.float64) @ np.abs(w) + 1e-30)
    ld = m + 5
    got = co.update_forward(x, w, scale=s, relu_input=relu, ld_out=ld)
    assert got.shape == (n, ld) and not got[:, m:].any()          # padding columns are exact zeros
    ws = want * s[:, None].astype(np.float64)
    close(got[:, :m], ws, 3e-7 * np.abs(ws) + 2e-7 * s[:, None] * (np.abs(xa).astype(np.float64) @ np.abs(w)) + 1e-30)


@pytest.mark.parametrize("n,k,m", SHAPES)
def test_update_backward_input_is_g_times_w_transposed(n, k, m):
    x, w, g, _ = data(n, k, m, 2)
    want = g.astype(np.float64) @ w.astype(np.float64).T
    close(co.update_backward_input(g, w), want, 2e-7 * (np.abs(g).astype(np.float64) @ np.abs(w).T) + 1e-30)
    got = co.update_backward_input(g, w, relu_ref=x)
    close(got, want * (x > 0), 2e-7 * (np.abs(g).astype(np.float64) @ np.abs(w).T) + 1e-30)
    assert not got[x <= 0].any()


@pytest.mark.parametrize("n,k,m", SHAPES)
@pytest.mark.parametrize("relu", [False, True])
def test_update_backward_weight_is_x_transposed_times_g(n, k, m, relu):
    x, _, g, _ = data(n, k, m, 3)
    xa = np.maximum(x, 0) if relu else x
    want = xa.astype(np.float64).T @ g.astype(np.float64)
    close(co.update_backward_weight(x, g, relu_input=relu), want, 2e-7 * (np.abs(xa).astype(np.float64).T @ np.abs(g)) + 1e-30)


def test_update_products_are_the_gradients_of_the_forward_product():
    """d/dW and d/dX of sum(C * (relu(X) @ W)) by central differences in float64."""
    rng = np.random.default_rng(5)
    n, k, m = 6, 5, 4
    x = rng.standard_normal((n, k)).astype(np.float32)
    w = rng.standard_normal((k, m)).astype(np.float32)
    c = rng.standard_normal((n, m)).astype(np.float32)

    def loss(xx, ww):
        return float(np.sum(c.astype(np.float64) * (np.maximum(xx, 0) @ ww)))

    eps = 1e-6
    dw = np.zeros((k, m)); dx = np.zeros((n, k))
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    for a in range(k):
        for b in range(m):
            e = np.zeros((k, m)); e[a, b] = eps
            dw[a, b] = (loss(x64, w64 + e) - loss(x64, w64 - e)) / (2 * eps)
    for a in range(n):
        for b in range(k):
            e = np.zeros((n, k)); e[a, b] = eps
            dx[a, b] = (loss(x64 + e, w64) - loss(x64 - e, w64)) / (2 * eps)
    np.testing.assert_allclose(co.update_backward_weight(x, c, relu_input=True), dw, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(co.update_backward_input(c, w, relu_ref=x), dx, rtol=1e-4, atol=1e-5)
