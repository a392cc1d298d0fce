"""Shared input builders for the tests (numpy, CPU)."""
from __future__ import annotations

import numpy as np


def random_symmetric_csr(n: int, m: int, seed: int, self_loops: bool = True, isolated: float = 0.0):
    """Symmetric 0/1 graph with m random undirected pairs; returns int32 (indptr, col).
    ``isolated``: fraction of vertices whose edges (incl. self-loop) are removed, to
    exercise zero-degree rows."""
    rng = np.random.default_rng(seed)
    u = rng.integers(0, n, m)
    v = rng.integers(0, n, m)
    rows = np.concatenate([u, v])
    cols = np.concatenate([v, u])
    if self_loops:
        rows = np.concatenate([rows, np.arange(n)])
        cols = np.concatenate([cols, np.arange(n)])
    if isolated > 0:
        dead = rng.random(n) < isolated
        ok = ~(dead[rows] | dead[cols])
        rows, cols = rows[ok], cols[ok]
    keys = np.unique(rows.astype(np.int64) * n + cols)
    rows, cols = keys // n, keys % n
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(rows, minlength=n), out=indptr[1:])
    return indptr.astype(np.int32), cols.astype(np.int32)


def hub_csr(n: int, hub_degree: int, seed: int):
    """Vertex 0 is adjacent to hub_degree other vertices; everyone has a self-loop and a few
    random edges: a row far longer than any group size next to rows of degree 1-3."""
    rng = np.random.default_rng(seed)
    others = rng.choice(np.arange(1, n), size=hub_degree, replace=False)
    u = np.concatenate([np.zeros(hub_degree, np.int64), rng.integers(0, n, n // 2)])
    v = np.concatenate([others, rng.integers(0, n, n // 2)])
    rows = np.concatenate([u, v, np.arange(n)])
    cols = np.concatenate([v, u, np.arange(n)])
    keys = np.unique(rows.astype(np.int64) * n + cols)
    rows, cols = keys // n, keys % n
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(rows, minlength=n), out=indptr[1:])
    return indptr.astype(np.int32), cols.astype(np.int32)


def scale_inv_sqrt(indptr):
    deg = np.maximum(np.diff(indptr.astype(np.int64)), 1).astype(np.float64)
    return (1.0 / np.sqrt(deg)).astype(np.float32)


def scale_sqrt(indptr):
    deg = np.maximum(np.diff(indptr.astype(np.int64)), 1).astype(np.float64)
    return np.sqrt(deg).astype(np.float32)
