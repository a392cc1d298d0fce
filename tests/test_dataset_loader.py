"""The data front-end against scipy's coo -> csr (what the reference's loader calls,
EPPGCN/dataset.py:107-108) on small files in both of the reference's formats."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from eppgcn_amd import dataset as ds


def pairs(n, m, seed):
    rng = np.random.default_rng(seed)
    src, dst = rng.integers(0, n, m), rng.integers(0, n, m)
    src[: m // 10] = src[m // 10: 2 * (m // 10)][: m // 10]      # some repeated pairs
    dst[: m // 10] = dst[m // 10: 2 * (m // 10)][: m // 10]
    return src, dst


def scipy_csr(src, dst, n):
    a = sp.coo_matrix((np.ones(src.size), (src, dst)), shape=(n, n)).tocsr()
    a.sum_duplicates()
    a.sort_indices()
    return a.indptr.astype(np.int32), a.indices.astype(np.int32)


@pytest.mark.parametrize("fmt", ["txt", "npz"])
def test_loader_matches_scipy_csr_and_reference_buffers(tmp_path, fmt):
    n, m = 57, 400
    src, dst = pairs(n - 1, m, 3)                       # vertex n-1 never appears in an edge
    src[0], dst[0] = n - 2, 0
    if fmt == "txt":
        path = str(tmp_path / "g.txt")
        np.savetxt(path, np.stack([src, dst], 1), fmt="%d")
        n_expected = int(max(src.max(), dst.max())) + 1   # a text file defines N by its largest id
    else:
        path = str(tmp_path / "g.npz")
        np.savez(path, src_li=src, dst_li=dst, num_nodes=n)
        n_expected = n
    mask = np.random.default_rng(1).random(n_expected) < 0.3
    ds.write_train_mask(str(tmp_path), 0.3, mask)
    d = ds.custom_dataset(path, str(tmp_path), 0.3, 8, 5, 3, load_from_txt=(fmt == "txt"), device="cpu")
    want_ptr, want_col = scipy_csr(src, dst, n_expected)
    assert d.num_nodes == n_expected
    assert np.array_equal(d.row_pointers.numpy(), want_ptr) and np.array_equal(d.column_index.numpy(), want_col)
    assert d.row_pointers.dtype == torch.int32 and d.column_index.dtype == torch.int32
    deg = np.maximum(np.diff(want_ptr), 1)
    assert np.allclose(d.degrees.numpy(), np.sqrt(deg), rtol=1e-7)
    assert np.array_equal(d.train_mask.numpy(), mask)
    assert d.x.shape == (n_expected, 8) and d.y.eq(1).all() and d.y.dtype == torch.long
    assert len(d.ngh_masks) == 2 and not any(t.any() for t in d.ngh_masks) and d.empty_mask.numel() == 0
    assert len(d.edge_masks) == 3 and all(t.eq(-1).all() and t.numel() == want_col.size for t in d.edge_masks)
    assert len(d.node_degs) == 3 and not any(t.any() for t in d.node_degs)
    assert int(d.val_mask.sum()) == int(n_expected * 0.3) and int(d.test_mask.sum()) == int(n_expected * 0.1)
    assert abs(d.avg_edgeSpan - np.mean(np.abs(src - dst))) < 1e-9


def test_loader_errors(tmp_path):
    np.savez(str(tmp_path / "g.npz"), src_li=np.array([0, 5]), dst_li=np.array([1, 2]), num_nodes=3)
    with pytest.raises(ValueError, match="outside"):
        ds.read_edge_list(str(tmp_path / "g.npz"))
    with pytest.raises(ValueError, match="npz"):
        ds.custom_dataset(str(tmp_path / "g.txt"), str(tmp_path), 0.1, 4, 2, 2, load_from_txt=False, device="cpu")
    np.savetxt(str(tmp_path / "e.txt"), np.array([[0, 1], [1, 2]]), fmt="%d")
    ds.write_train_mask(str(tmp_path), 0.0, np.ones(5))
    with pytest.raises(ValueError, match="values for 3 vertices"):
        ds.custom_dataset(str(tmp_path / "e.txt"), str(tmp_path), 0.0, 4, 2, 2, device="cpu")


def test_inv_sqrt_scale_mode(tmp_path):
    np.savetxt(str(tmp_path / "e.txt"), np.array([[0, 1], [1, 0], [1, 2], [2, 1], [0, 0]]), fmt="%d")
    d = ds.custom_dataset(str(tmp_path / "e.txt"), str(tmp_path), 0.5, 4, 2, 2, device="cpu", scale_mode="inv_sqrt",
                          train_mask=torch.tensor([True, False, True]), feature_seed=7)
    assert np.allclose(d.degrees.numpy(), [2 ** -0.5, 2 ** -0.5, 1.0])
    assert torch.equal(d.x, ds.custom_dataset(str(tmp_path / "e.txt"), str(tmp_path), 0.5, 4, 2, 2, device="cpu",
                                               train_mask=torch.tensor([True, False, True]), feature_seed=7).x)


def test_degree_order_is_a_block_preserving_permutation_and_renumbering_keeps_the_graph():
    """``graphs.degree_order`` / ``graphs.renumber`` (CPU tensors): a permutation that keeps every vertex in
    its block of ids and orders the block by descending degree; the renumbered CSR is the same edge set under
    the new names, rows ascending, and the scale vector moves with the vertices."""
    import numpy as np
    import torch
    from eppgcn_amd import graphs
    g = graphs.chung_lu_graph(3000, 9000, 2.1, 5)
    new_id = graphs.degree_order(g, block_shift=9)
    n = g.num_nodes
    assert sorted(new_id.tolist()) == list(range(n))
    ident = torch.arange(n)
    assert torch.equal(new_id >> 9, ident >> 9)
    deg = (g.row_pointers[1:] - g.row_pointers[:-1]).long()
    by_new = torch.empty(n, dtype=torch.long)
    by_new[new_id] = deg
    for lo in range(0, n, 512):
        block = by_new[lo:lo + 512]
        assert bool((block[:-1] >= block[1:]).all())
    h = graphs.renumber(g, new_id)
    assert h.num_edges == g.num_edges and h.num_nodes == n
    rows = torch.repeat_interleave(ident, deg)
    old_pairs = set(zip(new_id[rows].tolist(), new_id[g.column_index.long()].tolist()))
    hrows = torch.repeat_interleave(ident, (h.row_pointers[1:] - h.row_pointers[:-1]).long())
    assert set(zip(hrows.tolist(), h.column_index.tolist())) == old_pairs
    cols = h.column_index.numpy()
    ptr = h.row_pointers.numpy()
    assert all(np.all(np.diff(cols[ptr[r]:ptr[r + 1]]) > 0) for r in range(n))
    assert torch.equal(h.degrees[new_id], g.degrees)
