"""Data front-end: the reference's dataset object (EPPGCN/dataset.py:18-156) for its own file
formats, built on the device.

  graph file   ``.npz`` with ``src_li``, ``dst_li``, ``num_nodes`` (EPPGCN/dataset.py:79-93) or a
               text edge list, one ``src dst`` pair per line (EPPGCN/dataset.py:55-76)
  mask file    ``<dataPath>/train_mask`` (ratio 0.0) or ``<dataPath>/train_mask_<ratio>``: one
               0/1 value per vertex and line (EPPGCN/dataset.py:45-48)

The CSR is what scipy's ``coo_matrix(...).tocsr()`` gives there (rows ascending, columns
ascending within a row, duplicate pairs merged), computed with one sort on the device instead of
Python lists; the scale vector is the loader's ``sqrt(max(deg, 1))`` (EPPGCN/dataset.py:9-16,
118-119) unless ``scale_mode='inv_sqrt'`` asks for the symmetric GCN normalisation.  Per-run
buffers follow EPPGCN/dataset.py:135-156 except that ``edge_masks`` has one entry per CSR slot
(the reference sizes it by the number of input lines, which is larger when the file repeats
pairs; the path only ever touches the first nnz entries).
"""
from __future__ import annotations

import os

import numpy as np
import torch

from . import graphs


def read_edge_list(path: str):
    """-> (src int64 numpy, dst int64 numpy, num_nodes).  ``.npz`` or whitespace-separated text."""
    if path.endswith(".npz"):
        obj = np.load(path)                      # plain arrays only (allow_pickle stays False)
        src = np.asarray(obj["src_li"], dtype=np.int64)
        dst = np.asarray(obj["dst_li"], dtype=np.int64)
        num_nodes = int(obj["num_nodes"])
    else:
        pairs = np.loadtxt(path, dtype=np.int64, comments="#", ndmin=2)
        if pairs.size == 0:
            pairs = pairs.reshape(0, 2)
        if pairs.shape[1] < 2:
            raise ValueError(f"{path}: every line must hold 'src dst'")
        src, dst = pairs[:, 0].copy(), pairs[:, 1].copy()
        num_nodes = int(max(src.max(initial=-1), dst.max(initial=-1))) + 1
    if src.shape != dst.shape:
        raise ValueError(f"{path}: src and dst differ in length")
    if src.size and (min(src.min(), dst.min()) < 0 or max(src.max(), dst.max()) >= num_nodes):
        raise ValueError(f"{path}: vertex id outside [0, num_nodes)")
    return src, dst, num_nodes


def csr_from_directed_pairs(src: torch.Tensor, dst: torch.Tensor, num_nodes: int):
    """Directed pairs as given (no symmetrisation, no added self-loops), duplicates merged:
    int32 (row_pointers [N+1], column_index [nnz])."""
    n = int(num_nodes)
    keys = torch.unique(src.to(torch.int64) * n + dst.to(torch.int64))
    if keys.numel() >= 2 ** 31:
        raise ValueError("edge count does not fit the int32 CSR the aggregation path uses")
    rows = keys // n
    cols = (keys - rows * n).to(torch.int32)
    indptr = torch.zeros(n + 1, dtype=torch.int64, device=keys.device)
    torch.cumsum(torch.bincount(rows, minlength=n), 0, out=indptr[1:])
    return indptr.to(torch.int32), cols


def read_train_mask(data_path: str, ratio: float, num_nodes: int) -> np.ndarray:
    name = "train_mask" if ratio == 0.0 else "train_mask_" + str(ratio)
    mask = np.loadtxt(os.path.join(data_path, name), dtype=np.float64, ndmin=1)
    if mask.size != num_nodes:
        raise ValueError(f"{name} holds {mask.size} values for {num_nodes} vertices")
    return mask != 0


def write_train_mask(data_path: str, ratio: float, mask) -> str:
    """Writes a mask in the reference's file format (one 0/1 per line); returns the path."""
    name = "train_mask" if ratio == 0.0 else "train_mask_" + str(ratio)
    out = os.path.join(data_path, name)
    np.savetxt(out, np.asarray(mask).astype(np.int64), fmt="%d")
    return out


class custom_dataset(torch.nn.Module):
    """Same constructor arguments and attributes as the reference's class; ``device``,
    ``scale_mode``, ``feature_seed``, ``train_mask`` and ``degree_order`` are additions (a mask tensor
    given here replaces the mask file).

    ``degree_order=True`` renumbers the vertices after loading (``graphs.degree_order``: descending degree
    inside blocks of 2^17 ids, which the aggregation kernels reward with a few per cent); ``new_id`` then
    holds the new id of every vertex of the files, and the mask, the features and the labels are stored
    under the new ids.  Results for vertex v of the files are at row ``new_id[v]``."""

    def __init__(self, path, dataPath, ratio, dim, num_class, num_layer, load_from_txt=True, verbose=False,
                 device="cuda", scale_mode="sqrt", feature_seed=None, train_mask=None, degree_order=False):
        super().__init__()
        if not load_from_txt and not path.endswith(".npz"):
            raise ValueError("graph file must be a .npz file")
        self.load_from_txt = load_from_txt
        self.num_features, self.num_classes, self.num_layers = dim, num_class, num_layer
        self.verbose_flag = verbose
        src, dst, n = read_edge_list(path)
        self.num_nodes = n
        self.avg_edgeSpan = float(np.mean(np.abs(src - dst))) if src.size else 0.0
        self.row_pointers, self.column_index = csr_from_directed_pairs(
            torch.from_numpy(src).to(device), torch.from_numpy(dst).to(device), n)
        self.num_edges = int(self.column_index.numel())     # CSR entries (the reference: input lines)
        self.raw_num_edges = int(src.size)
        # the decider's automatic group size reads avg_degree, which the reference computes from the
        # number of input lines, repeated pairs included (EPPGCN/dataset.py:73,100)
        self.avg_degree = self.raw_num_edges / max(1, n)
        self.degrees = graphs.scale_vector(self.row_pointers, scale_mode)
        if verbose:
            print(f"# nodes: {n}\n# avg_degree: {self.avg_degree:.2f}\n# avg_edgeSpan: {int(self.avg_edgeSpan)}")
        # EPPGCN/dataset.py:121-133: N(0,1) features, every label 1
        self.x = (torch.randn(n, dim, device=device) if feature_seed is None
                  else graphs.normal32(feature_seed, (n, dim), device))
        self.y = torch.ones(n, dtype=torch.long, device=device)
        if train_mask is None:
            train_mask = torch.from_numpy(read_train_mask(dataPath, ratio, n))
        self.train_mask = train_mask.to(device=device, dtype=torch.bool)
        if self.train_mask.numel() != n:
            raise ValueError("train_mask must have one entry per vertex")
        self.new_id = None
        if degree_order:
            g = self.graph()
            self.new_id = graphs.degree_order(g)
            g = graphs.renumber(g, self.new_id)
            self.row_pointers, self.column_index, self.degrees = g.row_pointers, g.column_index, g.degrees
            for name in ("x", "y", "train_mask"):
                old = getattr(self, name)
                moved = torch.empty_like(old)
                moved[self.new_id] = old
                setattr(self, name, moved)
        self._init_masks(device)

    def _init_masks(self, device):
        n, e, layers = self.num_nodes, self.num_edges, self.num_layers
        head = lambda frac: torch.arange(n, device=device) < int(n * frac)   # EPPGCN/dataset.py:136-139
        self.val_mask, self.test_mask = head(0.3), head(0.1)
        self.ngh_masks = [torch.zeros(n, dtype=torch.bool, device=device) for _ in range(layers - 1)]
        self.empty_mask = torch.zeros(0, dtype=torch.bool, device=device)
        self.edge_masks = [torch.full((e,), -1, dtype=torch.int32, device=device) for _ in range(layers)]
        self.node_degs = [torch.zeros(n, dtype=torch.int32, device=device) for _ in range(layers)]

    def graph(self, name="dataset") -> graphs.Graph:
        return graphs.Graph(name, self.num_nodes, self.row_pointers, self.column_index, self.degrees)
