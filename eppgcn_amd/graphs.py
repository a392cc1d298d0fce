"""Seeded synthetic graphs for the five benchmark configurations.

Every generator is built on one counter-based integer hash evaluated with
torch int64 arithmetic, so the same (seed, index) pair yields the same draw
on the CPU and on the GPU: a graph generated on the GPU box is bit-identical
to the one a CPU test generates.

Graph contract (what the reference's loader hands to the aggregation path,
EPPGCN/dataset.py:100-119): an int32 CSR (``row_pointers`` [N+1],
``column_index`` [E]) with column indices sorted and de-duplicated inside each
row (scipy ``coo.tocsr()`` semantics) and a per-vertex fp32 scale vector
``degrees``.  All graphs here are symmetric and carry one self-loop per vertex.
"""
from __future__ import annotations

import dataclasses
import math

import torch

_MASK64 = (1 << 64) - 1


def _i64(x: int) -> int:
    """Reinterpret an unsigned 64-bit constant as the signed value torch stores."""
    x &= _MASK64
    return x - (1 << 64) if x >= (1 << 63) else x


_GOLDEN = _i64(0x9E3779B97F4A7C15)
_MIX1 = _i64(0xBF58476D1CE4E5B9)
_MIX2 = _i64(0x94D049BB133111EB)


def _lsr(x: torch.Tensor, k: int) -> torch.Tensor:
    """Logical shift right of an int64 tensor (torch's >> is arithmetic)."""
    return (x >> k) & ((1 << (64 - k)) - 1)


def hash64(seed: int, idx: torch.Tensor, stream: int = 0) -> torch.Tensor:
    """splitmix64 finaliser of (seed, stream, idx); int64 in, int64 out (all 64 bits random)."""
    z = idx * _GOLDEN + _i64(seed * 0xD1342543DE82EF95 + stream * 0xA0761D6478BD642F + 0x1234567)
    z = (z ^ _lsr(z, 30)) * _MIX1
    z = (z ^ _lsr(z, 27)) * _MIX2
    return z ^ _lsr(z, 31)


def uniform32(seed: int, idx: torch.Tensor, stream: int = 0) -> torch.Tensor:
    """Uniform integers in [0, 2^32) as int64."""
    return _lsr(hash64(seed, idx, stream), 32)


def uniform01(seed: int, idx: torch.Tensor, stream: int = 0) -> torch.Tensor:
    """Uniform float64 in [0, 1) with 53 random bits."""
    return _lsr(hash64(seed, idx, stream), 11).to(torch.float64) * (1.0 / (1 << 53))


def normal32(seed: int, shape, device="cpu", stream: int = 0) -> torch.Tensor:
    """fp32 N(0,1) draws (Box-Muller on hashed uniforms), identical on every device."""
    n = 1
    for s in shape:
        n *= int(s)
    out = torch.empty(n, dtype=torch.float32, device=device)
    chunk = 1 << 24
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        idx = torch.arange(lo, hi, dtype=torch.int64, device=device)
        u1 = uniform01(seed, idx, stream * 2 + 101)
        u2 = uniform01(seed, idx, stream * 2 + 102)
        r = torch.sqrt(-2.0 * torch.log1p(-u1))
        out[lo:hi] = (r * torch.cos(2.0 * math.pi * u2)).to(torch.float32)
    return out.reshape(*shape)


@dataclasses.dataclass
class Graph:
    """int32 CSR + scale vector, all on one device."""

    name: str
    num_nodes: int
    row_pointers: torch.Tensor  # int32 [N+1]
    column_index: torch.Tensor  # int32 [E]
    degrees: torch.Tensor       # fp32 [N]  per-vertex scale s (weight of edge i->j is s_i*s_j)

    @property
    def num_edges(self) -> int:
        return int(self.column_index.numel())

    @property
    def avg_degree(self) -> float:
        return self.num_edges / self.num_nodes

    def to(self, device) -> "Graph":
        return Graph(self.name, self.num_nodes, self.row_pointers.to(device),
                     self.column_index.to(device), self.degrees.to(device))

    def row_index(self) -> torch.Tensor:
        """Row id of every CSR slot (int64 [E])."""
        deg = (self.row_pointers[1:] - self.row_pointers[:-1]).to(torch.int64)
        return torch.repeat_interleave(
            torch.arange(self.num_nodes, device=deg.device, dtype=torch.int64), deg)

    def stats(self) -> dict:
        deg = (self.row_pointers[1:] - self.row_pointers[:-1])
        return {"name": self.name, "N": self.num_nodes, "E": self.num_edges,
                "avg_degree": round(self.avg_degree, 3), "max_degree": int(deg.max().item())}


def scale_vector(row_pointers: torch.Tensor, mode: str = "inv_sqrt") -> torch.Tensor:
    """Per-vertex scale s.

    ``inv_sqrt``: s = deg^-1/2, the symmetric GCN normalisation 1/sqrt(d_i d_j).
    ``sqrt``    : s = sqrt(max(deg,1)), the filling of the reference's own loader
                  (EPPGCN/dataset.py:9-16,118-119).
    The scale is computed in float64 and rounded once to fp32.
    """
    deg = (row_pointers[1:] - row_pointers[:-1]).to(torch.float64).clamp_(min=1.0)
    if mode == "inv_sqrt":
        return deg.rsqrt().to(torch.float32)
    if mode == "sqrt":
        return deg.sqrt().to(torch.float32)
    raise ValueError(f"unknown scale mode {mode!r}")


def csr_from_pairs(name: str, src: torch.Tensor, dst: torch.Tensor, num_nodes: int,
                   scale_mode: str = "inv_sqrt") -> Graph:
    """Symmetrise, add self-loops, sort and de-duplicate; return the int32 CSR."""
    device = src.device
    n = int(num_nodes)
    src = src.to(torch.int64)
    dst = dst.to(torch.int64)
    loops = torch.arange(n, dtype=torch.int64, device=device)
    keys = torch.cat([src * n + dst, dst * n + src, loops * n + loops])
    del src, dst
    keys = torch.unique(keys)  # sorted ascending -> rows ascending, columns ascending in a row
    if keys.numel() >= 2 ** 31:
        raise ValueError("edge count does not fit the int32 CSR the aggregation path uses")
    rows = keys // n
    cols = (keys - rows * n).to(torch.int32)
    del keys
    counts = torch.bincount(rows, minlength=n)
    del rows
    indptr = torch.zeros(n + 1, dtype=torch.int64, device=device)
    torch.cumsum(counts, 0, out=indptr[1:])
    indptr = indptr.to(torch.int32)
    return Graph(name, n, indptr, cols, scale_vector(indptr, scale_mode))


def degree_order(graph: Graph, block_shift: int = 17) -> torch.Tensor:
    """new_id int64[N]: a renumbering of the vertices in which, inside every aligned block of
    2^block_shift ids, the vertices come in order of descending degree (ties: old order).  Vertices stay
    in their block, so anything that depends on the coarse position of an id is unchanged.

    Why a caller may want it: the aggregation kernels gather feature rows by vertex id; with the rows of
    one block ordered by degree the hot 64-byte rows share 128-byte lines and the rows are processed and
    written in an order that follows their length (forward aggregation of an R-MAT scale-22 graph on an
    MI355X: -3.7 % at width 16, -3.1 % at width 22).  The numbering of the vertices is the caller's, so
    this is offered to the caller and never applied behind its back."""
    n = graph.num_nodes
    dev = graph.row_pointers.device
    deg = (graph.row_pointers[1:] - graph.row_pointers[:-1]).to(torch.int64)
    ident = torch.arange(n, dtype=torch.int64, device=dev)
    order = torch.argsort((ident >> block_shift) * (1 << 32) + ((1 << 31) - deg), stable=True)
    new_id = torch.empty(n, dtype=torch.int64, device=dev)
    new_id[order] = ident
    return new_id


def renumber(graph: Graph, new_id: torch.Tensor) -> Graph:
    """The same graph with vertex v called new_id[v] (a permutation of 0..N-1): row new_id[r] holds the
    columns new_id[c] of the old row r, ascending; the scale vector moves with the vertices.  Per-vertex
    data of the caller moves the same way: ``x_new[new_id] = x_old``."""
    n = graph.num_nodes
    new_id = new_id.to(torch.int64)
    deg = (graph.row_pointers[1:] - graph.row_pointers[:-1]).to(torch.int64)
    rows = torch.repeat_interleave(torch.arange(n, device=new_id.device), deg)
    keys = torch.sort(new_id[rows] * n + new_id[graph.column_index.long()]).values
    del rows
    r = keys // n
    cols = (keys - r * n).to(torch.int32)
    del keys
    indptr = torch.zeros(n + 1, dtype=torch.int64, device=new_id.device)
    torch.cumsum(torch.bincount(r, minlength=n), 0, out=indptr[1:])
    degrees = torch.empty_like(graph.degrees)
    degrees[new_id] = graph.degrees
    return Graph(graph.name + "_renumbered", n, indptr.to(torch.int32), cols, degrees)


def _first_distinct_pairs(seed: int, n: int, want: int, draw, device) -> tuple:
    """First ``want`` distinct unordered non-loop pairs in draw order."""
    total = 0
    batch = max(1024, int(want * 1.3))
    seen_keys = torch.empty(0, dtype=torch.int64, device=device)
    seen_pos = torch.empty(0, dtype=torch.int64, device=device)
    while True:
        idx = torch.arange(total, total + batch, dtype=torch.int64, device=device)
        u, v = draw(idx)
        lo, hi = torch.minimum(u, v), torch.maximum(u, v)
        ok = lo != hi
        keys = torch.cat([seen_keys, (lo * n + hi)[ok]])
        pos = torch.cat([seen_pos, idx[ok]])
        # keep the earliest draw of every key
        order = torch.argsort(keys, stable=True)
        ks, ps = keys[order], pos[order]
        first = torch.ones_like(ks, dtype=torch.bool)
        first[1:] = ks[1:] != ks[:-1]
        seen_keys, seen_pos = ks[first], ps[first]
        total += batch
        if seen_keys.numel() >= want:
            break
    order = torch.argsort(seen_pos)[:want]
    k = seen_keys[order]
    return k // n, k % n


def uniform_graph(num_nodes: int = 2708, undirected_edges: int = 5278, seed: int = 0,
                  device="cpu", scale_mode: str = "inv_sqrt") -> Graph:
    """Config 1: distinct undirected pairs drawn uniformly, both directions + self-loops."""
    n = num_nodes

    def draw(idx):
        return uniform32(seed, idx, 1) % n, uniform32(seed, idx, 2) % n

    u, v = _first_distinct_pairs(seed, n, undirected_edges, draw, device)
    return csr_from_pairs(f"uniform_n{n}", u, v, n, scale_mode)


def chung_lu_graph(num_nodes: int = 19717, undirected_edges: int = 44325, exponent: float = 2.1,
                   seed: int = 0, device="cpu", scale_mode: str = "inv_sqrt") -> Graph:
    """Config 2: Chung-Lu power-law graph, expected degree of rank r proportional to r^(-1/(exponent-1))."""
    n = num_nodes
    w = torch.arange(1, n + 1, dtype=torch.float64, device=device) ** (-1.0 / (exponent - 1.0))
    cdf = torch.cumsum(w, 0)
    cdf = cdf / cdf[-1]

    def draw(idx):
        u = torch.searchsorted(cdf, uniform01(seed, idx, 1)).clamp_(max=n - 1)
        v = torch.searchsorted(cdf, uniform01(seed, idx, 2)).clamp_(max=n - 1)
        return u, v

    u, v = _first_distinct_pairs(seed, n, undirected_edges, draw, device)
    return csr_from_pairs(f"chunglu_n{n}", u, v, n, scale_mode)


def rmat_pairs(scale: int, num_pairs: int, abcd=(0.57, 0.19, 0.19, 0.05), seed: int = 0,
               device="cpu") -> tuple:
    """R-MAT endpoints: one hashed 32-bit draw per (pair, level) picks the quadrant."""
    a, b, c, _ = abcd
    t_a = int(round(a * 2 ** 32))
    t_ab = int(round((a + b) * 2 ** 32))
    t_abc = int(round((a + b + c) * 2 ** 32))
    src = torch.empty(num_pairs, dtype=torch.int64, device=device)
    dst = torch.empty(num_pairs, dtype=torch.int64, device=device)
    chunk = 1 << 23
    for lo in range(0, num_pairs, chunk):
        hi = min(num_pairs, lo + chunk)
        idx = torch.arange(lo, hi, dtype=torch.int64, device=device)
        s = torch.zeros(hi - lo, dtype=torch.int64, device=device)
        d = torch.zeros(hi - lo, dtype=torch.int64, device=device)
        for level in range(scale):
            r = uniform32(seed, idx, 16 + level)
            row_bit = (r >= t_ab).to(torch.int64)                       # quadrants c, d
            col_bit = (((r >= t_a) & (r < t_ab)) | (r >= t_abc)).to(torch.int64)  # quadrants b, d
            s = (s << 1) | row_bit
            d = (d << 1) | col_bit
        src[lo:hi] = s
        dst[lo:hi] = d
    return src, dst


def rmat_graph(scale: int, pairs_per_vertex: int, abcd=(0.57, 0.19, 0.19, 0.05), seed: int = 0,
               device="cpu", scale_mode: str = "inv_sqrt") -> Graph:
    """Configs 3-5: R-MAT with 2^scale vertices and pairs_per_vertex * 2^scale generated pairs."""
    n = 1 << scale
    src, dst = rmat_pairs(scale, pairs_per_vertex * n, abcd, seed, device)
    return csr_from_pairs(f"rmat_s{scale}_ef{pairs_per_vertex}", src, dst, n, scale_mode)


def bernoulli_mask(num_nodes: int, ratio: float, seed: int = 2, device="cpu") -> torch.Tensor:
    """Train mask: independent Bernoulli(ratio) per vertex (bool [N])."""
    idx = torch.arange(num_nodes, dtype=torch.int64, device=device)
    return uniform01(seed, idx, 7) < ratio


def uniform_weights(seed: int, fan_in: int, fan_out: int, device="cpu") -> torch.Tensor:
    """U(-1/sqrt(out), 1/sqrt(out)) weights, the reference layer's init (EPPGCN/gcn_conv.py:47-49)."""
    idx = torch.arange(fan_in * fan_out, dtype=torch.int64, device=device)
    stdv = 1.0 / math.sqrt(fan_out)
    u = uniform01(seed, idx, 9)
    return ((2.0 * u - 1.0) * stdv).to(torch.float32).reshape(fan_in, fan_out)


def uniform_labels(seed: int, num_nodes: int, num_classes: int, device="cpu") -> torch.Tensor:
    idx = torch.arange(num_nodes, dtype=torch.int64, device=device)
    return (uniform32(seed, idx, 11) % num_classes).to(torch.int64)


# name -> constructor of the five benchmark configurations (seeds: graph 0).
CONFIGS = {
    "cfg1_uniform": lambda device="cpu", scale_mode="inv_sqrt": uniform_graph(
        2708, 5278, 0, device, scale_mode),
    "cfg2_chunglu": lambda device="cpu", scale_mode="inv_sqrt": chung_lu_graph(
        19717, 44325, 2.1, 0, device, scale_mode),
    "cfg3_rmat20": lambda device="cpu", scale_mode="inv_sqrt": rmat_graph(
        20, 4, seed=0, device=device, scale_mode=scale_mode),
    "cfg4_rmat22": lambda device="cpu", scale_mode="inv_sqrt": rmat_graph(
        22, 16, seed=0, device=device, scale_mode=scale_mode),
}


def make_graph(name: str, device="cpu", scale_mode: str = "inv_sqrt") -> Graph:
    """A named benchmark configuration, or ``rmat:<scale>:<pairs per vertex>`` for an R-MAT graph
    of another size (same generator and seed as the named ones), e.g. ``rmat:24:16``."""
    if name.startswith("rmat:"):
        _, scale, factor = name.split(":")
        return rmat_graph(int(scale), int(factor), seed=0, device=device, scale_mode=scale_mode)
    return CONFIGS[name](device=device, scale_mode=scale_mode)
