"""Pins the integer half of the CPU checker (build_part, mask marking, compaction, split,
group-size heuristics).  The reference has no tests or golden vectors for these, so each
function is pinned three ways: hand-computed known answers, the C restatement against an
independently written numpy closed form, and structural invariants."""
import numpy as np
import pytest

from oracle import c_oracle as co
from oracle import closed_forms as cf
from tests.helpers import hub_csr, random_symmetric_csr


# ----------------------------------------------------------------------------- build_part
def test_build_part_hand_case():
    # rows of degree 3, 0, 5 with group size 2 -> groups [0,2) [2,3) | - | [3,5) [5,7) [7,8)
    indptr = np.array([0, 3, 3, 8], np.int32)
    pp, p2n = co.build_part(2, indptr)
    assert pp.tolist() == [0, 2, 3, 5, 7, 8]
    assert p2n.tolist() == [0, 0, 2, 2, 2]
    pp2, p2n2 = cf.build_part(2, indptr)
    assert pp2.tolist() == pp.tolist() and p2n2.tolist() == p2n.tolist()


def test_build_part_exact_multiple_and_last_row_empty():
    # degree exactly a multiple of the group size; last row empty: terminator still written
    indptr = np.array([0, 4, 8, 8], np.int32)
    pp, p2n = co.build_part(4, indptr)
    assert pp.tolist() == [0, 4, 8] and p2n.tolist() == [0, 1]


@pytest.mark.parametrize("ps", [1, 2, 3, 5, 8, 32, 1000])
def test_build_part_c_vs_closed_form_and_invariants(tiny_graphs, ps):
    graphs = list(tiny_graphs) + [hub_csr(500, 300, 7), random_symmetric_csr(300, 900, 11, isolated=0.3)]
    for indptr, col in graphs:
        pp, p2n = co.build_part(ps, indptr)
        pp2, p2n2 = cf.build_part(ps, indptr)
        assert np.array_equal(pp, pp2) and np.array_equal(p2n, p2n2)
        sizes = np.diff(pp)
        if sizes.size:
            assert sizes.min() >= 1 and sizes.max() <= ps
        assert sizes.sum() == col.size
        # a group never crosses a row boundary
        assert np.all(pp[:-1] >= indptr[p2n]) and np.all(pp[1:] <= indptr[p2n + 1])
        assert np.all(np.diff(p2n) >= 0)


# ----------------------------------------------------------------------------- mask_forward
def _mask_c(indptr, col, ps, src, ngh, bem, degs, is_last):
    pp, p2n = co.build_part(ps, indptr)
    ngh = None if ngh is None else ngh.copy()
    bem, degs = bem.copy(), degs.copy()
    co.mask_forward(p2n, pp, col, src, ngh, bem, degs, is_last)
    return ngh, bem, degs


def test_mask_forward_hand_case():
    # path graph 0-1-2 with self-loops; src = {2}
    indptr = np.array([0, 2, 5, 7], np.int32)
    col = np.array([0, 1, 0, 1, 2, 1, 2], np.int32)
    src = np.array([0, 0, 1], bool)
    ngh, bem, degs = _mask_c(indptr, col, 2, src, np.zeros(3, bool), np.full(7, -1, np.int32),
                             np.zeros(3, np.int32), False)
    # kept slots are those whose COLUMN is vertex 2: slot 4 (row 1) and slot 6 (row 2)
    assert bem.tolist() == [-1, -1, -1, -1, 1, -1, 2]
    assert degs.tolist() == [0, 1, 1]
    # rows in src (row 2) mark themselves and all their neighbours {1, 2}
    assert ngh.tolist() == [False, True, True]
    # last layer: neighbour mask untouched (an empty tensor is passed by the caller)
    _, bem2, degs2 = _mask_c(indptr, col, 2, src, None, np.full(7, -1, np.int32), np.zeros(3, np.int32), True)
    assert bem2.tolist() == bem.tolist() and degs2.tolist() == degs.tolist()


@pytest.mark.parametrize("ratio", [0.0, 0.1, 0.5, 1.0])
def test_mask_forward_c_vs_closed_form(tiny_graphs, ratio):
    rng = np.random.default_rng(3)
    graphs = list(tiny_graphs) + [hub_csr(400, 250, 5), random_symmetric_csr(300, 700, 12, isolated=0.2)]
    for indptr, col in graphs:
        n, e = indptr.size - 1, col.size
        src = rng.random(n) < ratio
        pre_ngh = rng.random(n) < 0.05            # OR-into-existing semantics
        pre_degs = rng.integers(0, 3, n).astype(np.int32)   # += semantics
        for is_last in (False, True):
            want = cf.mask_forward(indptr, col, src, pre_ngh, np.full(e, -1, np.int32), pre_degs, is_last)
            for ps in (1, 3, 64):                 # result must not depend on the forward partition
                got = _mask_c(indptr, col, ps, src, pre_ngh, np.full(e, -1, np.int32), pre_degs, is_last)
                assert np.array_equal(got[0], want[0])
                assert np.array_equal(got[1], want[1])
                assert np.array_equal(got[2], want[2])


def test_mask_chain_two_layers_is_one_hop_closure():
    """Wiring of EPPGCN/gcn_main.py:130-139 for 2 layers: the last layer keeps edges whose column
    is a train vertex; the first layer keeps edges whose column is in train U N(train)."""
    indptr, col = random_symmetric_csr(200, 500, 21)
    n, e = 200, col.size
    rng = np.random.default_rng(0)
    train = rng.random(n) < 0.1
    row = cf.row_index(indptr)
    ngh0, bem_last, _ = cf.mask_forward(indptr, col, train, np.zeros(n, bool), np.full(e, -1, np.int32),
                                        np.zeros(n, np.int32), False)
    closure = train.copy()
    closure[col[train[row]]] = True
    assert np.array_equal(ngh0, closure)
    _, bem_first, _ = cf.mask_forward(indptr, col, ngh0, None, np.full(e, -1, np.int32),
                                      np.zeros(n, np.int32), True)
    assert np.array_equal(bem_last != -1, train[col])
    assert np.array_equal(bem_first != -1, closure[col])


# ----------------------------------------------------------------------------- compaction
def test_compact_mask_hand_case():
    em = np.array([-1, 4, -1, -1, 0, 7, -1], np.int32)
    col = np.array([10, 11, 12, 13, 14, 15, 16], np.int32)
    oid, oedge, v = co.compact_mask(em, col)
    assert v == 3
    assert oid.tolist() == [4, 0, 7, 0, 0, 0, 0]
    assert oedge.tolist() == [11, 14, 15, 0, 0, 0, 0]


@pytest.mark.parametrize("length", [0, 1, 63, 64, 65, 1023, 1024, 1025, 5000])
@pytest.mark.parametrize("density", [0.0, 0.1, 0.9, 1.0])
def test_compact_mask_c_vs_closed_form(length, density):
    rng = np.random.default_rng(length * 7 + int(density * 10))
    em = np.where(rng.random(length) < density, rng.integers(0, 1000, length), -1).astype(np.int32)
    col = rng.integers(0, 1000, length).astype(np.int32)
    a = co.compact_mask(em, col)
    b = cf.compact_mask(em, col)
    assert a[2] == b[2] == int((em != -1).sum())
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_compacted_path_invariants():
    indptr, col = hub_csr(600, 400, 9)
    n, e = 600, col.size
    src = np.random.default_rng(1).random(n) < 0.3
    oid, oedge, pp, v, p, degs = cf.pruned_path(indptr, col, src, 8)
    assert np.all(np.diff(oid[:v]) >= 0)                       # stability: rows ascending
    assert np.array_equal(np.bincount(oid[:v], minlength=n), degs)
    assert np.all(src[oedge[:v]])                              # only masked columns survive
    assert v == int(src[col].sum())
    assert co.compact_count(degs) == cf.compact_count(degs) == len(np.unique(oid[:v]))


# ----------------------------------------------------------------------------- split + scan
def test_split_hand_case():
    # kept degrees 0,5,0,2,4 with group size 2 -> counts 2,2,1 | 2 | 2,2 -> pointers 0,2,4,5,7,9,11
    degs = np.array([0, 5, 0, 2, 4], np.int32)
    pp, p = co.split_back_part(degs, 20, 2)
    assert p == 6
    assert pp[:7].tolist() == [0, 2, 4, 5, 7, 9, 11]
    assert not pp[7:].any()
    pp2, p2 = cf.split_back_part(degs, 20, 2)
    assert p2 == p and np.array_equal(pp, pp2)


@pytest.mark.parametrize("ps", [1, 2, 7, 8, 16, 32, 64])
def test_split_c_vs_closed_form_and_invariants(ps):
    rng = np.random.default_rng(ps)
    for n in (1, 5, 64, 1000, 4097):
        degs = (rng.integers(0, 40, n) * (rng.random(n) < 0.6)).astype(np.int32)
        e = int(degs.sum()) + 10
        a, pa = co.split_back_part(degs, e, ps)
        b, pb = cf.split_back_part(degs, e, ps)
        assert pa == pb and np.array_equal(a, b)
        assert a[pa] == degs.sum()                              # terminator = number of kept edges
        sizes = np.diff(a[: pa + 1])
        if sizes.size:
            assert sizes.min() >= 1 and sizes.max() <= ps
        # every group lies inside one vertex's run of the compacted id list
        ids = np.repeat(np.arange(n), degs)
        if pa:
            assert np.array_equal(ids[a[:pa]], ids[a[1: pa + 1] - 1])


def test_split_more_than_1023_groups_per_vertex():
    # the reference's bit-sliced counters stop at 1023 groups per vertex; the checker does not
    degs = np.array([3, 5000, 0, 2], np.int32)
    a, pa = co.split_back_part(degs, 6000, 2)
    b, pb = cf.split_back_part(degs, 6000, 2)
    assert pa == pb == 2 + 2500 + 1 and np.array_equal(a, b)
    assert a[pa] == 5005


# ----------------------------------------------------------------------------- heuristics
def test_group_size_regression_known_answers():
    # 0.65538 + 1.67431e-5*1000 - 2.24342e-6*5000 + 0.63641*5 = 3.8429559 -> 4
    assert co.map_back_part_size(1000, 5000) == cf.map_back_part_size(1000, 5000) == 4
    # 0.65538 + 1.67431 - 2.24342 + 0.63641*10 = 6.45037 -> 6
    assert co.map_back_part_size(100000, 1000000) == cf.map_back_part_size(100000, 1000000) == 6
    # large sparse path: negative result is returned as is (the caller must clamp)
    assert co.map_back_part_size(1000000, 100000000) == cf.map_back_part_size(1000000, 100000000)
    assert co.map_back_part_size(1000000, 100000000) == round(0.65538 + 16.7431 - 224.342 + 63.641)
    rng = np.random.default_rng(0)
    for _ in range(200):
        vn = int(rng.integers(1, 10 ** 6))
        vl = int(vn * rng.uniform(1, 60))
        assert co.map_back_part_size(vn, vl) == cf.map_back_part_size(vn, vl)


def test_c_round_is_half_away_from_zero():
    assert cf.c_round(2.5) == 3 and cf.c_round(3.5) == 4 and cf.c_round(-2.5) == -3
    assert round(2.5) == 2  # Python's own round would be wrong here


def test_group_size_thresholds_known_answers():
    for vn, vl, want in [(10, 39, 4), (10, 40, 8), (10, 159, 8), (10, 160, 16), (10, 639, 16),
                         (10, 640, 32), (10, 2559, 32), (10, 2560, 64), (10, 5119, 64), (10, 5120, 0)]:
        assert co.threshold_back_part_size(vn, vl) == cf.threshold_back_part_size(vn, vl) == want


def test_ginfo_known_answer_and_closed_form():
    degs = np.array([0, 1, 4, 5, 9, 10, 19, 20, 39, 40, 79, 80, 159, 160, 1000], np.int32)
    re = co.get_ginfo(degs, 777)
    want = np.array([14 / 1e4, 777 / 1e4, 777 / 14, 2 / 14, 2 / 14, 2 / 14, 2 / 14, 2 / 14, 2 / 14, 3 / 14],
                    np.float32)
    assert np.allclose(re, want, rtol=1e-6)
    assert np.allclose(cf.get_ginfo(degs, 777), re, rtol=1e-6)
