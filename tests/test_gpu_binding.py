"""GPU tests of the `GNNAdvisor` extension module and the autograd layer on top of it: the
twelve reference exports with their positional signatures, error behaviour (raise, never abort),
gradients against a dense float64 model, and the end-to-end loss trajectory against the host-CPU
sparse trainer."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import closed_forms as cf
from tests.helpers import hub_csr, random_symmetric_csr, scale_inv_sqrt

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def GNNA():
    import eppgcn_amd
    mod = eppgcn_amd.gnnadvisor()
    import GNNAdvisor            # the reference's import line works after gnnadvisor()
    assert GNNAdvisor is mod
    return mod


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_exports_match_the_reference_surface(GNNA):
    for name in ["forward", "backward", "mask_forward", "ours_backward", "print_time", "clear_time", "build_part",
                 "build_back_part", "compact_back_edge", "get_map_back_part_size", "split_back_part", "get_ginfo"]:
        assert callable(getattr(GNNA, name))


def test_build_part_accepts_cpu_indptr_and_returns_int32(GNNA):
    indptr, col = hub_csr(3000, 2000, 1)
    for ps in (1, 7, 32):
        want_pp, want_p2n = co.build_part(ps, indptr)
        for t in (torch.from_numpy(indptr), dev(indptr)):
            pp, p2n = GNNA.build_part(ps, t)
            # the reference's caller then does .int().to(device): both must be no-ops
            pp, p2n = pp.int().to("cuda"), p2n.int().to("cuda")
            assert pp.dtype == torch.int32 and np.array_equal(pp.cpu().numpy(), want_pp)
            assert np.array_equal(p2n.cpu().numpy(), want_p2n)


def test_forward_and_both_backwards_with_dense_products(GNNA):
    indptr, col = hub_csr(2000, 1500, 2)
    n = indptr.size - 1
    rng = np.random.default_rng(0)
    s = scale_inv_sqrt(indptr)
    x = rng.standard_normal((n, 96)).astype(np.float32)
    w = rng.uniform(-0.25, 0.25, (96, 16)).astype(np.float32)
    pp, p2n = co.build_part(6, indptr)
    args = (dev(indptr), dev(col), dev(s), dev(pp), dev(p2n), 6, 16, 8)
    y = GNNA.forward(dev(x), dev(w), *args)[0].cpu().numpy()
    t64 = x.astype(np.float64) @ w.astype(np.float64)
    want = cf.aggregate_csr64(indptr, col, s, t64)
    assert np.linalg.norm(y - want) / np.linalg.norm(want) < 1e-5

    src = rng.random(n) < 0.2
    dy = (rng.standard_normal((n, 16)) * src[:, None]).astype(np.float32)
    g64 = cf.aggregate_csr64(indptr, col, s, dy)
    want_dx, want_dw = g64 @ w.T.astype(np.float64), x.T.astype(np.float64) @ g64
    dx, dw = GNNA.backward(dev(dy), dev(x), dev(w), *args)
    assert np.linalg.norm(dx.cpu().numpy() - want_dx) / np.linalg.norm(want_dx) < 1e-5
    assert np.linalg.norm(dw.cpu().numpy() - want_dw) / np.linalg.norm(want_dw) < 1e-5

    # pruned path through the module's own preparation functions
    e = col.size
    bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
    degs = torch.zeros(n, dtype=torch.int32, device="cuda")
    GNNA.mask_forward(dev(p2n), dev(pp), dev(col), dev(src), torch.zeros(0, dtype=torch.bool, device="cuda"),
                      bem, degs, 2, 2, 4, 16)
    ids, edge_list, info = GNNA.compact_back_edge(bem, dev(col))
    v = int(info[0].item())
    assert v == int(src[col].sum()) and not info.is_cuda
    ps = GNNA.get_map_back_part_size(degs, v)
    assert ps == max(1, cf.map_back_part_size(cf.compact_count(degs.cpu().numpy()), v))
    part_pointer, pinfo = GNNA.split_back_part(degs, e, ps)
    want_pp, want_p = cf.split_back_part(degs.cpu().numpy(), e, ps)
    assert int(pinfo[0].item()) == want_p and pinfo.dtype == torch.int32 and not pinfo.is_cuda
    assert np.array_equal(part_pointer.cpu().numpy(), want_pp)
    dx2, dw2 = GNNA.ours_backward(dev(dy), dev(x), dev(w), ids, part_pointer, edge_list, dev(s), ps, want_p, 1, 4, 16)
    assert np.linalg.norm(dx2.cpu().numpy() - want_dx) / np.linalg.norm(want_dx) < 1e-5
    assert np.linalg.norm(dw2.cpu().numpy() - want_dw) / np.linalg.norm(want_dw) < 1e-5

    # the module remembers per path which rows it gathers (a fifth of them here) and pre-scales only
    # those: a second gradient through the same path, and garbage in the rows the path never reads
    dy_b = (rng.standard_normal((n, 16)) * src[:, None]).astype(np.float32)
    g64_b = cf.aggregate_csr64(indptr, col, s, dy_b)
    noisy = dy_b.copy()
    never_read = np.ones(n, bool)
    never_read[col[src[col]]] = False
    noisy[never_read] = 1e30
    dx3, dw3 = GNNA.ours_backward(dev(noisy), dev(x), dev(w), ids, part_pointer, edge_list, dev(s), ps, want_p, 1, 4, 16)
    assert np.linalg.norm(dx3.cpu().numpy() - g64_b @ w.T.astype(np.float64)) / np.linalg.norm(g64_b @ w.T) < 1e-5
    assert np.linalg.norm(dw3.cpu().numpy() - x.T.astype(np.float64) @ g64_b) / np.linalg.norm(x.T @ g64_b) < 1e-5
    # a path rewritten in place (same storage) is a different path: nothing remembered may be reused
    src_c = rng.random(n) < 0.25
    bem.fill_(-1); degs.zero_()
    GNNA.mask_forward(dev(p2n), dev(pp), dev(col), dev(src_c), torch.zeros(0, dtype=torch.bool, device="cuda"),
                      bem, degs, 2, 2, 4, 16)
    ids_c, edge_c, info_c = GNNA.compact_back_edge(bem, dev(col))
    pp_c, pinfo_c = GNNA.split_back_part(degs, e, ps)
    ids.copy_(ids_c); edge_list.copy_(edge_c); part_pointer.copy_(pp_c)
    dy_c = (rng.standard_normal((n, 16)) * src_c[:, None]).astype(np.float32)
    g64_c = cf.aggregate_csr64(indptr, col, s, dy_c)
    dx4, dw4 = GNNA.ours_backward(dev(dy_c), dev(x), dev(w), ids, part_pointer, edge_list, dev(s), ps,
                                  int(pinfo_c[0].item()), 1, 4, 16)
    assert np.linalg.norm(dx4.cpu().numpy() - g64_c @ w.T.astype(np.float64)) / np.linalg.norm(g64_c @ w.T) < 1e-5
    bem.fill_(-1); degs.zero_()
    GNNA.mask_forward(dev(p2n), dev(pp), dev(col), dev(src), torch.zeros(0, dtype=torch.bool, device="cuda"),
                      bem, degs, 2, 2, 4, 16)
    ids, edge_list, info = GNNA.compact_back_edge(bem, dev(col))

    # legacy all-in-one call: same lists, threshold group size
    ids3, el3, pp3, info3 = GNNA.build_back_part(bem, dev(col), degs, 0, 16)
    ps3 = cf.threshold_back_part_size(cf.compact_count(degs.cpu().numpy()), v)
    assert int(info3[0].item()) == ps3
    want_pp3, want_p3 = cf.split_back_part(degs.cpu().numpy(), e, ps3)
    assert int(info3[1].item()) == want_p3 and np.array_equal(pp3.cpu().numpy(), want_pp3)
    assert torch.equal(ids3, ids) and torch.equal(el3, edge_list)
    assert np.allclose(GNNA.get_ginfo(degs, v).numpy(), cf.get_ginfo(degs.cpu().numpy(), v), rtol=1e-6)


def test_argument_errors_raise_runtime_error(GNNA):
    x = torch.randn(8, 4, device="cuda")
    w = torch.randn(4, 3, device="cuda")
    i = torch.zeros(9, dtype=torch.int32, device="cuda")
    s = torch.ones(8, device="cuda")
    with pytest.raises(RuntimeError):
        GNNA.forward(x.cpu(), w, i, i, s, i, i[:8], 1, 1, 1)                  # not on the GPU
    with pytest.raises(RuntimeError):
        GNNA.forward(x.t(), w, i, i, s, i, i[:8], 1, 1, 1)                   # not contiguous / wrong shape
    with pytest.raises(RuntimeError):
        GNNA.forward(x, w, i.long(), i, s, i, i[:8], 1, 1, 1)                # wrong index dtype
    with pytest.raises(RuntimeError):
        GNNA.forward(x, w, i, i, s, i[:3], i[:8], 1, 1, 1)                   # part pointers too short
    with pytest.raises(RuntimeError):
        GNNA.split_back_part(i, 10, 0)                                       # group size 0
    with pytest.raises(RuntimeError):
        GNNA.compact_back_edge(i.float(), i)                                 # wrong dtype
    assert torch.isfinite(x).all()                                           # the process is still alive


def _dense_model_grads(indptr, col, s, x, w0, w1, train, y):
    """float64 autograd of the same 2-layer model with a dense normalised adjacency."""
    n = indptr.size - 1
    a = torch.zeros(n, n, dtype=torch.float64)
    a[torch.from_numpy(cf.row_index(indptr)), torch.from_numpy(col.astype(np.int64))] = 1.0
    w32 = (torch.from_numpy(s)[:, None] * torch.from_numpy(s)[None, :]).double()
    a = a * w32
    w0 = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    w1 = torch.tensor(w1, dtype=torch.float64, requires_grad=True)
    h = torch.relu(a @ (torch.from_numpy(x).double() @ w0))
    out = a @ (h @ w1)
    loss = torch.nn.functional.nll_loss(torch.log_softmax(out, 1)[torch.from_numpy(train)], torch.from_numpy(y)[torch.from_numpy(train)])
    loss.backward()
    return float(loss), w0.grad.numpy(), w1.grad.numpy()


@pytest.mark.parametrize("policy", [0, 1, -1])
def test_autograd_layer_gradients_vs_dense_float64(GNNA, policy):
    """policy 1 forces column-blocked execution plans (normally reserved for large graphs), so that
    the module's plan cache and the planned kernels are exercised through autograd as well."""
    from eppgcn_amd import graphs, train
    GNNA.set_plan_policy(policy)
    indptr, col = random_symmetric_csr(400, 1500, 3)
    n = indptr.size - 1
    g = graphs.Graph("t", n, dev(indptr), dev(col), dev(scale_inv_sqrt(indptr)))
    rng = np.random.default_rng(1)
    mask = rng.random(n) < 0.15
    tr = train.Trainer(g, dim=24, hidden=16, num_classes=22, train_mask=torch.from_numpy(mask), backsize=4,
                       labels="uniform")
    x = tr.dataset.x.cpu().numpy()
    y = tr.dataset.y.cpu().numpy()
    w0 = tr.model.convs[0].weights.detach().cpu().numpy()
    w1 = tr.model.convs[1].weights.detach().cpu().numpy()
    want_loss, want_g0, want_g1 = _dense_model_grads(indptr, col, scale_inv_sqrt(indptr), x, w0, w1, mask, y)
    tr.optimizer = torch.optim.SGD(tr.model.parameters(), lr=0.0)      # keep the weights fixed
    loss = tr.train_step(True)
    assert abs(float(loss) - want_loss) < 1e-5 * max(1.0, abs(want_loss))
    g0 = tr.model.convs[0].weights.grad.cpu().numpy()
    g1 = tr.model.convs[1].weights.grad.cpu().numpy()
    assert np.linalg.norm(g0 - want_g0) / np.linalg.norm(want_g0) < 1e-4
    assert np.linalg.norm(g1 - want_g1) / np.linalg.norm(want_g1) < 1e-4
    # later iterations reuse the prepared path and give the same gradients
    tr.train_step(False)
    assert np.allclose(tr.model.convs[0].weights.grad.cpu().numpy(), g0, rtol=1e-4, atol=1e-7)
    assert (GNNA.cached_plans() > 0) == (policy == 1)
    GNNA.set_plan_policy(0)


@pytest.mark.parametrize("cfg", ["cfg1_uniform", "cfg2_chunglu"])
def test_loss_trajectory_matches_cpu_sparse_trainer(GNNA, cfg):
    """Same seeds -> the GPU path and the CPU-sparse baseline follow the same loss curve."""
    import torch.nn.functional as F
    from eppgcn_amd import graphs, train
    g_cpu = graphs.make_graph(cfg)
    g = g_cpu.to("cuda")
    mask = graphs.bernoulli_mask(g.num_nodes, 0.1)
    tr = train.Trainer(g, train_mask=mask, backsize_mode="map", labels="uniform")
    gpu_losses = [float(tr.train_step(i == 0)) for i in range(100)]

    n = g_cpu.num_nodes
    row = g_cpu.row_index()
    a = torch.sparse_csr_tensor(g_cpu.row_pointers.long(), g_cpu.column_index.long(),
                                (g_cpu.degrees[row] * g_cpu.degrees[g_cpu.column_index.long()]).double(), size=(n, n))
    x = graphs.normal32(1, (n, 96)).double()
    y = graphs.uniform_labels(4, n, 22)
    w0 = graphs.uniform_weights(3, 96, 16).double().requires_grad_()
    w1 = graphs.uniform_weights(4, 16, 22).double().requires_grad_()
    opt = torch.optim.Adam([w0, w1], lr=0.01)
    cpu_losses = []
    for _ in range(100):
        opt.zero_grad()
        out = torch.sparse.mm(a, torch.relu(torch.sparse.mm(a, x @ w0)) @ w1)
        loss = F.nll_loss(F.log_softmax(out, 1)[mask], y[mask])
        loss.backward()
        opt.step()
        cpu_losses.append(float(loss))
    gpu_losses, cpu_losses = np.array(gpu_losses), np.array(cpu_losses)
    assert cpu_losses[-1] < cpu_losses[0]
    assert np.max(np.abs(gpu_losses - cpu_losses) / np.abs(cpu_losses)) < 2e-3


def test_print_time_lines(GNNA, capfd):
    from eppgcn_amd import graphs, train
    g = graphs.make_graph("cfg1_uniform", device="cuda")
    tr = train.Trainer(g)
    res = tr.run(epochs=3, warmup=2, kernel_timing=True)
    assert res["for_agg_time"] > 0 and res["back_agg_time"] > 0
    GNNA.set_timing(True)
    tr.train_step(False)
    GNNA.set_timing(False)
    tr.model.convs[0].print_time()
    out = capfd.readouterr().out
    for key in ("for_agg_time:", "back_agg_time:", "l1_back_agg_time:", "l2_back_agg_time:", "mask_time:"):
        assert key in out


@pytest.mark.parametrize("fuse_relu", [True, False])
@pytest.mark.parametrize("dense", [0, -1])
def test_gradients_with_fused_relu_and_with_torch_products(GNNA, fuse_relu, dense):
    """The activation applied inside the consuming layer's product, and the library's own dense
    products versus torch::mm (dense = -1), all give the float64 dense model's gradients."""
    from eppgcn_amd import graphs, train
    GNNA.set_dense_policy(dense)
    try:
        indptr, col = random_symmetric_csr(700, 2500, 8)
        n = indptr.size - 1
        g = graphs.Graph("t", n, dev(indptr), dev(col), dev(scale_inv_sqrt(indptr)))
        mask = np.random.default_rng(2).random(n) < 0.2
        tr = train.Trainer(g, dim=24, hidden=16, num_classes=22, train_mask=torch.from_numpy(mask), backsize=4,
                           labels="uniform", fuse_relu=fuse_relu)
        x, y = tr.dataset.x.cpu().numpy(), tr.dataset.y.cpu().numpy()
        w0 = tr.model.convs[0].weights.detach().cpu().numpy()
        w1 = tr.model.convs[1].weights.detach().cpu().numpy()
        want_loss, want_g0, want_g1 = _dense_model_grads(indptr, col, scale_inv_sqrt(indptr), x, w0, w1, mask, y)
        tr.optimizer = torch.optim.SGD(tr.model.parameters(), lr=0.0)
        loss = tr.train_step(True)
        assert abs(float(loss) - want_loss) < 1e-5 * max(1.0, abs(want_loss))
        g0 = tr.model.convs[0].weights.grad.cpu().numpy()
        g1 = tr.model.convs[1].weights.grad.cpu().numpy()
        assert np.linalg.norm(g0 - want_g0) / np.linalg.norm(want_g0) < 1e-4
        assert np.linalg.norm(g1 - want_g1) / np.linalg.norm(want_g1) < 1e-4
    finally:
        GNNA.set_dense_policy(0)


def test_keyword_additions_of_the_layer_ops(GNNA):
    """relu_input and need_dx, the two keyword arguments this build adds to the reference's calls."""
    indptr, col = random_symmetric_csr(900, 4000, 17)
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((n, 16)).astype(np.float32)
    w = rng.uniform(-0.3, 0.3, (16, 22)).astype(np.float32)
    dy = rng.standard_normal((n, 22)).astype(np.float32)
    pp, p2n = GNNA.build_part(6, dev(indptr))
    args = (dev(indptr), dev(col), dev(s), pp.int(), p2n.int(), 6, 32, 8)
    plain = GNNA.forward(torch.relu(dev(x)), dev(w), *args)[0]
    fused = GNNA.forward(dev(x), dev(w), *args, relu_input=True)[0]
    assert torch.allclose(plain, fused, rtol=1e-5, atol=1e-6)
    dx, dw = GNNA.backward(dev(dy), torch.relu(dev(x)), dev(w), *args)
    dx_f, dw_f = GNNA.backward(dev(dy), dev(x), dev(w), *args, relu_input=True)
    assert torch.allclose(dw, dw_f, rtol=1e-4, atol=1e-4)
    assert torch.allclose(dx * (dev(x) > 0), dx_f, rtol=1e-5, atol=1e-6)
    none, dw_only = GNNA.backward(dev(dy), dev(x), dev(w), *args, need_dx=False, relu_input=True)
    assert none.numel() == 0 and torch.equal(dw_only, dw_f)


def test_training_from_a_dataset_file(GNNA, tmp_path):
    """Reference-format files -> loader -> the same Trainer; the first-iteration gradients equal
    the float64 dense model's on the loaded graph (scale = the loader's sqrt(deg) filling would
    blow up a 2-layer model, so the symmetric normalisation is asked for)."""
    from eppgcn_amd import dataset as dsmod, train
    indptr, col = random_symmetric_csr(300, 1200, 31)
    n = indptr.size - 1
    rows = np.repeat(np.arange(n), np.diff(indptr))
    np.savez(str(tmp_path / "g.npz"), src_li=rows, dst_li=col, num_nodes=n)
    mask = np.random.default_rng(9).random(n) < 0.25
    dsmod.write_train_mask(str(tmp_path), 0.25, mask)
    d = dsmod.custom_dataset(str(tmp_path / "g.npz"), str(tmp_path), 0.25, 12, 7, 2, load_from_txt=False,
                             scale_mode="inv_sqrt", feature_seed=5)
    assert np.array_equal(d.row_pointers.cpu().numpy(), indptr) and np.array_equal(d.column_index.cpu().numpy(), col)
    tr = train.Trainer(None, hidden=16, dataset=d, backsize=4)
    w0 = tr.model.convs[0].weights.detach().cpu().numpy()
    w1 = tr.model.convs[1].weights.detach().cpu().numpy()
    want_loss, want_g0, want_g1 = _dense_model_grads(indptr, col, scale_inv_sqrt(indptr), d.x.cpu().numpy(), w0, w1,
                                                     mask, d.y.cpu().numpy())
    tr.optimizer = torch.optim.SGD(tr.model.parameters(), lr=0.0)
    loss = tr.train_step(True)
    assert abs(float(loss) - want_loss) < 1e-5 * max(1.0, abs(want_loss))
    assert np.linalg.norm(tr.model.convs[0].weights.grad.cpu().numpy() - want_g0) / np.linalg.norm(want_g0) < 1e-4
    assert np.linalg.norm(tr.model.convs[1].weights.grad.cpu().numpy() - want_g1) / np.linalg.norm(want_g1) < 1e-4


def test_dataset_in_degree_order_trains_the_same_model(GNNA, tmp_path):
    """``custom_dataset(degree_order=True)``: the vertices are renumbered after loading (features, labels and mask
    move with them), so the loss and the weight gradients are those of the files' numbering up to rounding, and
    the output rows are the old ones at ``new_id``."""
    from eppgcn_amd import dataset as dsmod, train
    indptr, col = random_symmetric_csr(900, 4000, 33)
    n = indptr.size - 1
    rows = np.repeat(np.arange(n), np.diff(indptr))
    np.savez(str(tmp_path / "g.npz"), src_li=rows, dst_li=col, num_nodes=n)
    mask = np.random.default_rng(10).random(n) < 0.2
    dsmod.write_train_mask(str(tmp_path), 0.2, mask)
    runs = []
    for order in (False, True):
        d = dsmod.custom_dataset(str(tmp_path / "g.npz"), str(tmp_path), 0.2, 12, 7, 2, load_from_txt=False,
                                 scale_mode="inv_sqrt", feature_seed=5, degree_order=order)
        tr = train.Trainer(None, hidden=16, dataset=d, backsize=4, weight_seed=3)
        tr.optimizer = torch.optim.SGD(tr.model.parameters(), lr=0.0)
        loss = float(tr.train_step(True))
        out = tr.model(d.x, tr.inputInfo, tr.mask_props, tr.back_props, False, False).detach()
        runs.append((d, loss, [c.weights.grad.cpu().numpy().copy() for c in tr.model.convs], out))
        GNNA.clear_plans()
    (d0, l0, g0, o0), (d1, l1, g1, o1) = runs
    assert d0.new_id is None and sorted(d1.new_id.tolist()) == list(range(n))
    assert abs(l0 - l1) <= 1e-5 * max(1.0, abs(l0))
    for a, b in zip(g0, g1):
        assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(a) + 1e-12
    assert torch.allclose(o1[d1.new_id], o0, rtol=1e-4, atol=1e-5)


def test_driver_command_line_end_to_end(GNNA, tmp_path, capsys):
    """`python -m eppgcn_amd.gcn_main` with the reference's flags on reference-format files: the
    report carries the reference's lines (EPPGCN/gcn_main.py:286-291), --verify_spmm passes, a
    synthetic graph name works without files and a missing file is an error, not a crash."""
    from eppgcn_amd import dataset as dsmod, gcn_main
    indptr, col = random_symmetric_csr(400, 1500, 17)
    n = indptr.size - 1
    rows = np.repeat(np.arange(n), np.diff(indptr))
    np.savetxt(str(tmp_path / "toy_snap"), np.stack([rows, col], 1), fmt="%d")
    dsmod.write_train_mask(str(tmp_path), 0.3, np.random.default_rng(2).random(n) < 0.3)
    common = ["--dataset", "toy", "--dataDir", str(tmp_path), "--dim", "24", "--hidden", "16", "--classes", "5",
              "--train_ratio", "0.3", "--num_epoches", "3", "--degree_norm", "inv_sqrt"]
    for extra in (["--layers", "3", "--backsize_mode", "map"], ["--layers", "2", "--backsize_mode", "wave64"],
                  ["--layers", "2", "--backsize_mode", "constant", "--backsize", "8", "--kernel_timers", "False",
                   "--manual_mode", "True", "--partSize", "4", "--verbose_mode", "True"]):
        assert gcn_main.main(common + extra) == 0
        out = capsys.readouterr().out
        for key in ("for_time:", "loss_time:", "back_time:", "build_time:", "Time:"):
            assert sum(line.startswith(key) for line in out.splitlines()) == 1, (key, out)
        assert out.startswith("||toy   0.3   ")
    assert gcn_main.main(common + ["--hip_graph", "True"]) == 0
    out = capsys.readouterr().out
    assert "Time:" in out and "for_time" not in out
    assert gcn_main.main(common + ["--verify_spmm", "True"]) == 0
    assert "PASS" in capsys.readouterr().out
    assert gcn_main.main(["--dataset", "cfg1_uniform", "--num_epoches", "2", "--degree_norm", "inv_sqrt",
                          "--backsize_mode", "constant", "--backsize", "16"]) == 0
    capsys.readouterr()
    with pytest.raises(FileNotFoundError):
        gcn_main.main(["--dataset", "no_such_graph", "--dataDir", str(tmp_path)])


@pytest.mark.parametrize("num_layers", [3, 4, 5, 6])
def test_deeper_models_follow_the_mask_chain(GNNA, num_layers):
    """3 to 6 layers (the depths the reference sweeps, EPPGCN/bench_EPPGCN.py:36): the marking of
    layer i feeds layer i+1's source mask and edge_masks[L-1-i]; gradients of every weight equal the
    float64 dense model's."""
    from eppgcn_amd import graphs, train
    indptr, col = random_symmetric_csr(500, 1400, 41)
    n = indptr.size - 1
    s = scale_inv_sqrt(indptr)
    g = graphs.Graph("t", n, dev(indptr), dev(col), dev(s))
    mask = np.random.default_rng(4).random(n) < 0.1
    tr = train.Trainer(g, dim=20, hidden=16, num_classes=9, num_layers=num_layers, train_mask=torch.from_numpy(mask),
                       backsize=4, labels="uniform")
    ws = [c.weights.detach().cpu().numpy() for c in tr.model.convs]
    a = torch.zeros(n, n, dtype=torch.float64)
    a[torch.from_numpy(cf.row_index(indptr)), torch.from_numpy(col.astype(np.int64))] = 1.0
    a = a * (torch.from_numpy(s)[:, None] * torch.from_numpy(s)[None, :]).double()
    w64 = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in ws]
    h = tr.dataset.x.cpu().double()
    for i, w in enumerate(w64):
        h = a @ (h @ w)
        if i < num_layers - 1:
            h = torch.relu(h)
    tm = torch.from_numpy(mask)
    want = torch.nn.functional.nll_loss(torch.log_softmax(h, 1)[tm], tr.dataset.y.cpu()[tm])
    want.backward()
    tr.optimizer = torch.optim.SGD(tr.model.parameters(), lr=0.0)
    loss = tr.train_step(True)
    assert abs(float(loss) - float(want)) < 1e-5 * max(1.0, abs(float(want)))
    for c, w in zip(tr.model.convs, w64):
        got, ref = c.weights.grad.cpu().numpy(), w.grad.numpy()
        assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 1e-4
    # the kept path grows from the last layer (train rows only) towards the first
    kept = [b.numParts for b in tr.back_props]
    assert all(kept[i] >= kept[i + 1] for i in range(num_layers - 1))
    # and every layer's compacted path is the closed form of the chain (EPPGCN/gcn_main.py:130-139):
    # step i keeps the slots whose column is in its source mask; the next source mask is the rows of
    # the current one that have slots, plus their neighbours
    row = cf.row_index(indptr)
    src = mask.copy()
    for i in range(num_layers):
        prop = tr.back_props[num_layers - 1 - i]
        keep = src[col]
        v = int(keep.sum())
        assert int(prop.partPointer[prop.numParts]) == v
        assert np.array_equal(prop.id[:v].cpu().numpy(), row[keep]) and np.array_equal(prop.edgeList[:v].cpu().numpy(), col[keep])
        nxt = np.zeros(n, bool)
        sel = src[row]
        nxt[row[sel]] = True
        nxt[col[sel]] = True
        src = nxt


@pytest.mark.parametrize("num_layers", [2, 4])
def test_unpruned_ablation_gives_the_gradients_of_the_pruned_path(GNNA, num_layers):
    """``Trainer(prune=False)`` (the driver's ``--prune False``): every layer's backward runs the module's unpruned
    ``backward`` over the forward groups.  The incoming gradient is zero outside the prepared path, so the weight
    gradients agree with the pruned run to rounding."""
    from eppgcn_amd import graphs, train
    indptr, col = random_symmetric_csr(700, 2100, 43)
    n = indptr.size - 1
    g = graphs.Graph("t", n, dev(indptr), dev(col), dev(scale_inv_sqrt(indptr)))
    mask = torch.from_numpy(np.random.default_rng(6).random(n) < 0.15)
    grads = []
    for prune in (True, False):
        tr = train.Trainer(g, dim=20, hidden=16, num_classes=9, num_layers=num_layers, train_mask=mask, backsize=4,
                           labels="uniform", prune=prune)
        tr.optimizer = torch.optim.SGD(tr.model.parameters(), lr=0.0)
        tr.train_step(True)
        tr.train_step(False)
        grads.append([c.weights.grad.cpu().numpy().copy() for c in tr.model.convs])
        res = tr.run(2, warmup=0, kernel_timing=True)
        assert res["pruned"] == prune and len(res["layer_back_agg_time"]) == num_layers
        assert all(k is not None and k > 0 for k in res["kept_edges"])
        assert (min(res["layer_back_agg_time"]) > 0) == prune       # the unpruned entry point has no per-layer timers
        GNNA.clear_plans()
    for a, b in zip(*grads):
        assert np.linalg.norm(a - b) <= 1e-5 * np.linalg.norm(a) + 1e-12


@pytest.mark.parametrize("num_layers", [2, 3])
def test_row_masked_dense_products_give_the_same_gradients(GNNA, num_layers):
    """With execution plans the pruned backward leaves the rows outside the path uncleared and its two dense products
    read only the rows the aggregation wrote (``set_masked_update``, on by default; the reference sketches the masked
    weight gradient at EPPGCN_kernel.cu:607,616).  The weight gradients of every layer are the bits of the run that
    clears and reads every row."""
    from eppgcn_amd import graphs, train
    indptr, col = random_symmetric_csr(3000, 9000, 47)
    n = indptr.size - 1
    g = graphs.Graph("t", n, dev(indptr), dev(col), dev(scale_inv_sqrt(indptr)))
    mask = torch.from_numpy(np.random.default_rng(7).random(n) < 0.1)
    grads = []
    GNNA.set_plan_policy(1)
    try:
        for masked in (True, False):
            GNNA.set_masked_update(masked)
            tr = train.Trainer(g, dim=20, hidden=16, num_classes=9, num_layers=num_layers, train_mask=mask, backsize=4,
                               labels="uniform")
            tr.optimizer = torch.optim.SGD(tr.model.parameters(), lr=0.0)
            tr.train_step(True)
            tr.train_step(False)
            grads.append([c.weights.grad.clone() for c in tr.model.convs])
            GNNA.clear_plans()
    finally:
        GNNA.set_masked_update(True)
        GNNA.set_plan_policy(0)
    assert all(a.abs().sum() > 0 for a in grads[0])
    for a, b in zip(*grads):
        assert torch.equal(a, b)


def test_group_size_rules_on_device_degrees(GNNA):
    """get_wave64_back_part_size / get_map_back_part_size on kept degrees that live on the device: the
    wave64 rule is 16 below 24 kept edges per kept row and 32 from there on; the fitted regression
    (EPPGCN/GCNConv/EPPGCN.cpp:303-310) is returned while it is at least 1 and replaced by the wave64
    rule where it goes negative (large paths), never by a clamp to 1."""
    from eppgcn_amd import capi, graphs, workload
    g = graphs.make_graph("cfg3_rmat20", device="cuda")
    wl = workload.prepare(g, 2, 0.1, 2, plan=False)
    for path in wl.paths:
        vn = int((path.node_degs != 0).sum())
        assert vn == path.valid_node
        want = 16 if path.valid_len // vn < 24 else 32
        assert GNNA.get_wave64_back_part_size(path.node_degs, path.valid_len) == want
        fitted = co.map_back_part_size(vn, path.valid_len)
        assert fitted >= 1, "the regression is positive at this size"
        assert GNNA.get_map_back_part_size(path.node_degs, path.valid_len) == fitted
        assert capi.auto_back_part_size(vn, path.valid_len) == (fitted, False)
    # a path the regression was never fitted for: 10^6 kept rows of 100 kept edges each -> -143
    degs = torch.full((1_000_000,), 100, dtype=torch.int32, device="cuda")
    assert co.map_back_part_size(1_000_000, 100_000_000) < 1
    assert capi.map_back_part_size(1_000_000, 100_000_000) == (1, True)
    assert GNNA.get_map_back_part_size(degs, 100_000_000) == 32      # (warns once per process)
    assert capi.auto_back_part_size(1_000_000, 100_000_000) == (32, True)
    degs[::2] = 0                                  # half of the rows keep nothing: 5 * 10^5 rows, 10 per row
    degs[1::2] = 10
    assert GNNA.get_wave64_back_part_size(degs, 5_000_000) == 16
    # get_ginfo takes the kept degrees from the host as well, as the reference's caller passes them
    assert torch.equal(GNNA.get_ginfo(degs.cpu(), 5_000_000), GNNA.get_ginfo(degs, 5_000_000))


def test_sweep_driver_runs_every_depth_in_one_process(GNNA, tmp_path, capsys):
    """The datasets x ratios x depths sweep (EPPGCN/bench_EPPGCN.py:17-61) over the driver: a dataset
    from files in the reference's layout and a synthetic one, depths 3-6, one report line each."""
    import json
    from eppgcn_amd import bench_eppgcn, dataset as ds_mod
    indptr, col = random_symmetric_csr(400, 1500, 77)
    folder = tmp_path / "toy"
    folder.mkdir()
    rows = cf.row_index(indptr)
    np.savetxt(folder / "toy_snap", np.stack([rows, col], 1), fmt="%d")
    ds_mod.write_train_mask(str(folder), 0.3, np.random.default_rng(1).random(400) < 0.3)
    rc = bench_eppgcn.main(["--dataRoot", str(tmp_path), "--datasets", "toy,12,5", "cfg1_uniform", "absent,8,3",
                            "--ratios", "0.3", "--layers", "3", "4", "5", "6", "--num_epoches", "3",
                            "--groupsize_model", "regression_equation"])
    assert rc == 0
    out = capsys.readouterr().out
    lines = [json.loads(l) for l in out.splitlines() if l.startswith("{")]
    assert len(lines) == 12
    ok = [l for l in lines if l["status"] == "ok"]
    assert [(l["dataset"], l["layers"]) for l in ok] == [(d, k) for d in ("toy", "cfg1_uniform") for k in (3, 4, 5, 6)]
    assert all(l["status"] == "skipped" for l in lines if l["dataset"] == "absent")
    for l in ok:
        assert l["Time"] > 0 and len(l["backward_group_sizes"]) == l["layers"] and min(l["backward_group_sizes"]) >= 1
    assert out.count("||toy   0.3   ") == 4 and out.count("Time: ") == 8
    assert bench_eppgcn.main(["--datasets", "cfg1_uniform", "--ratios", "0.1", "--layers", "3", "--num_epoches", "1",
                              "--groupsize_model", "SAGPG"]) == 1


def test_module_mark_compact_equals_the_two_reference_steps(GNNA):
    indptr, col = random_symmetric_csr(2000, 9000, 23)
    n, e = indptr.size - 1, col.size
    src = np.random.default_rng(6).random(n) < 0.2
    pp, p2n = GNNA.build_part(7, dev(indptr))
    pp, p2n = pp.int(), p2n.int()
    ngh_a = torch.zeros(n, dtype=torch.bool, device="cuda"); ngh_b = ngh_a.clone()
    degs_a = torch.zeros(n, dtype=torch.int32, device="cuda"); degs_b = degs_a.clone()
    bem = torch.full((e,), -1, dtype=torch.int32, device="cuda")
    GNNA.mask_forward(p2n, pp, dev(col), dev(src), ngh_a, bem, degs_a, 2, 1, 4, 16)
    id_a, el_a, info_a = GNNA.compact_back_edge(bem, dev(col))
    id_b, el_b, info_b = GNNA.mark_compact(p2n, pp, dev(col), dev(src), ngh_b, degs_b, 2, 1)
    assert torch.equal(id_a, id_b) and torch.equal(el_a, el_b) and float(info_a[0]) == float(info_b[0])
    assert torch.equal(ngh_a, ngh_b) and torch.equal(degs_a, degs_b)


def test_epoch_replayed_from_a_hip_graph_follows_the_eager_trajectory(GNNA):
    """One whole training epoch (layer ops, loss, backward, Adam) captured into a HIP graph: every
    replay, with eager work and synchronisations in between, gives the loss of the eager trainer
    at the same step."""
    from eppgcn_amd import graphs, train
    g = graphs.make_graph("cfg2_chunglu", device="cuda")
    mask = graphs.bernoulli_mask(g.num_nodes, 0.1, 2, "cuda")
    eager = train.Trainer(g, train_mask=mask, labels="uniform")
    graphed = train.Trainer(g, train_mask=mask, labels="uniform")
    for tr in (eager, graphed):
        for i in range(4):
            tr.train_step(i == 0)
    graph, loss = graphed.capture_epoch()          # three more eager epochs on a side stream, then the capture
    for _ in range(3):
        eager.train_step(False)
    for step in range(6):
        want = float(eager.train_step(False))
        graph.replay()
        torch.cuda.synchronize()
        got = float(loss)
        assert abs(got - want) <= 1e-5 * abs(want), f"replay {step}: {got} vs {want}"
        _ = torch.randn(512, 512, device="cuda") @ torch.randn(512, 512, device="cuda")   # unrelated eager work
        torch.cuda.synchronize()
    w_e = eager.model.convs[0].weights.detach()
    w_g = graphed.model.convs[0].weights.detach()
    assert torch.allclose(w_e, w_g, rtol=1e-4, atol=1e-6)


def test_entry_point_smoke_runs():
    """The repository's smoke entry point (one small pass of the whole path on cuda:0 against the checker) is part
    of the suite, so that a change of the library's contracts cannot leave it behind."""
    import __graft_entry__ as entry
    entry.smoke()
