"""CPU tests of the host-side pieces: benchmark graph generators, parameter records, byte
accounting.  No GPU, no HIP calls."""
import numpy as np
import pytest
import torch

from eppgcn_amd import graphs, param, workload


def _check_graph(g):
    indptr, col = g.row_pointers.numpy().astype(np.int64), g.column_index.numpy().astype(np.int64)
    n = g.num_nodes
    assert indptr[0] == 0 and indptr[-1] == col.size and indptr.size == n + 1
    row = np.repeat(np.arange(n), np.diff(indptr))
    keys = row * n + col
    assert np.all(np.diff(keys) > 0), "columns sorted and unique inside each row"
    assert np.array_equal(np.sort(col * n + row), keys), "symmetric"
    assert np.all(np.isin(np.arange(n) * n + np.arange(n), keys)), "one self-loop per vertex"
    deg = np.diff(indptr)
    assert np.allclose(g.degrees.numpy(), 1 / np.sqrt(deg), rtol=1e-6)


def test_cfg1_uniform_graph_matches_the_configuration():
    g = graphs.make_graph("cfg1_uniform")
    assert (g.num_nodes, g.num_edges) == (2708, 2 * 5278 + 2708)
    _check_graph(g)
    assert torch.equal(g.column_index, graphs.make_graph("cfg1_uniform").column_index)   # seeded


def test_cfg2_chung_lu_graph_matches_the_configuration():
    g = graphs.make_graph("cfg2_chunglu")
    assert (g.num_nodes, g.num_edges) == (19717, 2 * 44325 + 19717)
    _check_graph(g)
    deg = np.diff(g.row_pointers.numpy())
    assert deg.max() > 50 * np.median(deg)        # heavy tail


def test_rmat_generator_is_skewed_and_device_independent_arithmetic():
    g = graphs.rmat_graph(12, 8, seed=0)
    _check_graph(g)
    assert g.num_nodes == 4096 and 30000 < g.num_edges <= 2 * 8 * 4096 + 4096
    deg = np.diff(g.row_pointers.numpy())
    assert deg.max() > 20 * deg.mean()
    # quadrant probabilities: the top-left quadrant of the first level gets ~a of the pairs
    src, dst = graphs.rmat_pairs(12, 200000, seed=1)
    top_left = ((src < 2048) & (dst < 2048)).double().mean().item()
    assert abs(top_left - 0.57) < 0.01
    bottom_right = ((src >= 2048) & (dst >= 2048)).double().mean().item()
    assert abs(bottom_right - 0.05) < 0.01


def test_scale_vector_both_fillings():
    indptr = torch.tensor([0, 4, 4, 13], dtype=torch.int32)
    assert torch.allclose(graphs.scale_vector(indptr, "inv_sqrt"), torch.tensor([0.5, 1.0, 1 / 3]))
    assert torch.allclose(graphs.scale_vector(indptr, "sqrt"), torch.tensor([2.0, 1.0, 3.0]))


def test_mask_weights_features_are_seeded_and_distributed():
    m = graphs.bernoulli_mask(200000, 0.1, 2)
    assert abs(m.double().mean().item() - 0.1) < 0.005 and torch.equal(m, graphs.bernoulli_mask(200000, 0.1, 2))
    w = graphs.uniform_weights(3, 96, 16)
    assert w.abs().max() <= 0.25 and abs(w.mean().item()) < 0.02
    x = graphs.normal32(1, (50000, 4))
    assert abs(x.mean().item()) < 0.02 and abs(x.std().item() - 1) < 0.02


def test_get_block_size_table_is_one_wavefront():
    for dim, want in [(1, (2, 32)), (7, (2, 32)), (8, (4, 16)), (16, (4, 16)), (22, (4, 16)), (31, (4, 16)),
                      (32, (8, 8)), (95, (8, 8)), (96, (16, 4)), (191, (16, 4)), (192, (32, 2)), (256, (32, 2)),
                      (4096, (32, 2))]:
        assert param.getBlockSize(dim) == want
        assert want[0] * want[1] == 64


class _DS:
    num_nodes, avg_degree, num_features = 1000, 31.6, 96


def test_decider_rules():
    info = param.inputProperty(None, None, None, 32, 32, 8, 100, hiddenDim=16, dataset_obj=_DS(), manual_mode=False)
    info.decider()
    assert info.partSize == 31 and info.warpPerBlock_input == 8 and info.warpPerBlock_hidden == 8
    assert info.set_input().dimWorker == 32 and info.set_hidden().dimWorker == 16
    ds = _DS()
    ds.avg_degree = 0.4
    info = param.inputProperty(None, None, None, 32, 32, 8, 100, hiddenDim=16, dataset_obj=ds, manual_mode=False)
    info.decider()
    assert info.partSize == param.MIN_AUTO_PART_SIZE == 16     # never 0: the wave64 floor
    info = param.inputProperty(None, None, None, 5, 32, 8, 100, hiddenDim=16, dataset_obj=_DS(), manual_mode=True)
    info.decider()
    assert info.partSize == 5                      # manual group size respected
    with pytest.raises(ValueError):
        param.inputProperty()


def test_algorithmic_bytes_nominal_values():
    n, e = 4_194_304, 134_000_000
    assert abs(workload.bytes_forward(n, e, 16) / 1e9 - 9.95) < 0.05
    assert abs(workload.bytes_forward(n, e, 22) / 1e9 - 13.27) < 0.05
    assert workload.bytes_forward(10, 100, 16) == 100 * 72 + 10 * 72
    assert workload.bytes_pruned_backward(10, 50, 7, 22) == 50 * 96 + 10 * 88 + 56
    assert workload.bytes_compact(100, 10) == 400 + 120
    assert workload.bytes_compulsory(10, 100, 16) == 400 + 80 + 1280


def test_driver_command_line_takes_the_reference_flags(capsys):
    """Every flag EPPGCN/bench_EPPGCN.py:54-58 puts on the command line parses, with the
    reference's defaults (EPPGCN/gcn_main.py:21-50) except the 'net' group-size predictor, which
    is refused before anything touches a device."""
    from eppgcn_amd import gcn_main
    line = ("--dataset cora --dim 1433 --hidden 16 --classes 7 --layers 3 --partSize 0 --model gcn --warpPerBlock 8 "
            "--manual_mode False --verbose_mode False --loadFromTxt True --dataDir /data/cora --train_ratio 0.3 "
            "--backsize_mode constant --backsize 32").split()
    a = gcn_main.build_parser().parse_args(line)
    assert (a.dataset, a.dim, a.classes, a.layers, a.train_ratio, a.backsize_mode, a.backsize) == \
        ("cora", 1433, 7, 3, 0.3, "constant", 32)
    d = gcn_main.build_parser().parse_args([])
    assert (d.dim, d.hidden, d.classes, d.layers, d.train_ratio, d.num_epoches, d.partSize, d.dimWorker,
            d.warpPerBlock, d.sharedMem, d.manual_mode, d.loadFromTxt, d.backsize) == \
        (96, 16, 22, 2, 0.1, 100, 32, 32, 8, 100, "False", "True", 0)
    assert d.backsize_mode == "constant"
    assert gcn_main.main(["--backsize_mode", "net"]) == 2
    out = capsys.readouterr()
    assert out.out.startswith("||amazon0601   0.1   2") and "net" in out.err


def test_sweep_driver_formats_the_reference_flags():
    """The datasets x ratios x depths sweep hands the driver the flags the reference's script formats
    (EPPGCN/bench_EPPGCN.py:41-59): automatic forward group size, `map` for the fitted regression,
    constant 32 for `fixed_value`, `net` for the predictor (which the driver refuses)."""
    from eppgcn_amd import bench_eppgcn as sweep, gcn_main
    args = sweep.build_parser().parse_args([])
    assert [d[0] for d in args.datasets] == ["cora", "citeseer", "pubmed", "youtube", "amazon", "corafull", "catalog",
                                             "twitter", "google", "dblp"]
    assert (args.ratios, args.layers, args.hidden) == ([0.1, 0.3, 0.5, 0.8], [3, 4, 5, 6], [16])
    assert sweep.parse_dataset("pubmed") == ("pubmed", 500, 3)
    assert sweep.parse_dataset("mygraph") == ("mygraph", 96, 22) and sweep.parse_dataset("g,8,3") == ("g", 8, 3)
    with pytest.raises(Exception):
        sweep.parse_dataset("g,8")
    for model, mode, size in (("regression_equation", "map", 0), ("fixed_value", "constant", 32), ("SAGPG", "net", 0)):
        args = sweep.build_parser().parse_args(["--groupsize_model", model, "--dataRoot", "/nowhere"])
        argv = sweep.driver_arguments(args, "cora", 1433, 7, 16, 0.3, 5)
        ns = gcn_main.build_parser().parse_args(argv)          # every flag is one the driver knows
        assert (ns.dataset, ns.dim, ns.classes, ns.hidden, ns.layers, ns.train_ratio) == ("cora", 1433, 7, 16, 5, 0.3)
        assert (ns.backsize_mode, ns.backsize, ns.manual_mode, ns.partSize) == (mode, size, "False", 0)
        assert ns.dataDir == "/nowhere"


def test_counter_summary_is_only_used_for_the_sources_it_was_taken_from(tmp_path, monkeypatch):
    """bench.py reports measured traffic from a committed rocprofv3 summary only while the kernel sources
    still hash to what the summary names; otherwise the field is null with the reason."""
    import bench
    h = bench.kernel_source_hash()
    assert len(h) == 16 and h == bench.kernel_source_hash()
    prof = tmp_path / "profiles"
    prof.mkdir()
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    monkeypatch.setattr(bench, "kernel_source_hash", lambda: h)
    assert bench.measured_traffic("cfgX", "fwd")[0] is None
    (prof / "a.md").write_text(f"    kernel_source_sha256 = {h}\n    traffic_bytes cfgX fwd = 1.5e+09\n")
    assert bench.measured_traffic("cfgX", "fwd") == (1.5e9, "profiles/a.md")
    assert bench.measured_traffic("cfgX", "bwd")[0] is None
    (prof / "a.md").write_text("    kernel_source_sha256 = 0123456789abcdef\n    traffic_bytes cfgX fwd = 1.5e+09\n")
    value, why = bench.measured_traffic("cfgX", "fwd")
    assert value is None and "other kernel sources" in why
    (prof / "a.md").write_text("    traffic_bytes cfgX fwd = 1.5e+09\n")
    assert bench.measured_traffic("cfgX", "fwd")[0] is None


def test_live_counter_attribution_and_guards(tmp_path, monkeypatch):
    """bench.py's live traffic figure: the k-th stream-kernel dispatch of a `--traffic_probe` run belongs to call
    k mod 4, together with the clear / pre-scaling dispatches right before it and the fix-up right after it; a run
    with another number of stream-kernel dispatches is refused; no counter runs are started from a process that is
    itself under a profiler."""
    import csv
    import bench
    rows, did = [], 0

    def dispatch(name, **counters):
        nonlocal did
        did += 1
        for k, v in counters.items():
            for half in (0.25, 0.75):                      # rocprofv3 writes one row per counter instance
                rows.append({"Dispatch_Id": did, "Kernel_Name": name, "Counter_Name": k, "Counter_Value": v * half})

    rd = lambda n: {"TCC_EA0_RDREQ_sum": 3 * n, "TCC_EA0_RDREQ_32B_sum": n, "TCC_EA0_RDREQ_64B_sum": n, "TCC_EA0_RDREQ_128B_sum": n}
    dispatch("void eppgcn::plan_keys_kernel(int*)", **rd(1000))            # set-up: belongs to no call
    dispatch("eppgcn::zero_words_kernel(unsigned int*, unsigned long)", **rd(1000))
    dispatch("void at::native::something<float>(float*)", **rd(1000))
    for rep in range(bench.PROBE_REPS):
        dispatch("void eppgcn::scale_rows_flat4_kernel<unsigned int>(float*)", **rd(1))
        dispatch("void eppgcn::aggregate_stream_kernel<0, 4, 8, false>(float*, float*)", **rd(10))
        dispatch("void eppgcn::stream_fixup_kernel<0, 4>(float*)", **rd(100))
        dispatch("void eppgcn::scale_rows_kernel<unsigned int>(float*)", **rd(2))
        dispatch("void eppgcn::aggregate_stream_kernel<2, 8, 8, false>(float*, float*)", **rd(20))       # no fix-up
        dispatch("eppgcn::zero_words_kernel(unsigned int*, unsigned long)", **rd(3))
        dispatch("eppgcn::scale_listed_rows_kernel(float*)", **rd(3))
        dispatch("void eppgcn::aggregate_stream_kernel<2, 8, 8, false>(float*, float*)", **rd(30))
        dispatch("void eppgcn::stream_fixup_kernel<2, 8>(float*)", **rd(300))
        dispatch("void eppgcn::zero_listed_rows_kernel<4>(float*)", **rd(4))
        dispatch("eppgcn::scale_listed_rows_kernel(float*)", **rd(4))
        dispatch("void eppgcn::aggregate_stream_kernel<0, 4, 8, false>(float*, float*)", **rd(40))
        dispatch("void eppgcn::stream_fixup_kernel<0, 4>(float*)", **rd(400))
    path = tmp_path / "run_counter_collection.csv"
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"])
        w.writeheader()
        w.writerows(rows)
    read_b = lambda c: 32 * c["TCC_EA0_RDREQ_32B_sum"] + 64 * c["TCC_EA0_RDREQ_64B_sum"] + 128 * c["TCC_EA0_RDREQ_128B_sum"]
    got = bench.call_bytes_from_counters(str(path), read_b)
    assert got == {"fwd_agg_d16": 224.0 * 111, "fwd_agg_d22": 224.0 * 22, "bwd_agg_d22_last": 224.0 * 336,
                   "bwd_agg_d16_first": 224.0 * 448}
    with open(path, "a", newline="") as f:               # a thirteenth stream-kernel dispatch: not the probe's sequence
        csv.writer(f).writerow([did + 1, "void eppgcn::aggregate_stream_kernel<0, 4, 8, false>(float*)", "TCC_EA0_RDREQ_sum", 1])
    with pytest.raises(RuntimeError, match="13 stream-kernel dispatches"):
        bench.call_bytes_from_counters(str(path), read_b)
    monkeypatch.setenv("ROCPROFILER_LIBRARY_CTOR", "1")
    value, why = bench.live_traffic()
    assert value is None and "under a profiler" in why
