"""The reference driver's training loop around the aggregation path (EPPGCN/gcn_main.py:120-292)
as a library: a multi-layer GCN over the ``GNNAdvisor`` ops with the execution path prepared on
the first iteration, timed the way the reference times it; and the host-CPU comparison run (the
same model through ``torch.sparse.mm`` on the CPU)."""
from __future__ import annotations

import os
import time
from typing import List

import torch
import torch.nn.functional as F

from . import gnnadvisor, graphs
from .gcn_conv import GCNConv
from .param import backInputProperty, inputProperty, maskInputProperty


class GraphDataset:
    """The fields of the reference's dataset object the path needs (EPPGCN/dataset.py:22-156):
    CSR, scale vector, features, labels, train mask and the per-run buffers the path mutates
    (neighbour masks = False, edge masks = -1, kept degrees = 0)."""

    def __init__(self, graph: graphs.Graph, dim=96, num_classes=22, num_layers=2, train_mask=None,
                 train_ratio=0.1, labels="ones", feature_seed=1, mask_seed=2, label_seed=4):
        dev = graph.column_index.device
        n, e = graph.num_nodes, graph.num_edges
        self.num_nodes, self.num_edges = n, e
        self.num_features, self.num_classes, self.num_layers = dim, num_classes, num_layers
        self.avg_degree = e / n
        self.avg_edgeSpan = -1
        self.row_pointers, self.column_index, self.degrees = graph.row_pointers, graph.column_index, graph.degrees
        self.x = graphs.normal32(feature_seed, (n, dim), dev)
        # the reference labels every vertex 1 (EPPGCN/dataset.py:133); "uniform" draws real classes
        self.y = (torch.ones(n, dtype=torch.long, device=dev) if labels == "ones"
                  else graphs.uniform_labels(label_seed, n, num_classes, dev))
        self.train_mask = (graphs.bernoulli_mask(n, train_ratio, mask_seed, dev) if train_mask is None
                           else train_mask.to(dev))
        self.ngh_masks = [torch.zeros(n, dtype=torch.bool, device=dev) for _ in range(num_layers - 1)]
        self.empty_mask = torch.zeros(0, dtype=torch.bool, device=dev)
        self.edge_masks = [torch.full((e,), -1, dtype=torch.int32, device=dev) for _ in range(num_layers)]
        self.node_degs = [torch.zeros(n, dtype=torch.int32, device=dev) for _ in range(num_layers)]


class Net(torch.nn.Module):
    """The reference's model (EPPGCN/gcn_main.py:190-208): conv -> relu -> ... -> conv.  With
    ``fuse_relu`` (default) the activation between two layers is applied by the consuming layer
    while it loads its input instead of by a separate F.relu pass; the function computed is the
    same."""

    def __init__(self, dataset: GraphDataset, hidden: int, num_layers: int, weight_seed: int = None,
                 fuse_relu: bool = True):
        super().__init__()
        self.num_layers = num_layers
        self.fuse_relu = fuse_relu
        self.convs = torch.nn.ModuleList()
        for i in range(num_layers):
            fan_in = hidden if i != 0 else dataset.num_features
            fan_out = hidden if i < num_layers - 1 else dataset.num_classes
            conv = GCNConv(fan_in, fan_out, relu_input=fuse_relu and i != 0)
            if weight_seed is not None:
                with torch.no_grad():
                    conv.weights.copy_(graphs.uniform_weights(weight_seed + i, fan_in, fan_out))
            self.convs.append(conv)

    def forward(self, x, inputInfo, mask_props, back_props, isFirstIter, isBackModeNet):
        for i in range(self.num_layers):
            info = inputInfo.set_input() if i == 0 else inputInfo.set_hidden()
            x = self.convs[i](x, info, mask_props[i], back_props[i], isFirstIter, isBackModeNet)
            if i < self.num_layers - 1 and not self.fuse_relu:
                x = F.relu(x)
        return x


class Trainer:
    """Wiring of EPPGCN/gcn_main.py: decider -> build_part -> mask/back records -> Net -> Adam."""

    def __init__(self, graph: graphs.Graph, dim=96, hidden=16, num_classes=22, num_layers=2, train_ratio=0.1,
                 train_mask=None, backsize_mode="constant", backsize=32, labels="ones", weight_seed=3, lr=0.01,
                 fuse_relu=True, dataset=None, part_size=32, dim_worker=32, warp_per_block=8, shared_mem=100,
                 manual_mode=False, verbose=False, prune=True):
        """``dataset``: a loaded ``eppgcn_amd.dataset.custom_dataset`` (or any object with the same
        attributes) to train on instead of synthetic features over ``graph``.  ``part_size`` ...
        ``manual_mode`` are the driver's forward launch flags (EPPGCN/gcn_main.py:34-40).  ``prune=False``: the
        backward of every layer runs the unpruned aggregation (the module's ``backward`` export) instead of the
        pruned one over the prepared path - the ablation next to which the pruned times are read."""
        self.prune = bool(prune)
        self.GNNA = gnnadvisor()
        self.backsize_mode, self.backsize = backsize_mode, backsize
        if dataset is not None:
            ds = dataset
            dim, num_classes, num_layers = ds.num_features, ds.num_classes, ds.num_layers
        else:
            ds = GraphDataset(graph, dim, num_classes, num_layers, train_mask, train_ratio, labels)
        self.dataset = ds
        self.num_layers = num_layers
        info = inputProperty(ds.row_pointers, ds.column_index, ds.degrees, part_size, dim_worker, warp_per_block,
                             shared_mem, hiddenDim=hidden, dataset_obj=ds, manual_mode=manual_mode, verbose=verbose)
        info.decider()
        if verbose:
            info.set_input().print_param()
            info.set_hidden().print_param()
        part_ptr, part2node = self.GNNA.build_part(info.partSize, ds.row_pointers)
        info.partPtr, info.part2Node = part_ptr.int(), part2node.int()
        self.inputInfo = info
        self.mask_props: List[maskInputProperty] = []
        self.back_props: List[backInputProperty] = []
        for i in range(num_layers):
            src = ds.ngh_masks[i - 1] if i != 0 else ds.train_mask
            dst = ds.ngh_masks[i] if i < num_layers - 1 else ds.empty_mask
            width = hidden if i < num_layers - 1 else num_classes
            self.mask_props.append(maskInputProperty(src, dst, ds.edge_masks[num_layers - 1 - i],
                                                     ds.node_degs[num_layers - 1 - i], num_layers, i + 1, width))
            self.back_props.append(backInputProperty(degrees=ds.degrees, dim=width, layer=i + 1))
            self.back_props[-1].unpruned = not self.prune
        self.model = Net(ds, hidden, num_layers, weight_seed, fuse_relu).to(ds.x.device)
        self.optimizer = torch.optim.Adam(self.model.parameters(), lr=lr)
        self.for_time = self.loss_time = self.back_time = self.build_time = 0.0
        self.losses: List[float] = []
        self.train_idx = self.train_y = None
        self.kept_edges = [None] * num_layers      # per conv layer, filled by build_back_part

    def build_back_part(self):
        """EPPGCN/gcn_main.py:151-168 ('net' mode, which needs an unpublished predictor, is not offered)."""
        ds = self.dataset
        for i in range(self.num_layers):
            ids, edge_list, info = self.GNNA.compact_back_edge(ds.edge_masks[i], self.inputInfo.column_index)
            valid_len = int(info[0].item())
            if self.backsize_mode == "map":
                part_size = self.GNNA.get_map_back_part_size(ds.node_degs[i], valid_len)
            elif self.backsize_mode == "wave64":
                part_size = self.GNNA.get_wave64_back_part_size(ds.node_degs[i], valid_len)
            else:
                part_size = max(1, self.backsize)
            part_pointer, num_parts = self.GNNA.split_back_part(ds.node_degs[i], ds.num_edges, part_size)
            self.back_props[i].fillProperty(ids, part_pointer, edge_list, part_size, int(num_parts[0].item()))
            self.kept_edges[i] = valid_len
            ds.edge_masks[i] = None      # the marking buffer is not needed after compaction

    def _loss(self, out):
        """Mean negative log-likelihood of the training rows (F.nll_loss of F.log_softmax,
        EPPGCN/gcn_main.py:252-253).  Written as a gather and a mean: torch's nll_loss kernels
        reduce all rows in one workgroup (0.53 + 0.33 ms per epoch for 4.2e5 rows here)."""
        logp = F.log_softmax(out.index_select(0, self.train_idx), dim=1)
        return -logp.gather(1, self.train_y.unsqueeze(1)).mean()

    def train_step(self, is_first_iter: bool, record_loss: bool = False, phase_timers: bool = True):
        """One epoch.  ``phase_timers`` keeps the reference's three host synchronisations per epoch
        that split the time into forward / loss / backward (EPPGCN/gcn_main.py:242,254,260); without
        them the epoch is issued asynchronously and only the caller synchronises."""
        ds = self.dataset
        sync = torch.cuda.synchronize if phase_timers else (lambda: None)
        self.model.train()
        self.optimizer.zero_grad()
        t = time.perf_counter()
        out = self.model(ds.x, self.inputInfo, self.mask_props, self.back_props, is_first_iter, False)
        sync()
        self.for_time += time.perf_counter() - t
        if is_first_iter:
            t = time.perf_counter()
            self.build_back_part()
            torch.cuda.synchronize()
            self.build_time += time.perf_counter() - t
        t = time.perf_counter()
        # EPPGCN/gcn_main.py:252-253 takes log_softmax of every row and then selects the training
        # rows with the boolean mask (a device-to-host round trip per epoch); selecting the rows
        # first, through indices computed once, is the same function of `out`
        if self.train_idx is None:
            self.train_idx = ds.train_mask.nonzero().squeeze(1)
            self.train_y = ds.y[self.train_idx]
        loss = self._loss(out)
        sync()
        self.loss_time += time.perf_counter() - t
        t = time.perf_counter()
        loss.backward()
        sync()
        self.back_time += time.perf_counter() - t
        self.optimizer.step()
        if record_loss:
            self.losses.append(float(loss.item()))
        return loss

    def run(self, epochs=100, warmup=10, record_loss=False, kernel_timing=False, phase_timers=True):
        """10 warm-up epochs (the first prepares the path), timers cleared, then `epochs` timed
        epochs between two synchronisations (EPPGCN/gcn_main.py:272-292)."""
        for i in range(warmup):
            self.GNNA.set_timing(i == 0)      # path marking runs once, here: keep its time for print_time
            self.train_step(i == 0, record_loss)
        self.for_time = self.loss_time = self.back_time = 0.0
        self.GNNA.clear_time()
        self.GNNA.set_timing(bool(kernel_timing))
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(epochs):
            self.train_step(False, record_loss, phase_timers)
        torch.cuda.synchronize()
        total = time.perf_counter() - t
        self.GNNA.set_timing(False)
        res = {"epochs": epochs, "warmup": warmup, "Time": round(total, 6), "for_time": round(self.for_time, 6),
               "loss_time": round(self.loss_time, 6), "back_time": round(self.back_time, 6),
               "build_time": round(self.build_time, 6),
               "backward_group_sizes": [b.partSize for b in self.back_props],
               "backward_groups": [b.numParts for b in self.back_props],
               "kept_edges": list(self.kept_edges), "pruned": self.prune}
        if kernel_timing:
            res["for_agg_time"] = round(self.GNNA.get_time_ms(0) / 1e3, 6)
            res["back_agg_time"] = round(self.GNNA.get_time_ms(1) / 1e3, 6)
            res["mask_time"] = round(self.GNNA.get_time_ms(2) / 1e3, 6)
            # l{k}_back_agg_time of the reference's report (EPPGCN_kernel.cu:96-106); the unpruned ablation has no
            # per-layer timers (its entry point has no layer argument)
            res["layer_back_agg_time"] = [round(self.GNNA.get_time_ms(101 + k) / 1e3, 6) for k in range(self.num_layers)]
        return res


    # ------------------------------------------------------------------ whole epoch as one HIP graph
    def capture_epoch(self):
        """Records one steady-state epoch (forward, loss, backward, Adam step) into a HIP graph
        and returns (graph, loss tensor the replays overwrite).  The path must be prepared
        (run at least one first-iteration step before).  The optimizer is rebuilt with
        capturable state; the layer ops allocate from the graph's private pool and the library
        itself records kernel nodes only."""
        ds = self.dataset
        if self.train_idx is None:
            raise RuntimeError("run a first-iteration train_step before capturing")
        state = self.optimizer.state_dict()
        self.optimizer = torch.optim.Adam(self.model.parameters(), lr=state["param_groups"][0]["lr"], capturable=True)
        if state["state"]:
            for entry in state["state"].values():
                if not torch.is_tensor(entry["step"]) or not entry["step"].is_cuda:
                    entry["step"] = torch.as_tensor(float(entry["step"]), dtype=torch.float32, device=ds.x.device)
            for group in state["param_groups"]:
                group["capturable"] = True
            self.optimizer.load_state_dict(state)

        def epoch():
            self.optimizer.zero_grad(set_to_none=True)
            out = self.model(ds.x, self.inputInfo, self.mask_props, self.back_props, False, False)
            loss = self._loss(out)
            loss.backward()
            self.optimizer.step()
            return loss

        self.GNNA.set_timing(False)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):            # warm-up on a side stream, as graph capture requires
            for _ in range(3):
                epoch()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            loss = epoch()
        return graph, loss

    def run_graphed(self, epochs=100):
        """`epochs` replays of the captured epoch between two synchronisations."""
        graph, loss = self.capture_epoch()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(epochs):
            graph.replay()
        torch.cuda.synchronize()
        return {"epochs": epochs, "Time": round(time.perf_counter() - t, 6), "last_loss": float(loss.item())}


def time_gpu_training(graph, wl=None, epochs=100, warmup=10, backsize_mode="constant", backsize=32):
    """100-epoch time of the 2-layer GCN (96 -> 16 -> 22) on the GPU; runs twice: once untimed
    per kernel (the headline `Time`), once with per-kernel events for the aggregation split."""
    train_mask = None if wl is None else wl.train_mask
    tr = Trainer(graph, train_mask=train_mask, backsize_mode=backsize_mode, backsize=backsize)
    res = tr.run(epochs, warmup)
    res["Time_without_phase_timers"] = tr.run(epochs, 0, phase_timers=False)["Time"]
    timed = tr.run(min(epochs, 20), 0, kernel_timing=True)
    res["agg_ms_per_epoch_in_training"] = round(
        (timed["for_agg_time"] + timed["back_agg_time"]) * 1e3 / timed["epochs"], 4)
    res["mask_time"] = timed["mask_time"]
    try:                                     # the same epoch replayed from one HIP graph
        res["Time_hip_graph"] = tr.run_graphed(epochs)["Time"]
    except Exception as exc:                 # capture support must never hide the eager figures
        res["Time_hip_graph"] = repr(exc)
    return res


def smoke_step(graph, wl=None):
    tr = Trainer(graph, train_mask=None if wl is None else wl.train_mask, backsize=8, labels="uniform")
    first = float(tr.train_step(True).item())
    for _ in range(5):
        last = float(tr.train_step(False).item())
    assert last == last and last < first, f"loss did not decrease: {first} -> {last}"


# ------------------------------------------------------------------ host-CPU comparison run
class _SymSparseMM(torch.autograd.Function):
    """A @ X through torch.sparse.mm; the backward uses A's symmetry (dX = A @ dY) so that no
    transposed copy of A is built per step.  Both products are timed."""

    @staticmethod
    def forward(ctx, a, x, clock):
        ctx.a, ctx.clock = a, clock
        t = time.perf_counter()
        y = torch.sparse.mm(a, x)
        clock[0] += time.perf_counter() - t
        return y

    @staticmethod
    def backward(ctx, dy):
        t = time.perf_counter()
        dx = torch.sparse.mm(ctx.a, dy.contiguous())
        ctx.clock[0] += time.perf_counter() - t
        return None, dx, None


def time_cpu_sparse_training(graph, train_mask, epochs=100, max_seconds=60.0, dim=96, hidden=16,
                             num_classes=22, lr=0.01, weight_seed=3):
    """The same 2-layer GCN through PyTorch CPU sparse aggregation on the host cores.  Runs at
    least 2 and at most `epochs` epochs within `max_seconds` after one warm-up epoch and
    extrapolates linearly to `epochs` (stated in the result)."""
    g = graph.to("cpu")
    n = g.num_nodes
    row = g.row_index()
    vals = g.degrees[row] * g.degrees[g.column_index.long()]
    a = torch.sparse_csr_tensor(g.row_pointers.long(), g.column_index.long(), vals, size=(n, n))
    x = graphs.normal32(1, (n, dim), "cpu")
    y = torch.ones(n, dtype=torch.long)
    mask = train_mask.cpu()
    w0 = graphs.uniform_weights(weight_seed, dim, hidden).requires_grad_()
    w1 = graphs.uniform_weights(weight_seed + 1, hidden, num_classes).requires_grad_()
    opt = torch.optim.Adam([w0, w1], lr=lr)
    clock = [0.0]

    def epoch():
        opt.zero_grad()
        h = F.relu(_SymSparseMM.apply(a, x @ w0, clock))
        out = _SymSparseMM.apply(a, h @ w1, clock)
        loss = F.nll_loss(F.log_softmax(out, dim=1)[mask], y[mask])
        loss.backward()
        opt.step()
        return float(loss.item())

    epoch()
    clock[0] = 0.0
    done = 0
    t0 = time.perf_counter()
    while done < epochs and (done < 2 or time.perf_counter() - t0 < max_seconds):
        epoch()
        done += 1
    dt = time.perf_counter() - t0
    return {"epochs_run": done, "seconds_run": round(dt, 3), "Time_extrapolated_to": epochs,
            "Time": round(dt / done * epochs, 3), "agg_ms_per_epoch": round(clock[0] / done * 1e3, 2),
            "threads": torch.get_num_threads(), "host_cpus": os.cpu_count(),
            "note": "torch.sparse.mm (CSR, fp32) forward and backward; linear extrapolation from epochs_run"}
