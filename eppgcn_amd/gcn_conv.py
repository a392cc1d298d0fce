"""The GCN layer and its autograd function over the ``GNNAdvisor`` ops: same class names,
argument order and saved state as the reference's layer (EPPGCN/gcn_conv.py:7-65), so a model
written against the reference runs unchanged."""
from __future__ import annotations

import math

import torch

from . import gnnadvisor
from .param import *  # noqa: F401,F403  (the reference's module re-exports its parameter records)


def _graph_args(info):
    """Positional tail of GNNA.forward after (X, W): graph, groups and the three launch hints."""
    return (info.row_pointers, info.column_index, info.degrees, info.partPtr, info.part2Node, info.partSize,
            info.dimWorker, info.warpPerBlock)


def _marking_args(info, mask):
    """Arguments of GNNA.mask_forward for one layer."""
    return (info.part2Node, info.partPtr, info.column_index, mask.src_mask, mask.ngh_mask, mask.backEdgeMask,
            mask.node_degs, mask.num_layers, mask.layer, mask.blockx, mask.blocky)


def _path_args(back):
    """Positional tail of GNNA.ours_backward after (dY, X, W): the compacted path of the layer."""
    return (back.id, back.partPointer, back.edgeList, back.degrees, back.partSize, back.numParts, back.layer,
            back.blockx, back.blocky)


class GNNAFunction(torch.autograd.Function):
    """forward: X*W then neighbour-group aggregation; on the first iteration also marks this
    layer's share of the backward path.  backward: pruned aggregation over the compacted path,
    then the two dense products for dX and dW.

    ``reluInput`` (an addition, default off) makes the layer consume ``relu(X)`` without the
    activation ever being written out: the product applies it while loading X, and the backward
    returns the gradient with respect to X itself (masked where X <= 0).  dX is skipped when X
    needs no gradient (the first layer's features).

    A path record with ``unpruned = True`` (an addition, for the "no pruning" ablation the reference's module
    exports as ``backward`` but its layer never calls) makes the backward run the unpruned aggregation over the
    forward groups instead: the same gradients, since the incoming gradient is zero outside the path."""

    @staticmethod
    def forward(ctx, X, weight, inputInfo, maskInfo, backInfo, isFirstIter, isBackModeNet, reluInput=False):
        ops = gnnadvisor()
        ctx.save_for_backward(X, weight)
        # the reference keeps these on ctx as well; backward only needs the path record
        ctx.inputInfo, ctx.backInfo, ctx.reluInput = inputInfo, backInfo, bool(reluInput)
        ctx.partSize, ctx.dimWorker, ctx.warpPerBlock = inputInfo.partSize, inputInfo.dimWorker, inputInfo.warpPerBlock
        (aggregated,) = ops.forward(X, weight, *_graph_args(inputInfo), relu_input=ctx.reluInput)
        if isFirstIter and not isBackModeNet:
            ops.mask_forward(*_marking_args(inputInfo, maskInfo))
        return aggregated

    @staticmethod
    def backward(ctx, d_output):
        X, weight = ctx.saved_tensors
        wants_dx = bool(ctx.needs_input_grad[0])
        if getattr(ctx.backInfo, "unpruned", False):
            d_input, d_weight = gnnadvisor().backward(d_output.contiguous(), X, weight, *_graph_args(ctx.inputInfo),
                                                      need_dx=wants_dx, relu_input=ctx.reluInput)
        else:
            d_input, d_weight = gnnadvisor().ours_backward(d_output.contiguous(), X, weight, *_path_args(ctx.backInfo),
                                                           need_dx=wants_dx, relu_input=ctx.reluInput)
        # one gradient slot per forward argument after ctx
        return (d_input if wants_dx else None, d_weight) + (None,) * 6


class GCNConv(torch.nn.Module):
    def __init__(self, input_dim, output_dim, relu_input=False):
        super().__init__()
        self.relu_input = bool(relu_input)
        self.weights = torch.nn.Parameter(torch.empty(input_dim, output_dim))
        self.reset_parameters()

    def reset_parameters(self):
        # U(-1/sqrt(out), 1/sqrt(out)), EPPGCN/gcn_conv.py:47-49
        bound = 1.0 / math.sqrt(self.weights.size(1))
        with torch.no_grad():
            self.weights.uniform_(-bound, bound)

    def print_time(self):
        gnnadvisor().print_time()

    def clear_time(self):
        gnnadvisor().clear_time()

    def forward(self, X, inputInfo, maskInfo, backInfo, isFirstIter, isBackModeNet):
        """X: [N, in] node features; the three records carry the graph, the path-marking
        buffers and the compacted backward path of this layer."""
        return GNNAFunction.apply(X, self.weights, inputInfo, maskInfo, backInfo, isFirstIter, isBackModeNet,
                                  self.relu_input)
