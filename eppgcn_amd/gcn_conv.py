"""The GCN layer and its autograd function over the ``GNNAdvisor`` ops: same class names,
argument order and saved state as the reference's layer (EPPGCN/gcn_conv.py:7-65), so a model
written against the reference runs unchanged."""
from __future__ import annotations

import math

import torch

from . import gnnadvisor
from .param import *  # noqa: F401,F403  (the reference's module re-exports its parameter records)


class GNNAFunction(torch.autograd.Function):
    """forward: X*W then neighbour-group aggregation; on the first iteration also marks this
    layer's share of the backward path.  backward: pruned aggregation over the compacted path,
    then the two dense products for dX and dW.

    ``reluInput`` (an addition, default off) makes the layer consume ``relu(X)`` without the
    activation ever being written out: the product applies it while loading X, and the backward
    returns the gradient with respect to X itself (masked where X <= 0).  dX is skipped when X
    needs no gradient (the first layer's features)."""

    @staticmethod
    def forward(ctx, X, weight, inputInfo, maskInfo, backInfo, isFirstIter, isBackModeNet, reluInput=False):
        GNNA = gnnadvisor()
        ctx.save_for_backward(X, weight)
        ctx.inputInfo = inputInfo
        ctx.backInfo = backInfo
        ctx.reluInput = bool(reluInput)
        ctx.partSize, ctx.dimWorker, ctx.warpPerBlock = inputInfo.partSize, inputInfo.dimWorker, inputInfo.warpPerBlock
        X_prime = GNNA.forward(X, weight, inputInfo.row_pointers, inputInfo.column_index, inputInfo.degrees,
                               inputInfo.partPtr, inputInfo.part2Node, inputInfo.partSize, inputInfo.dimWorker,
                               inputInfo.warpPerBlock, relu_input=ctx.reluInput)[0]
        if isFirstIter and not isBackModeNet:
            GNNA.mask_forward(inputInfo.part2Node, inputInfo.partPtr, inputInfo.column_index, maskInfo.src_mask,
                              maskInfo.ngh_mask, maskInfo.backEdgeMask, maskInfo.node_degs, maskInfo.num_layers,
                              maskInfo.layer, maskInfo.blockx, maskInfo.blocky)
        return X_prime

    @staticmethod
    def backward(ctx, d_output):
        GNNA = gnnadvisor()
        X, weight = ctx.saved_tensors
        b = ctx.backInfo
        need_dx = bool(ctx.needs_input_grad[0])
        d_input, d_weight = GNNA.ours_backward(d_output.contiguous(), X, weight, b.id, b.partPointer, b.edgeList,
                                               b.degrees, b.partSize, b.numParts, b.layer, b.blockx, b.blocky,
                                               need_dx=need_dx, relu_input=ctx.reluInput)
        return (d_input if need_dx else None), d_weight, None, None, None, None, None, None


class GCNConv(torch.nn.Module):
    def __init__(self, input_dim, output_dim, relu_input=False):
        super().__init__()
        self.relu_input = bool(relu_input)
        self.weights = torch.nn.Parameter(torch.empty(input_dim, output_dim))
        self.reset_parameters()

    def reset_parameters(self):
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
