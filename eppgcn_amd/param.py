"""Launch-parameter records the layer passes to the ops.  The attribute names are the ones the
reference's autograd function reads (EPPGCN/gcn_conv.py:13-14,21-27,36-38; the records are
defined in EPPGCN/param.py).  The integers are hints sized for 32-lane warps: the HIP library
picks its own wave64 mapping from the feature width and only requires them to be positive, so
they are kept for signature compatibility and for reporting."""
from __future__ import annotations

# upper bounds of the feature width -> (lanes per group, groups per block); 64 threads each,
# i.e. one wavefront (table of EPPGCN/param.py:6-24)
_BLOCK_SHAPES = ((8, (2, 32)), (32, (4, 16)), (96, (8, 8)), (192, (16, 4)))


def getBlockSize(dim):
    for below, shape in _BLOCK_SHAPES:
        if dim < below:
            return shape
    return 32, 2


# Smallest automatic forward group size.  The reference's rule, int(average degree), was tuned for
# one 32-lane warp walking a group serially; a wave64 team gathers 8 rows at a time, and groups
# below about 16 slots leave most of that depth unused (R-MAT scale 20, average degree 8.8:
# group size 8 / 16 / 32 -> 0.245 / 0.214 / 0.212 ms per width-22 forward launch).
MIN_AUTO_PART_SIZE = 16


class _Record(object):
    """Attribute bag: every keyword becomes an attribute of the same name."""

    def _take(self, **fields):
        for name, value in fields.items():
            setattr(self, name, value)


class inputProperty(_Record):
    """Forward-side inputs: CSR, scale vector, neighbour groups and launch hints."""

    MAX_warpPerBlock = 8
    gap_smem = 100

    def __init__(self, row_pointers=None, column_index=None, degrees=None, partSize=None, dimWorker=None,
                 warpPerBlock=None, sharedMem=None, hiddenDim=None, dataset_obj=None, manual_mode=True,
                 verbose=False):
        if dataset_obj is None:
            raise ValueError("Dataset object MUST SET !!!")
        self._take(dataset_obj=dataset_obj, row_pointers=row_pointers, column_index=column_index, degrees=degrees,
                   partSize=partSize, dimWorker=dimWorker, warpPerBlock=warpPerBlock, hiddenDim=hiddenDim,
                   manual_mode=manual_mode, verbose_flag=verbose, partPtr=None, part2Node=None,
                   state_set_input=False)
        self._take(num_nodes=dataset_obj.num_nodes, avgNodeDegree=dataset_obj.avg_degree,
                   avgEdgeSpan=getattr(dataset_obj, "avg_edgeSpan", -1), inputDim=dataset_obj.num_features)
        # per-layer-kind hints chosen by decider(); set_input() / set_hidden() select one pair
        self._take(dimWorker_input=dimWorker, dimWorker_hidden=dimWorker, warpPerBlock_input=warpPerBlock,
                   warpPerBlock_hidden=warpPerBlock)
        self.share_memory = 0.4 * (100 if sharedMem is None else sharedMem)

    def _warps_for(self, width):
        """Warps per block from the reference's shared-memory estimate, between 1 and 8."""
        per_warp = 4 * (self.partSize + width)
        estimate_kb = min(self.MAX_warpPerBlock * (per_warp + 4 * self.gap_smem) / 1e3, self.share_memory)
        return max(1, min(int(estimate_kb * 1e3 / per_warp), self.MAX_warpPerBlock))

    def decider(self):
        """The reference's rule (EPPGCN/param.py:72-127): group size = int(average degree), warps per
        block from a shared-memory estimate capped at 8, dimension workers = min(width, 32).
        Unlike the reference, a manual group size is respected in manual mode and the automatic
        one never drops below MIN_AUTO_PART_SIZE (the reference's can reach 0, which divides by
        zero in build_part)."""
        if not (self.manual_mode and self.partSize):
            self.partSize = max(MIN_AUTO_PART_SIZE, int(self.avgNodeDegree))
        self._take(warpPerBlock_input=self._warps_for(self.inputDim),
                   warpPerBlock_hidden=self._warps_for(self.hiddenDim),
                   dimWorker_input=min(self.inputDim, 32), dimWorker_hidden=min(self.hiddenDim, 32))
        if self.verbose_flag:
            print("\n=> AUTO Decider Complete !!!\n")

    def _select(self, which):
        self._take(dimWorker=getattr(self, "dimWorker_" + which), warpPerBlock=getattr(self, "warpPerBlock_" + which),
                   state_set_input=(which == "input"))
        return self

    def set_input(self):
        return self._select("input")

    def set_hidden(self):
        return self._select("hidden")

    def print_param(self):
        if not self.verbose_flag:
            return
        tag = "{} {}".format("manual" if self.manual_mode else "auto", "INPUT" if self.state_set_input else "HIDDEN")
        for name in ("partSize", "dimWorker", "warpPerBlock"):
            print("# {} {}: {}".format(tag, name, getattr(self, name)))


class maskInputProperty(_Record):
    """Inputs of one path-marking step (one per layer, first iteration only)."""

    def __init__(self, src_mask=None, ngh_mask=None, backEdgeMask=None, node_degs=None, num_layers=None,
                 layer=None, dim=None):
        blockx, blocky = getBlockSize(dim)
        self._take(src_mask=src_mask, ngh_mask=ngh_mask, backEdgeMask=backEdgeMask, node_degs=node_degs,
                   num_layers=num_layers, layer=layer, dim=dim, blockx=blockx, blocky=blocky)


class backInputProperty(_Record):
    """The compacted backward path of one layer, filled in after path preparation."""

    def __init__(self, id=None, partPointer=None, edgeList=None, degrees=None, partSize=None, numParts=None,
                 dim=None, layer=None):
        blockx, blocky = getBlockSize(dim)
        self._take(degrees=degrees, dim=dim, layer=layer, blockx=blockx, blocky=blocky)
        self.fillProperty(id, partPointer, edgeList, partSize, numParts)

    def fillProperty(self, id=None, partPointer=None, edgeList=None, partSize=None, numParts=None):
        self._take(id=id, partPointer=partPointer, edgeList=edgeList, partSize=partSize, numParts=numParts)
