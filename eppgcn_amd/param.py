"""Launch-parameter records the layer passes to the ops; the attribute names are the ones the
reference's autograd function reads (EPPGCN/gcn_conv.py:13-14,21-27,36-38; records defined in
EPPGCN/param.py).  The integers are hints sized for 32-lane warps: the HIP library picks its own
wave64 mapping from the feature width and only requires them to be positive, so they are kept
for signature compatibility and for reporting."""
from __future__ import annotations


def getBlockSize(dim):
    """(lanes per group, groups per block) for a feature width; always 64 threads, i.e. one
    wavefront (table of EPPGCN/param.py:6-24)."""
    if dim < 8:
        return 2, 32
    if dim < 32:
        return 4, 16
    if dim < 96:
        return 8, 8
    if dim < 192:
        return 16, 4
    return 32, 2


class inputProperty(object):
    """Forward-side inputs: CSR, scale vector, neighbour groups and launch hints."""

    MAX_warpPerBlock = 8
    gap_smem = 100

    def __init__(self, row_pointers=None, column_index=None, degrees=None, partSize=None, dimWorker=None,
                 warpPerBlock=None, sharedMem=None, hiddenDim=None, dataset_obj=None, manual_mode=True,
                 verbose=False):
        if dataset_obj is None:
            raise ValueError("Dataset object MUST SET !!!")
        self.dataset_obj = dataset_obj
        self.row_pointers = row_pointers
        self.column_index = column_index
        self.degrees = degrees
        self.num_nodes = dataset_obj.num_nodes
        self.avgNodeDegree = dataset_obj.avg_degree
        self.avgEdgeSpan = getattr(dataset_obj, "avg_edgeSpan", -1)
        self.partSize = partSize
        self.dimWorker = dimWorker
        self.warpPerBlock = warpPerBlock
        self.dimWorker_input = self.dimWorker_hidden = dimWorker
        self.warpPerBlock_input = self.warpPerBlock_hidden = warpPerBlock
        self.inputDim = dataset_obj.num_features
        self.hiddenDim = hiddenDim
        self.manual_mode = manual_mode
        self.verbose_flag = verbose
        self.state_set_input = False
        self.share_memory = (sharedMem if sharedMem is not None else 100) * 0.4
        self.partPtr = None
        self.part2Node = None

    def decider(self):
        """The reference's rule (EPPGCN/param.py:72-127): group size = int(average degree), warps per
        block from a shared-memory estimate capped at 8, dimension workers = min(width, 32).
        Unlike the reference, a manual group size is respected in manual mode and the automatic
        one never drops below 1 (an average degree below 1 would otherwise divide by zero in
        build_part)."""
        if not (self.manual_mode and self.partSize):
            self.partSize = max(1, int(self.avgNodeDegree))
        kb_in = self.MAX_warpPerBlock * (self.partSize * 4 + self.inputDim * 4 + self.gap_smem * 4) / 1e3
        kb_hid = self.MAX_warpPerBlock * (self.partSize * 4 + self.hiddenDim * 4 + self.gap_smem * 4) / 1e3
        kb_in, kb_hid = min(kb_in, self.share_memory), min(kb_hid, self.share_memory)
        self.warpPerBlock_input = max(1, min(int(kb_in * 1e3 / (self.partSize * 4 + self.inputDim * 4)),
                                             self.MAX_warpPerBlock))
        self.warpPerBlock_hidden = max(1, min(int(kb_hid * 1e3 / (self.partSize * 4 + self.hiddenDim * 4)),
                                              self.MAX_warpPerBlock))
        self.dimWorker_input = min(self.inputDim, 32)
        self.dimWorker_hidden = min(self.hiddenDim, 32)
        if self.verbose_flag:
            print("\n=> AUTO Decider Complete !!!\n")

    def set_input(self):
        self.dimWorker = self.dimWorker_input
        self.warpPerBlock = self.warpPerBlock_input
        self.state_set_input = True
        return self

    def set_hidden(self):
        self.dimWorker = self.dimWorker_hidden
        self.warpPerBlock = self.warpPerBlock_hidden
        self.state_set_input = False
        return self

    def print_param(self):
        if self.verbose_flag:
            mode = "manual" if self.manual_mode else "auto"
            which = "INPUT" if self.state_set_input else "HIDDEN"
            print("# {} {} partSize: {}".format(mode, which, self.partSize))
            print("# {} {} dimWorker: {}".format(mode, which, self.dimWorker))
            print("# {} {} warpPerBlock: {}".format(mode, which, self.warpPerBlock))


class maskInputProperty(object):
    """Inputs of one path-marking step (one per layer, first iteration only)."""

    def __init__(self, src_mask=None, ngh_mask=None, backEdgeMask=None, node_degs=None, num_layers=None,
                 layer=None, dim=None):
        self.src_mask = src_mask
        self.ngh_mask = ngh_mask
        self.backEdgeMask = backEdgeMask
        self.node_degs = node_degs
        self.num_layers = num_layers
        self.layer = layer
        self.blockx, self.blocky = getBlockSize(dim)
        self.dim = dim


class backInputProperty(object):
    """The compacted backward path of one layer, filled in after path preparation."""

    def __init__(self, id=None, partPointer=None, edgeList=None, degrees=None, partSize=None, numParts=None,
                 dim=None, layer=None):
        self.id = id
        self.partPointer = partPointer
        self.edgeList = edgeList
        self.degrees = degrees
        self.partSize = partSize
        self.numParts = numParts
        self.dim = dim
        self.layer = layer
        self.blockx, self.blocky = getBlockSize(dim)

    def fillProperty(self, id=None, partPointer=None, edgeList=None, partSize=None, numParts=None):
        self.id = id
        self.partPointer = partPointer
        self.edgeList = edgeList
        self.partSize = partSize
        self.numParts = numParts
