"""The argument carrier that the conv modules read (the role of
YiTu_GNN/utils/input_info.py): the CSR, the per-node scale, the neighbour
partition and the three launch knobs of the reference's op signature, plus the
rule that picks those knobs and decides on reordering in automatic mode.

The gfx950 kernels choose their own row split, so the knobs do not steer them;
they are kept, and computed exactly as before, because callers set them, read
them back and pass them on.
"""
import math
from collections import namedtuple

MAX_WARPS_PER_BLOCK = 8
SHARED_MEMORY_SHARE = 0.4   # fraction of the device's shared memory the rule budgets
SMEM_GAP_WORDS = 100

AutoKnobs = namedtuple("AutoKnobs", "partSize warpPerBlock_input warpPerBlock_hidden "
                                    "dimWorker_input dimWorker_hidden")


def auto_knobs(avg_degree, input_dim, hidden_dim, shared_memory_kb) -> AutoKnobs:
    """The automatic choice of input_info.py:79-127. Groups are as wide as the
    average degree; a workgroup takes as many rows as fit the shared-memory budget
    (KB), at most eight; one lane per feature up to 32. The hidden-layer estimate
    adds ``hidden_dim`` bytes rather than words (input_info.py:93-97) and is kept so."""
    part = int(avg_degree)

    def warps(dim, estimate_bytes):
        budget_kb = min(MAX_WARPS_PER_BLOCK * estimate_bytes / 1e3, shared_memory_kb)
        return min(int(budget_kb * 1e3 / (4 * part + 4 * dim)), MAX_WARPS_PER_BLOCK)

    gap = 4 * SMEM_GAP_WORDS
    return AutoKnobs(part,
                     warps(input_dim, 4 * part + 4 * input_dim + gap),
                     warps(hidden_dim, 4 * part + hidden_dim + gap),
                     min(input_dim, 32), min(hidden_dim, 32))


def worth_reordering(avg_edge_span, num_nodes) -> bool:
    """input_info.py:131-136: reorder when neighbours are far apart in id space."""
    return math.sqrt(avg_edge_span) > math.sqrt(num_nodes) / 100


class InputInfo(object):
    # Replacing the column ids or the scale vector drops the per-edge scales derived from
    # them (prepare_edge_scale); writing INTO those tensors in place does not, and then
    # prepare_edge_scale has to be called again by whoever wrote.
    @property
    def column_index(self):
        return self._column_index

    @column_index.setter
    def column_index(self, value):
        self._column_index = value
        self.edge_scale = None

    @property
    def degrees(self):
        return self._degrees

    @degrees.setter
    def degrees(self, value):
        self._degrees = value
        self.edge_scale = None

    def __init__(self, row_pointers=None, column_index=None, degrees=None, partSize=None,
                 dimWorker=None, warpPerBlock=None, sharedMem=None, hiddenDim=None,
                 dataset_obj=None, enable_rabbit=False, manual_mode=True, verbose=False):
        if dataset_obj is None:
            raise ValueError("Dataset object MUST SET !!!")
        ds = self.dataset_obj = dataset_obj
        # graph
        self.row_pointers, self.column_index, self.degrees = row_pointers, column_index, degrees
        self.partPtr = self.part2Node = None
        self.num_nodes, self.avgNodeDegree, self.avgEdgeSpan = \
            ds.num_nodes, ds.avg_degree, ds.avg_edgeSpan
        self.inputDim, self.hiddenDim = ds.num_features, hiddenDim
        # knobs: the current pair, and the pairs for the input and the hidden layers
        self.partSize = partSize
        self.dimWorker = self.dimWorker_input = self.dimWorker_hidden = dimWorker
        self.warpPerBlock = self.warpPerBlock_input = self.warpPerBlock_hidden = warpPerBlock
        self.MAX_warpPerBlock = MAX_WARPS_PER_BLOCK
        self.share_memory = sharedMem * SHARED_MEMORY_SHARE
        self.gap_smem = SMEM_GAP_WORDS
        # mode and state
        self.manual_mode, self.enable_rabbit, self.verbose_flag = manual_mode, enable_rabbit, verbose
        self.state_set_input = False
        self.reorder_status = False
        # per-edge column scales for the GCN aggregation (see prepare_edge_scale); not in
        # the reference's carrier
        self.edge_scale = None

    def _reorder(self, wanted: bool):
        self.dataset_obj.reorder_flag = wanted
        self.reorder_status = wanted

    def decider(self):
        """Manual mode (input_info.py:65-77): the given knobs stand; the graph is
        reordered iff asked, and the carrier then takes the dataset's new CSR.
        Automatic mode (:78-143): knobs from ``auto_knobs``; with reordering enabled
        the dataset's ``rabbit_reorder`` is always called and acts iff
        ``worth_reordering`` set its flag."""
        if self.manual_mode:
            self._reorder(bool(self.enable_rabbit))
            if self.enable_rabbit:
                self.dataset_obj.rabbit_reorder()
                self.row_pointers = self.dataset_obj.row_pointers
                self.column_index = self.dataset_obj.column_index
            return
        (self.partSize, self.warpPerBlock_input, self.warpPerBlock_hidden, self.dimWorker_input,
         self.dimWorker_hidden) = auto_knobs(self.avgNodeDegree, self.inputDim, self.hiddenDim,
                                             self.share_memory)
        if self.enable_rabbit:
            self._reorder(worth_reordering(self.avgEdgeSpan, self.num_nodes))
            self.dataset_obj.rabbit_reorder()

    def prepare_edge_scale(self):
        """Per-graph preparation for the GCN layers: ``edge_scale[e] = degrees[column_index[e]]``
        (YiTu_GNN_kernel.edge_scale), so the aggregation reads the column scale of an edge
        in edge order instead of gathering ``degrees``. Call after ``decider`` (a reorder
        replaces the CSR) and again whenever ``column_index`` or ``degrees`` are replaced;
        setting ``self.edge_scale = None`` returns to the reference's form. Returns self."""
        from .. import YiTu_GNN_kernel
        self.edge_scale = YiTu_GNN_kernel.edge_scale(self.column_index, self.degrees)
        return self

    def _select(self, for_input: bool):
        suffix = "_input" if for_input else "_hidden"
        self.dimWorker = getattr(self, "dimWorker" + suffix)
        self.warpPerBlock = getattr(self, "warpPerBlock" + suffix)
        self.state_set_input = for_input
        return self

    def set_input(self):
        """Knobs of the first layer (width = input features); returns self."""
        return self._select(True)

    def set_hidden(self):
        """Knobs of the later layers (width = hidden features); returns self."""
        return self._select(False)

    def print_param(self):
        if not self.verbose_flag:
            return
        where = "%s %s" % ("manual" if self.manual_mode else "auto",
                           "INPUT" if self.state_set_input else "HIDDEN")
        for knob in ("partSize", "dimWorker", "warpPerBlock"):
            print("# %s %s: %s" % (where, knob, getattr(self, knob)))
        if not self.manual_mode:
            print("# %s reorder_flag: %s" % (where, self.reorder_status))
