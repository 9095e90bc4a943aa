"""Parameter carrier consumed by the conv modules (YiTu_GNN/utils/input_info.py).

Holds the CSR, the per-node scale, the neighbour-group partition and the three
tuning knobs of the reference signature. The knobs are kept because callers set
and read them; the gfx950 kernels pick their own row split and ignore them.
"""
import math


class InputInfo(object):
    def __init__(self, row_pointers=None, column_index=None, degrees=None, partSize=None,
                 dimWorker=None, warpPerBlock=None, sharedMem=None, hiddenDim=None,
                 dataset_obj=None, enable_rabbit=False, manual_mode=True, verbose=False):
        if dataset_obj is None:
            raise ValueError("Dataset object MUST SET !!!")
        self.dataset_obj = dataset_obj
        self.row_pointers = row_pointers
        self.column_index = column_index
        self.degrees = degrees
        self.num_nodes = dataset_obj.num_nodes
        self.avgNodeDegree = dataset_obj.avg_degree
        self.avgEdgeSpan = dataset_obj.avg_edgeSpan
        self.partSize = partSize
        self.dimWorker = dimWorker
        self.warpPerBlock = warpPerBlock
        self.dimWorker_input = dimWorker
        self.dimWorker_hidden = dimWorker
        self.warpPerBlock_input = warpPerBlock
        self.warpPerBlock_hidden = warpPerBlock
        self.inputDim = dataset_obj.num_features
        self.hiddenDim = hiddenDim
        self.manual_mode = manual_mode
        self.enable_rabbit = enable_rabbit
        self.verbose_flag = verbose
        self.state_set_input = False
        self.reorder_status = False
        self.MAX_warpPerBlock = 8
        self.share_memory = sharedMem * 0.4
        self.gap_smem = 100
        self.partPtr = None
        self.part2Node = None

    def decider(self):
        """Manual mode keeps the given knobs and reorders iff asked; auto mode
        derives them from the average degree and feature widths and reorders iff
        sqrt(avgEdgeSpan) > sqrt(N) / 100 (input_info.py:58-143)."""
        if self.manual_mode:
            if self.enable_rabbit:
                self.dataset_obj.reorder_flag = True
                self.dataset_obj.rabbit_reorder()
                self.reorder_status = True
                self.row_pointers = self.dataset_obj.row_pointers
                self.column_index = self.dataset_obj.column_index
            else:
                self.dataset_obj.reorder_flag = False
                self.reorder_status = False
            return
        self.partSize = int(self.avgNodeDegree)
        est = self.MAX_warpPerBlock * (self.partSize * 4 + self.inputDim * 4 + self.gap_smem * 4) / 1e3
        share_memory_input = min(est, self.share_memory)
        # the hidden-layer estimate really adds hiddenDim unscaled (input_info.py:93-97)
        est = self.MAX_warpPerBlock * (self.partSize * 4 + self.hiddenDim + 4 * self.gap_smem) / 1e3
        share_memory_hidden = min(est, self.share_memory)
        self.warpPerBlock_input = min(
            int(share_memory_input * 1e3 / (self.partSize * 4 + self.inputDim * 4)),
            self.MAX_warpPerBlock)
        self.warpPerBlock_hidden = min(
            int(share_memory_hidden * 1e3 / (self.partSize * 4 + self.hiddenDim * 4)),
            self.MAX_warpPerBlock)
        self.dimWorker_input = 32 if self.inputDim > 32 else self.inputDim
        self.dimWorker_hidden = 32 if self.hiddenDim > 32 else self.hiddenDim
        if self.enable_rabbit:
            reorder = math.sqrt(self.avgEdgeSpan) > math.sqrt(self.num_nodes) / 100
            self.dataset_obj.reorder_flag = reorder
            self.reorder_status = reorder
            self.dataset_obj.rabbit_reorder()

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
        if not self.verbose_flag:
            return
        mode = "manual" if self.manual_mode else "auto"
        layer = "INPUT" if self.state_set_input else "HIDDEN"
        print("# {} {} partSize: {}".format(mode, layer, self.partSize))
        print("# {} {} dimWorker: {}".format(mode, layer, self.dimWorker))
        print("# {} {} warpPerBlock: {}".format(mode, layer, self.warpPerBlock))
        if not self.manual_mode:
            print("# {} {} reorder_flag: {}".format(mode, layer, self.reorder_status))
