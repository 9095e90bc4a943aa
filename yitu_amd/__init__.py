"""MI355X-native sparse message passing behind YiTu's operator interfaces.

Sub-packages are imported on use: ``YiTu_GNN_kernel`` and ``nn`` (GCN / GIN
aggregation), ``graph_ext`` and ``xgnn_h`` (multi-head SpMM, SDDMM, fused GAT,
typed GEMMs, the capture / lower / stitch / execute pipeline), ``rabbit``
(vertex reordering), ``sampler_core`` and ``temporal`` (recent-neighbour sampling
and temporal attention). Everything computes through ``libyitu_hip.so``; there
is no CPU path."""
