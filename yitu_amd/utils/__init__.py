"""Per-graph bookkeeping of the GCN / GIN layers (``input_info.InputInfo``)."""
