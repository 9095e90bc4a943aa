"""Temporal neighbour attention (YiTu_GNN/YiTu_T/layers.py) over the HIP ops."""
from .layers import TemporalBlock, TimeEncode, TransfomerAttentionLayer  # noqa: F401
from .tcsr import build_tcsr  # noqa: F401
