"""Host-side mirror of the reference's ``xgnn_h`` op wrappers
(YiTu_GNN/YiTu_H/xgnn_h/{sparse,bundle,block,convert}.py) over the HIP ops."""
from . import block, bundle, convert, layers, sparse  # noqa: F401
