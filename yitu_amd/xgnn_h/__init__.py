"""Host-side mirror of the reference's ``xgnn_h`` package
(YiTu_GNN/YiTu_H/xgnn_h): the op wrappers over the HIP kernels
(``sparse``, ``bundle``, ``block``, ``convert``) and the capture -> lower ->
stitch -> execute pipeline (``mp``, ``trace``, ``ir``, ``ast``, ``optimizer``,
``stitcher``, ``executor``, ``printer``) with the reference's entry points."""
from . import block, bundle, convert, ir, layers, models, mp, sparse  # noqa: F401
from .ast import Module2IR  # noqa: F401
from .block import Block  # noqa: F401
from .executor import Executor  # noqa: F401
from .optimizer import Optimizer  # noqa: F401
from .printer import Printer  # noqa: F401
from .stitcher import Stitcher  # noqa: F401
