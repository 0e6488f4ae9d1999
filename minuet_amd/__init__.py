"""MI355X-native sparse convolution with Minuet's Python API.

``import minuet_amd as minuet`` (or the ``minuet`` alias package shipped next to
it) gives ``SparseTensor``, ``nn.SparseConv3d`` / ``nn.SparseConv``,
``nn.KernelMapCache`` and the helpers of the reference's top-level namespace
(minuet/__init__.py:1-8)."""
from .tensors import *
from . import utils
from . import nn
from .nn.functional.convolution import set_gemm_parallel_level
from .utils.helpers import set_kernel_map_cache
from .utils.helpers import autotune
from .utils.helpers import load_tunable_config
from .utils.helpers import dump_tunable_config
from .utils.graphs import capture_forward
from .utils.helpers import invalidate_cached_weights
