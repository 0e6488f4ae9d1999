"""Drop-in alias: ``import minuet`` resolves to the MI355X-native package, so
model code written against the reference's module paths (``minuet.nn``,
``minuet.nn.functional``, ``minuet.utils.helpers`` ...) runs unchanged."""
import importlib
import sys

import minuet_amd as _impl

_ALIASES = ["tensors", "utils", "utils.helpers", "utils.typing", "utils.random", "nn",
            "nn.functional", "nn.functional._C", "nn.functional.indexing", "nn.functional.hash",
            "nn.functional.scan", "nn.functional.convolution", "nn.functional.memory",
            "nn.functional.pooling", "nn.functional.concat", "nn.convolutions",
            "nn.activations", "nn.normalizations", "nn.pooling"]
for _name in _ALIASES:
    sys.modules[f"minuet.{_name}"] = importlib.import_module(f"minuet_amd.{_name}")

from minuet_amd import *  # noqa: E402,F401
from minuet_amd import (nn, utils, set_gemm_parallel_level, set_kernel_map_cache, autotune,  # noqa: E402,F401
                        load_tunable_config, dump_tunable_config)
