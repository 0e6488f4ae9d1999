"""Host-side helpers: kernel offsets, tuple normalisation, cache wiring and
the autotune / tunable-config drivers (mirrors minuet/utils/helpers.py)."""
import contextlib
import json
import os
from typing import Iterable, Optional

import numpy as np
from torch.nn import Module

__all__ = ["as_tuple", "generate_kernel_offsets", "set_kernel_map_cache",
           "dump_tunable_config", "load_tunable_config", "autotune", "invalidate_cached_weights"]


def as_tuple(value, *, size: int = 3, name: Optional[str] = None):
    """A scalar becomes a ``size``-tuple of itself; an iterable must already have
    ``size`` elements (reference: helpers.py:138-162)."""
    if type(value) is tuple and len(value) == size:
        return value
    if isinstance(value, (int, float)) or not isinstance(value, Iterable):
        return tuple(value for _ in range(size))
    value = tuple(value)
    if len(value) != size:
        raise ValueError(f"{name or 'Value'} must be a scalar or a iterable of size {size} but "
                         f"found {len(value)} elements")
    return value


def generate_kernel_offsets(ndim: int, kernel_size, source_stride, dilation,
                            layout: str = "minuet") -> np.ndarray:
    """Weight offsets ``[K^D, D]`` of a sparse convolution.  An odd extent ``k``
    spans ``-k//2 .. k//2`` and an even one ``-k/2+1 .. k/2``; the "minuet"
    layout enumerates dimension 0 slowest, "minkowski" reverses that order and
    "torchsparse" reverses it for odd kernel volumes only.  Offsets are scaled
    by ``source_stride * dilation`` (reference: helpers.py:165-212)."""
    kernel_size = as_tuple(kernel_size, size=ndim, name="kernel_size")
    source_stride = as_tuple(source_stride, size=ndim, name="source_stride")
    dilation = as_tuple(dilation, size=ndim, name="dilation")
    if layout not in ("minuet", "torchsparse", "minkowski"):
        raise NotImplementedError
    axes = [np.arange(-(k // 2) + (1 - k % 2), k // 2 + 1) for k in kernel_size]
    grid = np.stack(np.meshgrid(*axes, copy=False, indexing="ij"), axis=ndim)
    reverse = layout == "minkowski" or (layout == "torchsparse" and np.prod(kernel_size) % 2 == 1)
    if reverse:
        grid = np.transpose(grid, axes=list(range(ndim - 1, -1, -1)) + [ndim])
    offsets = np.reshape(grid, (-1, ndim))
    return offsets * np.asarray(source_stride) * np.asarray(dilation)


def set_kernel_map_cache(module: Module, cache):
    """Attach ``cache`` to every layer below ``module`` that accepts one
    (reference: helpers.py:29-46)."""
    if hasattr(module, "set_kernel_map_cache"):
        module.set_kernel_map_cache(cache)
    for child in module.children():
        set_kernel_map_cache(child, cache=cache)
    return module


def invalidate_cached_weights(module: Module):
    """Drops every derived copy of parameters that inference passes keep below
    ``module``: packed convolution kernels and the per-channel scale / shift of
    folded BatchNorm layers.  Those copies follow the parameters by storage and
    version counter, which writes through ``.data`` do not bump; call this
    after such writes (no counterpart in the reference, which repacks its
    weights in every forward, csrc/minuet/cuda/functions/sparse_convolution.cu:526-553)."""
    for child in module.modules():
        drop = getattr(child, "invalidate_cached_weights", None)
        if callable(drop):
            drop()
        else:
            child.__dict__.pop("_minuet_affine", None)


def _ensure_directory(path: str):
    if not path:
        return path
    if not os.path.exists(path):
        os.makedirs(path)
    elif not os.path.isdir(path):
        raise RuntimeError(f"Path {path} is not a directory")
    return path


def autotune(model: Module, model_cache, data, cache_path: Optional[str] = None):
    """Tune every tunable layer of ``model`` on the given sample tensors, or load
    the result from ``cache_path`` when that file exists; a fresh result is
    written there (reference: helpers.py:49-94)."""
    from minuet_amd.tensors import SparseTensor
    if isinstance(data, SparseTensor):
        data = [data]
    if cache_path is not None and os.path.exists(cache_path):
        with open(cache_path) as reader:
            return load_tunable_config(model, config=json.load(reader))
    with contextlib.ExitStack() as stack:
        def enter(module: Module):
            if hasattr(module, "autotune"):
                stack.enter_context(module.autotune())
            for child in module.children():
                enter(child)

        enter(model)
        for tensor in data:
            model_cache.reset()
            model(tensor)
    if cache_path is not None:
        _ensure_directory(os.path.dirname(cache_path))
        with open(cache_path, "w") as writer:
            json.dump(dump_tunable_config(model), writer, indent=2)
    return model


def load_tunable_config(module: Module, config: dict):
    """Apply a nested config dict, keyed by child-module names, to ``module``
    (reference: helpers.py:97-115)."""
    if hasattr(module, "tunable_config"):
        module.tunable_config.update(config)
    for name, child in module.named_children():
        load_tunable_config(child, config=config[name])
    return module


def dump_tunable_config(module: Module) -> dict:
    """Nested dict of the tunable configs below ``module``
    (reference: helpers.py:118-135)."""
    if hasattr(module, "tunable_config"):
        return module.tunable_config
    return {name: dump_tunable_config(child) for name, child in module.named_children()}
