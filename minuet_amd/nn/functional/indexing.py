"""Coordinate sorting and kernel-map queries (mirrors
minuet/nn/functional/indexing.py of the reference)."""
from typing import Optional

import torch

from . import _C

__all__ = ["arg_sort_coordinates", "build_sorted_index", "query_sorted_index_with_offsets"]


def arg_sort_coordinates(coordinates: torch.Tensor,
                         batch_dims: Optional[torch.Tensor] = None,
                         dtype: Optional[torch.dtype] = None,
                         enable_flattening: bool = True) -> torch.Tensor:
    """Order that sorts ``coordinates`` lexicographically (dimension 0 most
    significant); with ``batch_dims`` every point cloud is sorted on its own and
    the clouds stay in batch order.  Equal rows keep their input order.

    ``enable_flattening`` is accepted for compatibility: keys are always packed
    when they fit 64 bits, and multi-round sorting takes over when they do not
    (reference: minuet/nn/functional/indexing.py:14-56)."""
    coordinates = coordinates.contiguous()
    if not coordinates.is_cuda:
        raise NotImplementedError
    if batch_dims is not None:
        index = _C.cuda_multi_arg_sort_coordinates(coordinates, batch_dims.contiguous(),
                                                   enable_flattening)
    else:
        index = _C.cuda_arg_sort_coordinates(coordinates, enable_flattening)
    return index if dtype is None else index.to(dtype=dtype)


def build_sorted_index(coordinates: torch.Tensor,
                       batch_dims: Optional[torch.Tensor] = None,
                       enable_flattening: bool = True) -> torch.Tensor:
    """``arg_sort_coordinates`` as int64, ready for tensor indexing
    (reference: indexing.py:59-79)."""
    return arg_sort_coordinates(coordinates, batch_dims=batch_dims, dtype=torch.int64,
                                enable_flattening=enable_flattening)


def query_sorted_index_with_offsets(sources: torch.Tensor,
                                    targets: torch.Tensor,
                                    offsets: torch.Tensor,
                                    source_batch_dims: Optional[torch.Tensor] = None,
                                    target_batch_dims: Optional[torch.Tensor] = None
                                    ) -> torch.Tensor:
    """Dense kernel map ``[N_weight, N_out]``: entry ``(o, t)`` is the index of
    the source equal to ``targets[t] + offsets[o]`` or -1.  ``sources`` and
    ``targets`` must be sorted (reference: indexing.py:82-127)."""
    if (source_batch_dims is None) != (target_batch_dims is None):
        raise ValueError("source_batch_dims and target_batch_dims must be both "
                         "provided or neither provided")
    sources, targets, offsets = sources.contiguous(), targets.contiguous(), offsets.contiguous()
    if not offsets.is_cuda:
        raise NotImplementedError
    if source_batch_dims is not None:
        return _C.cuda_multi_query_sorted_index_with_offsets(
            source_batch_dims.contiguous(), target_batch_dims.contiguous(), sources, targets,
            offsets)
    return _C.cuda_query_sorted_index_with_offsets(sources, targets, offsets)
