"""Duplicate removal on sorted coordinates (mirrors the conv-path half of
minuet/nn/functional/hash.py; ``simple_hash`` is not used by any convolution
path and is not provided)."""
from typing import Optional

import torch

from . import _C

__all__ = ["unique_coordinates"]


def unique_coordinates(coordinates: torch.Tensor, batch_dims: Optional[torch.Tensor] = None):
    """Drop duplicates from SORTED coordinates.  Returns ``(unique, index)`` where
    ``index[i]`` counts the unique rows before sorted position ``i`` (length
    N+1), so ``index[batch_dims]`` are the batch boundaries of the result
    (reference: hash.py:28-50)."""
    coordinates = coordinates.contiguous()
    if not coordinates.is_cuda:
        raise NotImplementedError
    if batch_dims is None:
        return _C.cuda_unique_coordinates(coordinates)
    return _C.cuda_multi_unique_coordinates(coordinates, batch_dims.contiguous())
