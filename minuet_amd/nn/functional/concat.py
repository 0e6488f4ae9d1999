"""Channel concatenation of SparseTensors that share coordinates (mirrors
minuet/nn/functional/concat.py)."""
from typing import Iterable

import torch

__all__ = ["cat"]


def cat(tensors: Iterable["SparseTensor"]):
    """Concatenate the features of tensors with identical coordinate tensors
    (not checked); coordinates, stride and batch_dims come from the first."""
    from minuet_amd.tensors import SparseTensor
    tensors = list(tensors)
    head = tensors[0]
    return SparseTensor(features=torch.cat([t.F for t in tensors], dim=1),
                        coordinates=head.C, stride=head.stride, batch_dims=head.batch_dims)
