"""Batch normalisation on the features of a SparseTensor (mirrors
minuet/nn/normalizations.py)."""
import torch

from minuet_amd.tensors import SparseTensor

__all__ = ["BatchNorm"]


class BatchNorm(torch.nn.BatchNorm1d):
    """:class:`torch.nn.BatchNorm1d` over the ``[N, C]`` feature tensor."""

    def forward(self, x: SparseTensor) -> SparseTensor:
        return SparseTensor.like(x, super().forward(x.F))
