"""Pointwise activations on the features of a SparseTensor (mirrors
minuet/nn/activations.py)."""
import torch

from minuet_amd.tensors import SparseTensor

__all__ = ["ReLU", "ReLU6", "LeakyReLU"]


def _on_features(base):
    def forward(self, x: SparseTensor) -> SparseTensor:
        return SparseTensor.like(x, base.forward(self, x.F))
    return forward


class ReLU(torch.nn.ReLU):
    """:class:`torch.nn.ReLU` applied to ``x.F``."""
    forward = _on_features(torch.nn.ReLU)


class ReLU6(torch.nn.ReLU6):
    """:class:`torch.nn.ReLU6` applied to ``x.F``."""
    forward = _on_features(torch.nn.ReLU6)


class LeakyReLU(torch.nn.LeakyReLU):
    """:class:`torch.nn.LeakyReLU` applied to ``x.F``."""
    forward = _on_features(torch.nn.LeakyReLU)
