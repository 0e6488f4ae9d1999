"""Batch normalisation on the features of a SparseTensor (mirrors
minuet/nn/normalizations.py)."""
import torch

from minuet_amd.tensors import SparseTensor

__all__ = ["BatchNorm"]


class BatchNorm(torch.nn.BatchNorm1d):
    """:class:`torch.nn.BatchNorm1d` over the ``[N, C]`` feature tensor."""

    def invalidate_cached_weights(self):
        """Drops the per-channel scale / shift that fused inference passes keep
        for this module (see ``SparseConv.invalidate_cached_weights``: needed
        after writes through ``.data`` only)."""
        self.__dict__.pop("_minuet_affine", None)

    def reset_parameters(self):
        super().reset_parameters()
        self.invalidate_cached_weights()

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)
        self.invalidate_cached_weights()

    def _apply(self, fn, *args, **kwargs):
        result = super()._apply(fn, *args, **kwargs)
        self.invalidate_cached_weights()
        return result

    def forward(self, x: SparseTensor) -> SparseTensor:
        return SparseTensor.like(x, super().forward(x.F))
