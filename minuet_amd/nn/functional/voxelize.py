"""Input preparation next to the convolution path: points -> voxels, and a
batch of clouds -> one SparseTensor (the step before the first layer)."""
from typing import Optional, Sequence

import torch

from minuet_amd.utils.helpers import as_tuple
from . import _C
from .hash import unique_coordinates

__all__ = ["voxelize", "collate"]


def voxelize(coordinates: torch.Tensor, voxel_size=1, dtype: torch.dtype = torch.int32,
             return_reverse_indices: bool = False):
    """Voxel coordinates ``floor(p / voxel_size)`` of the points ``p``, sorted and
    without duplicates; with ``return_reverse_indices`` also the row of the
    result each input point fell into.

    Same interface as the reference's ``voxelize`` (voxelize.py:11-35), which
    cannot run as written: it builds the voxel-size tensor on
    ``device=coordinates.dtype`` and hands unsorted rows to
    ``unique_coordinates``, which only merges neighbouring duplicates.  Here
    the rows are sorted first, so every voxel appears once."""
    if not coordinates.is_cuda:
        raise NotImplementedError
    ndim = coordinates.shape[1]
    size = torch.tensor(as_tuple(voxel_size, size=ndim, name="voxel_size"), dtype=coordinates.dtype,
                        device=coordinates.device)
    voxels = torch.floor(coordinates / size).to(dtype).contiguous()
    order, ordered = _C.sort_coordinates(voxels)
    unique, index = unique_coordinates(ordered)
    if not return_reverse_indices:
        return unique
    # index[i] = number of runs of equal rows that end before ordered row i,
    # which is the row of the result that ordered row i is written to
    reverse = torch.empty(voxels.shape[0], dtype=torch.int64, device=voxels.device)
    reverse[order.long()] = index[:-1].long()
    return unique, reverse


def collate(coordinates: Sequence[torch.Tensor], features: Optional[Sequence[torch.Tensor]] = None):
    """One batch from several clouds of voxel coordinates (each free of
    duplicates, in any order): ``(coordinates, batch_dims)`` with every cloud
    sorted inside its ``[batch_dims[g], batch_dims[g + 1])`` range, the layout
    ``SparseTensor`` and the batched kernels expect (tensors.py:38-95); with
    ``features`` also the feature rows in the same order."""
    if len(coordinates) == 0:
        raise ValueError("collate needs at least one cloud")
    if features is not None and len(features) != len(coordinates):
        raise ValueError("features and coordinates must list the same clouds")
    stacked = torch.cat(list(coordinates), dim=0).contiguous()
    if not stacked.is_cuda:
        raise NotImplementedError
    counts = torch.tensor([0] + [int(c.shape[0]) for c in coordinates], dtype=torch.int64)
    batch_dims = torch.cumsum(counts, dim=0).to(dtype=stacked.dtype, device=stacked.device)
    order, ordered = _C.sort_coordinates(stacked, batch_dims)
    if features is None:
        return ordered, batch_dims
    return ordered, batch_dims, torch.cat(list(features), dim=0)[order.long()]
