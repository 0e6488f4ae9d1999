"""``SparseTensor``: features plus sorted, unique integer coordinates (mirrors
minuet/tensors.py of the reference)."""
from typing import Optional

import torch

from minuet_amd.utils.helpers import as_tuple

__all__ = ["SparseTensor"]


def _validate(features: torch.Tensor, coordinates: torch.Tensor):
    if coordinates.ndim != 2:
        raise ValueError(f"The coordinates tensor must be a 2-D tensor but found "
                         f"{coordinates.ndim}-D")
    if coordinates.shape[0] != features.shape[0]:
        raise ValueError(f"The features tensor indicate {features.shape[0]} coordinates but "
                         f"expected {coordinates.shape[0]} coordinates")
    if coordinates.device != features.device:
        raise ValueError(f"The features tensor is expected to be on the same device as the "
                         f"coordinates tensor {coordinates.device} but found {features.device}")
    if coordinates.requires_grad:
        raise ValueError("The coordinates tensor should never requires gradients")
    if coordinates.dtype not in (torch.int32, torch.int64):
        raise ValueError(f"The coordinates tensor must be int32 or int64 but found "
                         f"{coordinates.dtype}")


class SparseTensor(object):
    """A batch of point clouds: ``F`` is ``[N, C]`` features, ``C`` is ``[N, D]``
    int32/int64 coordinates that are sorted and unique inside every cloud, and
    ``batch_dims`` (``[B+1]`` prefix offsets, or ``None`` for a single cloud)
    says which rows belong to which cloud.  ``stride`` is the tensor stride of
    the coordinates.  A ``batch_dims`` with at most two entries describes a
    single cloud and is dropped (reference: minuet/tensors.py:64-79)."""

    def __init__(self, features: torch.Tensor, coordinates: torch.Tensor, *,
                 stride=1, batch_dims: Optional[torch.Tensor] = None):
        _validate(features, coordinates)
        self._features = features
        self._coordinates = coordinates
        self._stride = as_tuple(stride, size=self.ndim, name="strides")
        self._batch_dims = batch_dims if batch_dims is not None and len(batch_dims) > 2 else None

    @classmethod
    def like(cls, other: "SparseTensor", features: torch.Tensor, coordinates=None, stride=None,
             batch_dims=None) -> "SparseTensor":
        """New tensor that takes from ``other`` whatever is not given.  For the
        layers of this package, whose outputs are consistent by construction:
        nothing is validated again."""
        new = cls.__new__(cls)
        new._features = features
        new._coordinates = other._coordinates if coordinates is None else coordinates
        new._stride = other._stride if stride is None else stride
        new._batch_dims = other._batch_dims if coordinates is None else batch_dims
        return new

    # ---- shape-like properties -------------------------------------------
    @property
    def F(self) -> torch.Tensor:
        return self._features

    @F.setter
    def F(self, features: torch.Tensor):
        if features.device != self._features.device:
            raise ValueError(f"The new features is on the device {features.device} which is "
                             f"different from expected {self._features.device}")
        if features.shape != self._features.shape:
            raise ValueError(f"The new features has shape {features.shape} which is different "
                             f"from expected {self._features.shape}")
        self._features = features

    @property
    def C(self) -> torch.Tensor:
        return self._coordinates

    @property
    def batch_dims(self) -> Optional[torch.Tensor]:
        return self._batch_dims

    @property
    def batch_size(self) -> int:
        return 1 if self._batch_dims is None else len(self._batch_dims) - 1

    @property
    def stride(self):
        return self._stride

    @property
    def device(self):
        return self._coordinates.device

    @property
    def dtype(self):
        return self._features.dtype

    @property
    def shape(self):
        return self._features.shape

    @property
    def num_features(self) -> int:
        return self._features.shape[1]

    @property
    def ndim(self) -> int:
        return self._coordinates.shape[1]

    @property
    def n(self) -> int:
        return self._coordinates.shape[0]

    # ---- tensor-like methods ---------------------------------------------
    def _rewrap(self, features, coordinates=None, batch_dims="same"):
        return SparseTensor(features,
                            self._coordinates if coordinates is None else coordinates,
                            stride=self._stride,
                            batch_dims=self._batch_dims if batch_dims == "same" else batch_dims)

    def clone(self):
        bd = None if self._batch_dims is None else self._batch_dims.clone()
        return self._rewrap(self._features.clone(), self._coordinates.clone(), bd)

    def to(self, device=None, dtype=None, non_blocking: bool = False, copy: bool = False):
        """Move everything to ``device``; ``dtype`` applies to the features only.
        With ``copy`` a new SparseTensor is returned, otherwise this one is
        updated in place and returned."""
        kwargs = {"device": device, "non_blocking": non_blocking, "copy": copy}
        coordinates = self._coordinates.to(**kwargs)
        features = self._features.to(**kwargs, dtype=dtype)
        batch_dims = None if self._batch_dims is None else self._batch_dims.to(**kwargs)
        if copy:
            return self._rewrap(features, coordinates, batch_dims)
        self._coordinates, self._features, self._batch_dims = coordinates, features, batch_dims
        return self

    def cuda(self, device=None, non_blocking: bool = False):
        kwargs = {"device": device, "non_blocking": non_blocking}
        self._coordinates = self._coordinates.cuda(**kwargs)
        self._features = self._features.cuda(**kwargs)
        if self._batch_dims is not None:
            self._batch_dims = self._batch_dims.cuda(**kwargs)
        return self

    def cpu(self):
        self._coordinates = self._coordinates.cpu()
        self._features = self._features.cpu()
        if self._batch_dims is not None:
            self._batch_dims = self._batch_dims.cpu()
        return self

    def contiguous(self):
        self._coordinates = self._coordinates.contiguous()
        self._features = self._features.contiguous()
        if self._batch_dims is not None:
            self._batch_dims = self._batch_dims.contiguous()
        return self

    def detach(self):
        return self._rewrap(self._features.detach())

    def detach_(self):
        self._features = self._features.detach_()
        return self

    def half(self):
        return self._rewrap(self._features.half())

    def backward(self, **kwargs):
        return self._features.backward(**kwargs)

    @property
    def requires_grad(self) -> bool:
        return self._features.requires_grad

    @requires_grad.setter
    def requires_grad(self, value: bool):
        self._features.requires_grad = value

    def __repr__(self):
        return (f"SparseTensor(n={self.n}, channels={self.num_features}, stride={self._stride}, "
                f"batch_size={self.batch_size}, dtype={self.dtype}, device={self.device})")
