"""``KernelMap``: everything the library knows about one kernel map.

The reference hands a layer's kernel map around as the 4-tuple
``(source_masks, target_masks, kernel_map_order, kernel_map_sizes)``
(minuet/nn/convolutions.py:165-173) and reads the sizes back from the device
in every forward (csrc/minuet/cuda/functions/sparse_convolution.cu:555-557).
A ``KernelMap`` IS that tuple (it unpacks and indexes like it, so code
written against the reference keeps working) and additionally carries what
makes the forward pass wait for nothing: host copies of sizes and order, the
per-offset pair lists, the dense map of the single-kernel dataflow and the
target-major row lists of the list-driven Scatter."""
from typing import Optional

import numpy as np
import torch

__all__ = ["KernelMap"]


class KernelMap(tuple):
    """``(source_masks, target_masks, kernel_map_order, kernel_map_sizes)`` plus:

    * ``sizes_host`` / ``order_host``: int64 numpy copies of sizes and order
      (``order_host`` is None when the rows are in offset order);
    * ``in_idx`` / ``out_idx``: int32 ``[nnz]`` pair lists, rows in the order
      of ``kernel_map_order``, hits in target order: the source row and the
      target row of every buffer row;
    * ``dense``: int32 ``[O, T]`` source row per (offset, target) in the
      ORIGINAL offset order (-1: none), what the single-kernel forward walks;
    * ``row_ptr`` / ``out_pos``: int32 ``[T + 1]`` and ``[nnz]``: target ``t``
      sums the buffer rows ``row_ptr[t] .. row_ptr[t + 1] - 1`` and the product
      of list entry ``p`` is written to buffer row ``out_pos[p]`` (the
      target-major layout of the list-driven Gather-GEMM-Scatter);
    * ``num_sources`` / ``num_targets`` / ``num_offsets`` / ``nnz``.

    Any of the tensors may be None when that form of the map was not built."""

    def __new__(cls, source_masks: Optional[torch.Tensor], target_masks: Optional[torch.Tensor],
                kernel_map_order: Optional[torch.Tensor], kernel_map_sizes: Optional[torch.Tensor],
                sizes_host=None, order_host=None, in_idx: Optional[torch.Tensor] = None,
                out_idx: Optional[torch.Tensor] = None, dense: Optional[torch.Tensor] = None,
                row_ptr: Optional[torch.Tensor] = None, out_pos: Optional[torch.Tensor] = None,
                num_sources: Optional[int] = None, num_targets: Optional[int] = None):
        self = super().__new__(cls, (source_masks, target_masks, kernel_map_order, kernel_map_sizes))
        self.sizes_host = None if sizes_host is None else np.ascontiguousarray(sizes_host, dtype=np.int64)
        self.order_host = None if order_host is None else np.ascontiguousarray(order_host, dtype=np.int64)
        self.in_idx, self.out_idx, self.dense = in_idx, out_idx, dense
        self.row_ptr, self.out_pos = row_ptr, out_pos
        if num_sources is None and source_masks is not None:
            num_sources = source_masks.shape[1]
        if num_targets is None:
            num_targets = (target_masks.shape[1] if target_masks is not None
                           else dense.shape[1] if dense is not None else None)
        self.num_sources, self.num_targets = num_sources, num_targets
        self.inverse_dense = None           # dense map of the transposed direction, made on first use
        self.prepared = None                # the forward call's view of this map, worked out on first use
        return self

    source_masks = property(lambda self: self[0])
    target_masks = property(lambda self: self[1])
    kernel_map_order = property(lambda self: self[2])
    kernel_map_sizes = property(lambda self: self[3])

    @property
    def num_offsets(self) -> int:
        for tensor in (self[3], self[1], self.dense):
            if tensor is not None:
                return int(tensor.shape[0])
        return 0 if self.sizes_host is None else int(self.sizes_host.shape[0])

    @property
    def nnz(self) -> Optional[int]:
        return None if self.sizes_host is None else int(self.sizes_host.sum())

    def ensure_row_lists(self) -> bool:
        """Builds ``row_ptr`` / ``out_pos`` (the target-major row lists of the
        list-driven dataflow) if they are missing; needs the dense map, the pair
        lists and the host sizes, at most 1024 offsets.  Waits for nothing on
        the device.  Returns whether the map has them afterwards."""
        if self.row_ptr is not None:
            return True
        from minuet_amd.nn.functional import _C
        if (self.dense is None or self.in_idx is None or self.sizes_host is None or not self.dense.is_cuda
                or not 0 < self.num_offsets <= _C.MAX_ROW_LIST_OFFSETS):
            return False
        self.row_ptr, self.out_pos = _C.kernel_map_row_lists(self.dense, self.sizes_host, self.order_host)
        return True

    def swapped(self, dense: Optional[torch.Tensor] = None) -> "KernelMap":
        """The same map read the other way round, as a transposed layer uses it
        (minuet/nn/convolutions.py:135-140 swaps the two rank tables): sources
        and targets change roles, ``dense`` is the inverse dense map."""
        return KernelMap(self[1], self[0], self[2], self[3], sizes_host=self.sizes_host,
                         order_host=self.order_host, in_idx=self.out_idx, out_idx=self.in_idx,
                         dense=dense, num_sources=self.num_targets, num_targets=self.num_sources)

    def with_tables(self, source_masks: torch.Tensor, target_masks: torch.Tensor) -> "KernelMap":
        """A copy whose rank tables are the given tensors (clones, casts, tensors
        moved between streams ...); everything else is shared."""
        other = KernelMap(source_masks, target_masks, self[2], self[3], sizes_host=self.sizes_host,
                          order_host=self.order_host, in_idx=self.in_idx, out_idx=self.out_idx,
                          dense=self.dense, row_ptr=self.row_ptr, out_pos=self.out_pos,
                          num_sources=self.num_sources, num_targets=self.num_targets)
        other.inverse_dense = self.inverse_dense
        return other

    def __repr__(self) -> str:
        have = [name for name in ("source_masks", "target_masks", "in_idx", "dense", "row_ptr")
                if getattr(self, name) is not None]
        return (f"KernelMap(offsets={self.num_offsets}, sources={self.num_sources}, "
                f"targets={self.num_targets}, nnz={self.nnz}, forms={have})")
