"""Building a pass's coordinate levels and kernel maps ahead of its layers.

A network asks its :class:`~minuet_amd.nn.KernelMapCache` for the same levels
and maps, in the same order, for every cloud.  With ``lookahead=True`` the
cache remembers those requests and, at the first request of the next pass,
hands all of them to the library's worker thread (``mnt_lookahead_start``),
which builds them for the new cloud on a stream of its own while the Python
thread goes on enqueueing layers; a request that the worker was given is then
served by waiting for its item.  The reference builds every map at the first
layer that needs it (minuet/nn/convolutions.py:58-173); the results here are
those of the same library calls, only made earlier and elsewhere.

Outputs live in one allocation sized for the worst case (no level has more
rows than the input cloud); the tensors handed out are views of it."""
import weakref
from typing import Dict, Optional

import numpy as np
import torch

from minuet_amd.nn.functional import _C

__all__ = ["AheadLayout", "AheadSession", "end_running_session"]

# The session the library's worker is running for (a weak reference): a session
# object that is no longer this one neither takes items nor ends anything.
_running = None


def end_running_session(device: torch.device):
    """Ends whatever session the worker is running; the cache that started it
    builds the rest of its pass the ordinary way."""
    global _running
    _running = None
    _C.lookahead_finish(device)


_ALIGN = 256
_ROW_STEP = 1 << 14          # layouts are made for row counts rounded up to this


class AheadLayout:
    """Where every output of a recipe goes inside one allocation, and the item
    list that tells the library so: worked out once per (recipe, cloud shape)
    and reused by the sessions of later passes.

    ``recipe`` is a sequence of ``("coords", source_stride, target_stride)``,
    ``("dense", key)``, ``("tables", key, reorder)`` and ``("invert", key)``
    entries in the order a pass made them, ``key`` being the cache's
    ``(source_stride, target_stride, kernel_size, kernel_dilation)``.  Raises
    ``ValueError`` when the recipe cannot be run from ``stride`` (an entry that
    needs a level or a map no earlier entry makes)."""

    def __init__(self, recipe, offsets_of, stride, capacity: int, ndim: int, coord_dtype: torch.dtype,
                 index_dtype: Optional[torch.dtype], num_batches: int):
        self.signature = (recipe, tuple(stride), capacity, ndim, coord_dtype, index_dtype, num_batches)
        self.capacity, self.ndim = capacity, ndim
        self.coord_dtype, self.index_dtype, self.num_batches = coord_dtype, index_dtype, num_batches
        n = capacity
        levels = {tuple(stride): 0}
        dense_of: Dict[tuple, int] = {}
        plan = []                         # per item: (tag, kind, fields, byte sizes of out0..out5)
        for entry in recipe:
            what = entry[0]
            if what == "coords":
                _, source, target = entry
                if source not in levels or target in levels:
                    raise ValueError(f"level {target} cannot be built from {source} here")
                levels[target] = len(levels)
                sizes = [n * ndim * coord_dtype.itemsize,
                         (num_batches + 1) * index_dtype.itemsize if index_dtype is not None else 0]
                plan.append((("coords", target), _C.AHEAD_COORDS,
                             dict(source_level=levels[source], target_level=levels[target], stride=target,
                                  capacity=n), sizes))
            elif what == "dense":
                key = entry[1]
                source, target, kernel_size, dilation = key
                if source not in levels or target not in levels or key in dense_of:
                    raise ValueError(f"map {key} cannot be built here")
                offsets = offsets_of(source, kernel_size, dilation)
                dense_of[key] = len(plan)
                plan.append((("dense", key), _C.AHEAD_DENSE,
                             dict(source_level=levels[source], target_level=levels[target], offsets=offsets,
                                  num_offsets=offsets.shape[0], capacity=offsets.shape[0] * n),
                             [offsets.shape[0] * n * 4]))
            elif what == "tables":
                _, key, reorder = entry
                if key not in dense_of:
                    raise ValueError(f"tables of {key} need its dense map first")
                num_offsets = plan[dense_of[key]][2]["num_offsets"]
                full = num_offsets * n * 4
                plan.append((("tables", key), _C.AHEAD_TABLES,
                             dict(dense_item=dense_of[key], reorder=1 if reorder else 0,
                                  capacity=num_offsets * n, num_offsets=num_offsets),
                             [full, full, full, full, num_offsets * 4, num_offsets * 4]))
            elif what == "invert":
                key = entry[1]
                if key not in dense_of:
                    raise ValueError(f"the inverse of {key} needs its dense map first")
                num_offsets = plan[dense_of[key]][2]["num_offsets"]
                plan.append((("invert", key), _C.AHEAD_INVERT,
                             dict(dense_item=dense_of[key], capacity=num_offsets * n, num_offsets=num_offsets),
                             [num_offsets * n * 4]))
            else:
                raise ValueError(f"unknown recipe entry {entry!r}")
        if not plan:
            raise ValueError("empty recipe")
        # one allocation for every output, each at a multiple of 256 bytes
        total = 0
        self.places = []
        for _, _, _, sizes in plan:
            mine = []
            for size in sizes:
                mine.append(total if size else None)
                total += -(-size // _ALIGN) * _ALIGN
            self.places.append(mine)
        self.total = max(total, _ALIGN)
        self.plan = plan
        self.num_levels = len(levels)
        self.producer = {fields["target_level"]: i for i, (_, kind, fields, _) in enumerate(plan)
                         if kind == _C.AHEAD_COORDS}
        self.tags = {tag: i for i, (tag, _, _, _) in enumerate(plan)}
        self.items = (_C.LookaheadItem * len(plan))()
        self.hosts = {}                    # item -> (sizes, order) host arrays of a tables item
        self._keep = []                    # offset arrays the items point into
        for i, (_, kind, fields, _) in enumerate(plan):
            item = self.items[i]
            item.kind = kind
            item.source_level = fields.get("source_level", 0)
            item.target_level = fields.get("target_level", 0)
            item.dense_item = fields.get("dense_item", 0)
            item.reorder = fields.get("reorder", 0)
            item.capacity = fields["capacity"]
            if "stride" in fields:
                for k, value in enumerate(fields["stride"]):
                    item.stride[k] = int(value)
            if "offsets" in fields:
                offsets = fields["offsets"]
                self._keep.append(offsets)
                item.offsets = offsets.ctypes.data
                item.num_offsets = offsets.shape[0]
        self.bound_to = None

    def bind(self, base: int):
        """Points the items' outputs into the allocation at ``base``; tables
        items get fresh host arrays (the last pass's may still be in use)."""
        if base != self.bound_to:
            for i, places in enumerate(self.places):
                item = self.items[i]
                for slot, place in enumerate(places):
                    setattr(item, f"out{slot}", None if place is None else base + place)
            self.bound_to = base
        for i, (_, kind, fields, _) in enumerate(self.plan):
            if kind == _C.AHEAD_TABLES:
                sizes_host = np.zeros(fields["num_offsets"], dtype=np.int64)
                order_host = np.zeros(fields["num_offsets"], dtype=np.int64)
                self.hosts[i] = (sizes_host, order_host)
                self.items[i].host0 = sizes_host.ctypes.data
                self.items[i].host1 = order_host.ctypes.data


class AheadSession:
    """One pass's worth of requests running on the library's worker thread.
    ``layout`` is the last session's, reused when recipe and cloud shape match."""

    def __init__(self, recipe, offsets_of, coordinates: torch.Tensor, stride,
                 batch_dims: Optional[torch.Tensor], bounds=None, layout: Optional[AheadLayout] = None):
        self._open = False
        if not coordinates.is_cuda or not coordinates.is_contiguous() or coordinates.shape[0] == 0:
            raise ValueError("the look-ahead needs a non-empty contiguous cloud on a GPU")
        if batch_dims is not None and batch_dims.numel() <= 2:
            raise ValueError("a single cloud carries no batch boundaries here")
        self.device = coordinates.device
        n, ndim = coordinates.shape
        capacity = -(-n // _ROW_STEP) * _ROW_STEP
        index_dtype = batch_dims.dtype if batch_dims is not None else None
        num_batches = batch_dims.numel() - 1 if batch_dims is not None else 1
        signature = (recipe, tuple(stride), capacity, ndim, coordinates.dtype, index_dtype, num_batches)
        if layout is None or layout.signature != signature:
            layout = AheadLayout(recipe, offsets_of, stride, capacity, ndim, coordinates.dtype, index_dtype,
                                 num_batches)
        self.layout = layout
        # a fresh allocation every pass: views of the last one may still be in use
        # (when they are not, the allocator hands the same block back)
        self.pool = torch.empty((layout.total,), dtype=torch.uint8, device=self.device)
        self._words = self.pool.view(torch.int32)
        self._coords = self._words if coordinates.dtype == torch.int32 else self.pool.view(coordinates.dtype)
        self._dims = (None if index_dtype is None else
                      self._words if index_dtype == torch.int32 else self.pool.view(index_dtype))
        layout.bind(self.pool.data_ptr())
        self.hosts = dict(layout.hosts)
        self.index = dict(layout.tags)
        self._rows = {0: n}               # level -> number of rows, as items are taken
        _C.lookahead_start(coordinates, batch_dims, bounds, layout.items, layout.num_levels)
        self._open = True                  # only a session that started may finish the worker's
        global _running
        _running = weakref.ref(self)
        self._inputs = (coordinates, batch_dims)       # alive while the worker may read them

    def _ints(self, item: int, slot: int, rows: int, columns: int) -> torch.Tensor:
        """int32 [rows, columns] (or [rows] for columns = 0) at output ``slot`` of ``item``."""
        at = self.layout.places[item][slot] // 4
        if columns:
            return torch.as_strided(self._words, (rows, columns), (columns, 1), at)
        return torch.as_strided(self._words, (rows,), (1,), at)

    def _rows_of(self, level: int) -> int:
        rows = self._rows.get(level)
        if rows is None:
            rows = self._rows[level] = _C.lookahead_wait(self.layout.producer[level], self.device)
        return rows

    def take(self, tag):
        """What the worker built for ``tag``, the current stream ordered after
        it: ``(coordinates, batch_dims)``, the dense map, the dict
        ``kernel_map_tables`` returns, or the inverse map."""
        if not self._is_running():
            raise RuntimeError("this look-ahead session is over")
        item = self.index.pop(tag)
        size = _C.lookahead_wait(item, self.device)
        layout = self.layout
        _, kind, fields, _ = layout.plan[item]
        if kind == _C.AHEAD_COORDS:
            self._rows[fields["target_level"]] = size
            ndim = layout.ndim
            coords = torch.as_strided(self._coords, (size, ndim), (ndim, 1),
                                      layout.places[item][0] // layout.coord_dtype.itemsize)
            dims = None
            if self._dims is not None:
                dims = torch.as_strided(self._dims, (layout.num_batches + 1,), (1,),
                                        layout.places[item][1] // layout.index_dtype.itemsize)
            return coords, dims
        num_offsets = fields["num_offsets"]
        if kind == _C.AHEAD_DENSE:
            self._rows.setdefault(fields["target_level"], size)
            return self._ints(item, 0, num_offsets, size)
        if kind == _C.AHEAD_INVERT:
            return self._ints(item, 0, num_offsets, size)
        dense_fields = layout.plan[fields["dense_item"]][2]
        num_sources = self._rows_of(dense_fields["source_level"])
        num_targets = self._rows_of(dense_fields["target_level"])
        sizes_host, order_host = self.hosts[item]
        return dict(sizes_host=sizes_host, order_host=order_host,
                    sizes=self._ints(item, 4, num_offsets, 0), order=self._ints(item, 5, num_offsets, 0),
                    source_masks=self._ints(item, 0, num_offsets, num_sources),
                    target_masks=self._ints(item, 1, num_offsets, num_targets),
                    in_idx=self._ints(item, 2, size, 0), out_idx=self._ints(item, 3, size, 0))

    def _is_running(self) -> bool:
        return self._open and _running is not None and _running() is self

    def finish(self):
        """Waits for the worker to go idle and orders the current stream after
        everything it enqueued; the buffers may be released afterwards."""
        global _running
        if self._open:
            running = self._is_running()
            self._open = False
            if running:
                _running = None
                _C.lookahead_finish(self.device)
            self._inputs = None

    def __del__(self):
        try:
            self.finish()
        except Exception:
            pass
