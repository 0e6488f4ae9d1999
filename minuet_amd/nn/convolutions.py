"""``SparseConv`` / ``SparseConv3d`` and the ``KernelMapCache`` they share
(mirrors minuet/nn/convolutions.py of the reference).

The cache builds target coordinates and kernel maps with fused library calls
(``_C.target_coordinates``, ``_C.kernel_map_build``) instead of chains of
tensor expressions, keeps a host copy of the per-offset sizes so that the
forward pass never reads them back from the device, and orders offsets by
size with a STABLE sort (the reference's device sort is unstable, so its tie
order is not reproducible)."""
import contextlib
import functools
import os
import operator
from typing import Any, Dict, Optional, Union

import numpy as np
import torch
from torch.nn import Module

from minuet_amd.nn import functional as F
from minuet_amd.nn.functional import _C
from minuet_amd.nn.kernel_map import KernelMap
from minuet_amd.tensors import SparseTensor
from minuet_amd.utils.helpers import as_tuple, generate_kernel_offsets

__all__ = ["SparseConv", "SparseConv3d", "KernelMapCache"]

_TRANSPOSED_FIRST = ("Layer must transpose=True must have its corresponding non-transposed layer "
                     "before its execution")


class KernelMapCache(object):
    """Shares target coordinates and kernel maps between the layers of a network.

    Coordinates are cached per tensor stride (first writer wins), kernel maps
    per ``(source stride, target stride, kernel size, dilation)``; a transposed
    layer looks up the map of its forward twin and swaps the two rank tables.
    ``reset()`` must be called before every new input
    (reference: convolutions.py:18-173).

    A map exists in up to two forms: the dense map (``get_dense_kernel_map``,
    the query alone, no wait on the device) and the rank tables with sizes and
    order (``get_kernel_map``, the reference's tuple), made from the dense map
    when a layer asks for them.

    ``lookahead=True`` (or ``MINUET_LOOKAHEAD=1`` in the environment) makes the
    cache remember what a pass built and hand that list, at the first request
    after the next ``reset()``, to a worker thread of the library, which builds
    the levels and maps of the new cloud on a stream of its own while the
    calling thread enqueues layers (:mod:`minuet_amd.nn.lookahead`).  Results
    are the same; the price is one worst-case allocation per pass (no level has
    more rows than the input cloud) and one such session per process at a time
    (a second cache builds the ordinary way meanwhile).  ``num_ahead_hits``
    counts the requests served that way."""

    def __init__(self, ndim: int, dtype: torch.dtype, device: Union[str, torch.device],
                 layout: str = "minuet", disable_reordering: bool = False, lookahead: bool = False):
        self._ndim = ndim
        self._dtype = dtype
        self._device = device
        self._layout = layout
        self._disable_reordering = disable_reordering
        self._kernel_maps_cache = dict()        # key -> KernelMap of the forward layer
        self._swapped_maps_cache = dict()       # key -> the same map as its transposed layer reads it
        self._key_memo = dict()
        self._dense_maps_cache = dict()         # key -> (dense kernel map [O, T], number of sources)
        self._inverse_maps_cache = dict()       # key -> its inverse [O, S] (transposed layers)
        self._offset_groups_cache = dict()      # key -> offset-group tables of the dense map (False: none)
        self._coordinates_cache = dict()
        self._bounds_cache = dict()
        self.num_map_builds = 0
        self.num_coordinate_builds = 0
        # look-ahead: the requests of the last pass that built something, and the
        # session that builds them for the current cloud on the library's worker thread
        self._lookahead = lookahead or os.environ.get("MINUET_LOOKAHEAD", "") == "1"
        self._recording = []
        self._recipe = None
        self._recipe_rest = None      # the recipe without a first entry that this thread builds itself
        self._ahead = None
        self._ahead_layout = None
        self._ahead_tried = False
        self.num_ahead_hits = 0

    @functools.lru_cache(maxsize=None)
    def _kernel_offsets(self, source_stride, kernel_size, kernel_dilation) -> np.ndarray:
        return np.ascontiguousarray(
            generate_kernel_offsets(ndim=self._ndim, kernel_size=kernel_size,
                                    source_stride=source_stride, dilation=kernel_dilation,
                                    layout=self._layout), dtype=np.int64)

    def reset(self):
        if self._ahead is not None:
            # the worker may still write buffers of maps nobody asked for
            self._ahead.finish()
            self._ahead = None
        if self._recording:
            recipe = tuple(self._recording)
            if recipe != self._recipe:
                self._recipe = recipe
                # The first request of a pass is needed at once: when it is a dense
                # map that no later entry builds on, the asking thread makes it
                # itself while the worker starts on the rest.
                first = recipe[0]
                alone = first[0] == "dense" and not any(
                    entry[0] in ("tables", "invert") and entry[1] == first[1] for entry in recipe[1:])
                self._recipe_rest = recipe[1:] if alone and len(recipe) > 1 else None
            self._recording = []
        self._ahead_tried = False
        self._coordinates_cache.clear()
        self._kernel_maps_cache.clear()
        self._swapped_maps_cache.clear()
        self._dense_maps_cache.clear()
        self._inverse_maps_cache.clear()
        self._offset_groups_cache.clear()
        self._bounds_cache.clear()

    def _from_ahead(self, tag, record, coordinates, stride, batch_dims):
        """Notes the request ``record`` for the next pass's recipe and, with the
        look-ahead on, returns what the worker built for ``tag`` (None when it
        was not given that request, or failed at it).  The first request of a
        pass starts the worker on the recipe of the last one, from the cloud
        ``coordinates`` of stride ``stride``."""
        if not self._lookahead:
            return None
        self._recording.extend(record)
        if self._ahead is None:
            if self._ahead_tried or self._recipe is None or coordinates is None:
                return None
            self._ahead_tried = True
            from minuet_amd.nn.lookahead import AheadSession
            recipe = self._recipe
            if self._recipe_rest is not None and record and record[0] == recipe[0]:
                recipe = self._recipe_rest
            try:
                self._ahead = AheadSession(recipe, self._kernel_offsets, coordinates, tuple(stride),
                                           batch_dims, self._known_bounds(coordinates),
                                           layout=self._ahead_layout)
            except (ValueError, RuntimeError):
                _C.cuda_reset_error()
                return None
            self._ahead_layout = self._ahead.layout
        if tag not in self._ahead.index:
            return None
        try:
            result = self._ahead.take(tag)
        except RuntimeError:
            _C.cuda_reset_error()
            return None
        self.num_ahead_hits += 1
        return result

    def _known_bounds(self, coordinates: torch.Tensor):
        """Host copy of the per-dimension min / max of a coordinate tensor seen
        before (keyed by its storage), or None."""
        entry = self._bounds_cache.get((coordinates.data_ptr(), coordinates.shape[0]))
        return None if entry is None else entry[1]

    def _remember_bounds(self, coordinates: torch.Tensor, bounds: np.ndarray):
        # the entry keeps the tensor alive until reset(): its storage cannot be
        # handed to another tensor while the bounds are filed under its address
        self._bounds_cache[(coordinates.data_ptr(), coordinates.shape[0])] = (
            coordinates, np.array(bounds, dtype=np.int64))

    def get_target_coordinates(self, source_coordinates: torch.Tensor,
                               source_batch_dims: Optional[torch.Tensor],
                               source_stride, kernel_stride, transposed: bool = False):
        """Coordinates, stride and batch_dims of a layer's output
        (reference: convolutions.py:58-100)."""
        ndim = source_coordinates.shape[1]
        source_stride = as_tuple(source_stride, size=ndim, name="source_stride")
        kernel_stride = as_tuple(kernel_stride, size=ndim, name="kernel_stride")
        self._coordinates_cache.setdefault(
            source_stride, (source_coordinates, source_stride, source_batch_dims))
        combine = operator.floordiv if transposed else operator.mul
        target_stride = tuple(combine(a, b) for a, b in zip(source_stride, kernel_stride))
        hit = self._coordinates_cache.get(target_stride)
        if hit is not None:
            return hit
        if transposed:
            raise RuntimeError(_TRANSPOSED_FIRST)
        known = self._known_bounds(source_coordinates)
        ahead = self._from_ahead(("coords", target_stride), [("coords", source_stride, target_stride)],
                                 source_coordinates, source_stride, source_batch_dims)
        if ahead is not None:
            coords, batch_dims = ahead
        else:
            coords, batch_dims = _C.target_coordinates(source_coordinates.contiguous(),
                                                       source_batch_dims, target_stride,
                                                       source_bounds=known)
        self.num_coordinate_builds += 1
        if known is not None and source_coordinates.shape[0] > 0:
            # floor(c / s) * s is monotone, so the extremes map to the extremes
            ts = np.asarray(target_stride, dtype=np.int64)
            derived = known.copy()
            derived[:ndim] = np.floor_divide(known[:ndim], ts) * ts
            derived[4:4 + ndim] = np.floor_divide(known[4:4 + ndim], ts) * ts
            self._remember_bounds(coords, derived)
        entry = (coords, target_stride, batch_dims)
        self._coordinates_cache[target_stride] = entry
        return entry

    def coordinates_at(self, coordinates: torch.Tensor, stride, batch_dims: Optional[torch.Tensor]):
        """What ``get_target_coordinates`` returns for a layer of stride 1: the
        entry of the level ``stride`` (a tuple of ints), which these coordinates
        open if it is new."""
        entry = self._coordinates_cache.get(stride)
        if entry is None:
            entry = (coordinates, stride, batch_dims)
            self._coordinates_cache[stride] = entry
        return entry

    def _map_key(self, ndim, source_stride, target_stride, kernel_size, kernel_dilation, transposed):
        raw = (ndim, source_stride, target_stride, kernel_size, kernel_dilation, transposed)
        try:
            return self._key_memo[raw]
        except (KeyError, TypeError):          # first time, or an unhashable argument
            pass
        result = self._make_map_key(*raw)
        try:
            self._key_memo[raw] = result
        except TypeError:
            pass
        return result

    @staticmethod
    def _make_map_key(ndim, source_stride, target_stride, kernel_size, kernel_dilation, transposed):
        source_stride = as_tuple(source_stride, size=ndim, name="source_stride")
        target_stride = as_tuple(target_stride, size=ndim, name="target_stride")
        kernel_size = as_tuple(kernel_size, size=ndim, name="kernel_size")
        kernel_dilation = as_tuple(kernel_dilation, size=ndim, name="kernel_dilation")
        strides = (target_stride, source_stride) if transposed else (source_stride, target_stride)
        return strides + (kernel_size, kernel_dilation), source_stride, kernel_size, kernel_dilation

    def get_dense_kernel_map(self, source_coordinates: torch.Tensor, source_stride,
                             source_batch_dims: Optional[torch.Tensor],
                             target_coordinates: torch.Tensor, target_stride,
                             target_batch_dims: Optional[torch.Tensor], kernel_size,
                             kernel_dilation, transposed: bool = False) -> torch.Tensor:
        """The dense kernel map of a layer alone: ``[O, N_out]`` int32, source row
        per (offset, output row) in the layer's own offset order, -1 for none
        (the output of ``query_sorted_index_with_offsets``,
        reference: convolutions.py:147-153).  This is all the single-kernel
        dataflow needs; building it waits for nothing on the device.  A
        transposed layer gets the inverse of its forward layer's map."""
        key, source_stride, kernel_size, kernel_dilation = self._map_key(
            source_coordinates.shape[1], source_stride, target_stride, kernel_size, kernel_dilation,
            transposed)
        entry = self._dense_maps_cache.get(key)
        if entry is None:
            if transposed:
                raise RuntimeError(_TRANSPOSED_FIRST)
            offsets = self._kernel_offsets(source_stride, kernel_size, kernel_dilation)
            source_coordinates = source_coordinates.contiguous()
            target_coordinates = target_coordinates.contiguous()
            dense = self._from_ahead(("dense", key), [("dense", key)], source_coordinates, source_stride,
                                     source_batch_dims)
            if dense is None:
                dense, bounds = _C.kernel_map_dense(
                    source_coordinates, target_coordinates, offsets, source_batch_dims, target_batch_dims,
                    source_bounds=self._known_bounds(source_coordinates),
                    target_bounds=self._known_bounds(target_coordinates))
                if source_coordinates.shape[0] > 0 and target_coordinates.shape[0] > 0:
                    self._remember_bounds(source_coordinates, bounds[:8])
                    self._remember_bounds(target_coordinates, bounds[8:])
            self.num_map_builds += 1
            entry = (dense, source_coordinates.shape[0])
            self._dense_maps_cache[key] = entry
        if not transposed:
            return entry[0]
        return self._inverse_of(key)

    def get_offset_groups(self, source_coordinates: torch.Tensor, source_stride,
                          source_batch_dims: Optional[torch.Tensor],
                          target_coordinates: torch.Tensor, target_stride,
                          target_batch_dims: Optional[torch.Tensor], kernel_size,
                          kernel_dilation, transposed: bool = False):
        """The offset-group tables of a layer whose 27 offsets form a 3 x 3 x 3 grid
        (``_C.OffsetGroups``; None for other kernels and for transposed layers):
        what the ``offset_groups`` dataflow reads instead of rank tables.  Made
        from the dense kernel map in three launches; waits for nothing on the
        device.  Not in the reference, whose kernel map has one row per offset
        (convolutions.py:147-170)."""
        if transposed:
            return None
        key, stride_key, size_key, dilation_key = self._map_key(
            source_coordinates.shape[1], source_stride, target_stride, kernel_size, kernel_dilation, False)
        entry = self._offset_groups_cache.get(key)
        if entry is None:
            offsets = self._kernel_offsets(stride_key, size_key, dilation_key)
            entry = False
            if offsets.shape == (27, 3) and _C.offset_group_table(offsets) is not None:
                dense = self.get_dense_kernel_map(source_coordinates, source_stride, source_batch_dims,
                                                  target_coordinates, target_stride, target_batch_dims,
                                                  kernel_size, kernel_dilation)
                entry = _C.kernel_map_offset_groups(dense, offsets) or False
            self._offset_groups_cache[key] = entry
        return entry or None

    def _inverse_of(self, key) -> torch.Tensor:
        """Dense map of the transposed layer of ``key`` ([O, S]), made on first use."""
        inverse = self._inverse_maps_cache.get(key)
        if inverse is None:
            dense, num_sources = self._dense_maps_cache[key]
            inverse = self._from_ahead(("invert", key), [("invert", key)], None, None, None)
            if inverse is None:
                inverse = _C.kernel_map_invert(dense, num_sources)
            self._inverse_maps_cache[key] = inverse
        return inverse

    def get_kernel_map(self, source_coordinates: torch.Tensor, source_stride,
                       source_batch_dims: Optional[torch.Tensor],
                       target_coordinates: torch.Tensor, target_stride,
                       target_batch_dims: Optional[torch.Tensor], kernel_size, kernel_dilation,
                       disable_reordering: bool = False, transposed: bool = False) -> KernelMap:
        """The layer's :class:`KernelMap`, which unpacks like the reference's tuple
        ``(source_masks, target_masks, kernel_map_order, kernel_map_sizes)``
        (reference: convolutions.py:102-173)."""
        key, source_stride, kernel_size, kernel_dilation = self._map_key(
            source_coordinates.shape[1], source_stride, target_stride, kernel_size, kernel_dilation,
            transposed)
        cached = self._swapped_maps_cache if transposed else self._kernel_maps_cache
        hit = cached.get(key)
        if hit is not None:
            return hit
        forward = self._kernel_maps_cache.get(key)
        if forward is None:
            if transposed and key not in self._dense_maps_cache:
                raise RuntimeError(_TRANSPOSED_FIRST)
            forward = self._build_tables(key, source_coordinates, source_batch_dims, target_coordinates,
                                         target_batch_dims, source_stride, kernel_size, kernel_dilation,
                                         disable_reordering)
        if not transposed:
            return forward
        swapped = forward.swapped(dense=self._inverse_of(key))
        self._swapped_maps_cache[key] = swapped
        return swapped

    def _build_tables(self, key, source_coordinates, source_batch_dims, target_coordinates,
                      target_batch_dims, source_stride, kernel_size, kernel_dilation,
                      disable_reordering):
        """Rank tables, order and sizes of the forward layer of ``key``: from the
        dense map when a layer already asked for that, else everything at once.
        (For a transposed caller the coordinate arguments are the other way
        round, but then the dense map exists and they are not used.)"""
        reorder = not self._disable_reordering and not disable_reordering
        entry = self._dense_maps_cache.get(key)
        if entry is None and self._lookahead:
            # the worker builds the two halves as two items: take the dense map first
            dense = self._from_ahead(("dense", key), [("dense", key)], source_coordinates, source_stride,
                                     source_batch_dims)
            if dense is not None:
                self.num_map_builds += 1
                entry = self._dense_maps_cache[key] = (dense, source_coordinates.shape[0])
            else:
                del self._recording[-1]           # the all-at-once build below notes its own requests
        if entry is not None:
            # the query ran earlier for a layer that needed the dense map only
            dense, num_sources = entry
            built = self._from_ahead(("tables", key), [("tables", key, reorder)], source_coordinates,
                                     source_stride, source_batch_dims)
            if built is None:
                built = _C.kernel_map_tables(dense, num_sources, reorder=reorder, want_lists=True)
        else:
            if self._lookahead:
                self._recording.extend([("dense", key), ("tables", key, reorder)])
            offsets = self._kernel_offsets(source_stride, kernel_size, kernel_dilation)
            source_coordinates = source_coordinates.contiguous()
            target_coordinates = target_coordinates.contiguous()
            built = _C.kernel_map_build(source_coordinates, target_coordinates, offsets,
                                        source_batch_dims, target_batch_dims, reorder=reorder,
                                        want_lists=True, want_dense=True,
                                        source_bounds=self._known_bounds(source_coordinates),
                                        target_bounds=self._known_bounds(target_coordinates))
            self.num_map_builds += 1
            if source_coordinates.shape[0] > 0 and target_coordinates.shape[0] > 0:
                self._remember_bounds(source_coordinates, built["bounds"][:8])
                self._remember_bounds(target_coordinates, built["bounds"][8:])
            dense, num_sources = built["kernel_map"], source_coordinates.shape[0]
            self._dense_maps_cache[key] = (dense, num_sources)
        index_dtype = (source_coordinates.dtype if source_batch_dims is None
                       else source_batch_dims.dtype)
        cast = (lambda t: t) if index_dtype == torch.int32 else (lambda t: t.to(index_dtype))
        kernel_map = KernelMap(cast(built["source_masks"]), cast(built["target_masks"]),
                               cast(built["order"]) if reorder else None, cast(built["sizes"]),
                               sizes_host=built["sizes_host"],
                               order_host=built["order_host"] if reorder else None,
                               in_idx=built["in_idx"], out_idx=built["out_idx"], dense=dense,
                               num_sources=num_sources, num_targets=dense.shape[1])
        self._kernel_maps_cache[key] = kernel_map
        return kernel_map


class SparseConv(Module):
    r"""Sparse convolution over a :class:`SparseTensor`.

    With input points :math:`\mathcal{P}` and stride :math:`s` the output points
    are :math:`\mathcal{Q} = \{\lfloor p / s \rfloor s : p \in \mathcal{P}\}`
    (elementwise) and

    .. math:: F^{\mathcal{Q}}_i = \sum_j \sum_k
              [p_j = q_i + \delta_k] \, F^{\mathcal{P}}_j W_k

    with the offsets :math:`\delta_k` from
    :func:`~minuet_amd.utils.helpers.generate_kernel_offsets`.  Parameters are
    ``kernel`` ``[K^D, C_in, C_out]`` and optionally ``bias`` ``[C_out]``.  A
    transposed layer maps back to the coordinates its forward twin started from
    and therefore has to run after it (reference: convolutions.py:176-499).
    """

    __AVAILABLE_THRESHOLD__ = [-1, *list(np.linspace(0, 2, num=50)), None]
    __NUM_TUNING_ROUNDS__ = 10
    # The reference times its bucket GEMMs under every threshold because padded
    # rows are computed there (convolutions.py:367-389).  The grouped GEMM here
    # stops each group's tiles at the group's size, so the threshold changes the
    # buffer layout only and the sweep would time the same work 52 times: the
    # tuner keeps -1 (no padded rows, least scratch) unless this is set.
    __TUNE_THRESHOLD__ = False

    def __init__(self, ndim: int, in_channels: int, out_channels: int, kernel_size,
                 stride=1, dilation=1, bias: bool = False, transposed: bool = False,
                 dtype: Optional[torch.dtype] = None,
                 device: Optional[torch.device] = None):
        super().__init__()
        self.ndim = ndim
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = as_tuple(kernel_size, size=ndim, name="kernel_size")
        self.stride = as_tuple(stride, size=ndim, name="stride")
        self.dilation = as_tuple(dilation, size=ndim, name="dilation")
        self.transposed = transposed
        factory = {"device": device, "dtype": dtype}
        volume = int(np.prod(self.kernel_size))
        self._packed = None
        self.kernel = torch.nn.Parameter(torch.empty(volume, in_channels, out_channels, **factory))
        if bias:
            self.bias = torch.nn.Parameter(torch.empty(out_channels, **factory))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()
        self._kernel_map_cache: Optional[KernelMapCache] = None
        # Tile size 0 lets the library pick 16 bytes per lane.  (The reference
        # starts from one element per thread, convolutions.py:277-281, and
        # relies on autotune to leave that setting.)
        self._tunable_config = {"threshold": -1, "gather_tile_size": 0, "scatter_tile_size": 0,
                                "dataflow": "auto"}
        self._tuning_data = None
        self._identity_map = None
        self._routes = dict()
        self._trivial = None

    @property
    def _allow_shortcut_matmul(self) -> bool:
        return (all(x == 1 for x in self.dilation) and all(x == 1 for x in self.stride)
                and not self._kernel_map_cache._disable_reordering)

    @property
    def tunable_config(self) -> Dict[str, Any]:
        """Padding threshold and gather / scatter tile sizes of this layer."""
        return self._tunable_config

    @property
    def is_trivial(self) -> bool:
        return self._shape_flags()[0]

    @property
    def _unit_stride(self) -> bool:
        return self._shape_flags()[1]

    def _shape_flags(self):
        """(1x1x1 kernel with stride and dilation 1, stride 1), worked out once
        per setting of the three tuples."""
        shape = (self.stride, self.dilation, self.kernel_size)
        if self._trivial is None or self._trivial[0] != shape:
            self._trivial = (shape, (all(x == 1 for x in self.stride + self.dilation + self.kernel_size),
                                     all(x == 1 for x in self.stride)))
        return self._trivial[1]

    def extra_repr(self) -> str:
        parts = [f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}"]
        if any(x != 1 for x in self.stride):
            parts.append(f"stride={self.stride}")
        if any(x != 1 for x in self.dilation):
            parts.append(f"dilation={self.dilation}")
        if self.bias is None:
            parts.append("bias=False")
        if self.transposed:
            parts.append("transposed=True")
        return ", ".join(parts)

    def reset_parameters(self):
        """Uniform init in ``+-1/sqrt(C * K^D)`` with ``C`` the input (transposed:
        output) channel count (reference: convolutions.py:311-319)."""
        fan = self.out_channels if self.transposed else self.in_channels
        bound = 1.0 / np.sqrt(fan * len(self.kernel))
        with torch.no_grad():
            self.kernel.uniform_(-bound, bound)
            if self.bias is not None:
                self.bias.uniform_(-bound, bound)
        self.invalidate_cached_weights()

    def invalidate_cached_weights(self):
        """Drops the packed copy of ``kernel`` that inference passes keep.  The
        copy follows the parameter by its storage and version counter, which
        every in-place operation on the parameter itself bumps; writes through
        ``kernel.data`` (``kernel.data.copy_(...)``, ``.data.normal_()``) bump
        nothing, so call this after them (``reset_parameters``, ``load_state_dict``
        and ``.to()`` / ``.half()`` / ``.cuda()`` do it themselves)."""
        self._packed = None

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)
        self.invalidate_cached_weights()

    def _apply(self, fn, *args, **kwargs):
        result = super()._apply(fn, *args, **kwargs)
        self.invalidate_cached_weights()
        return result

    def set_kernel_map_cache(self, cache: KernelMapCache):
        self._kernel_map_cache = cache

    # ------------------------------------------------------------ autotune ----
    def _score(self, timer, **kwargs):
        times = []
        for _ in range(self.__NUM_TUNING_ROUNDS__):
            for kernel_map in self._tuning_data:
                times.append(timer(weights=self.kernel, source_masks=kernel_map.source_masks,
                                   target_masks=kernel_map.target_masks,
                                   kernel_map_sizes=kernel_map.kernel_map_sizes,
                                   allow_shortcut_matmul=self._allow_shortcut_matmul, **kwargs))
        return float(np.average(times)) if times else float("inf")

    @contextlib.contextmanager
    def autotune(self, free_buffers: bool = True):
        """Context that records the kernel maps of every forward call made inside
        it and, on exit, picks the fastest padding threshold, gather tile and
        scatter tile for them (reference: convolutions.py:337-444)::

            with conv.autotune():
                for x in samples:
                    conv(x)
        """
        try:
            self._tuning_data = list()
            if free_buffers:
                F.cuda_free_buffers()
            yield
            if free_buffers:
                F.cuda_free_buffers()
            if self.is_trivial or not self._tuning_data:
                return
            best = None
            thresholds = self.__AVAILABLE_THRESHOLD__ if self.__TUNE_THRESHOLD__ else []
            if not self.__TUNE_THRESHOLD__:
                self._tunable_config["threshold"] = -1
            for threshold in thresholds:
                try:
                    score = self._score(F.cuda_time_gemm, threshold=threshold)
                except RuntimeError:
                    F.cuda_reset_error()
                    print(f"Threshold {threshold} overflows memory exiting tuning")
                    print(f"optimal={self._tunable_config['threshold']}")
                    break
                if best is None or score < best:
                    best = score
                    self._tunable_config["threshold"] = threshold
            if free_buffers:
                F.cuda_free_buffers()
            for key, timer, channels in (("gather_tile_size", F.cuda_time_gather, self.in_channels),
                                         ("scatter_tile_size", F.cuda_time_scatter, self.out_channels)):
                best = None
                for tile in range(1, channels + 1):
                    if channels % tile != 0:
                        continue
                    try:
                        score = self._score(timer, tile_size=tile,
                                            threshold=self._tunable_config["threshold"])
                    except RuntimeError:
                        F.cuda_reset_error()      # tile shape this build does not offer
                        continue
                    if best is None or score < best:
                        best = score
                        self._tunable_config[key] = tile
                if free_buffers:
                    F.cuda_free_buffers()
            self._tune_dataflow()
        finally:
            self._tuning_data = None

    def _tune_dataflow(self):
        """Times one whole layer per dataflow on the recorded kernel maps (random
        features) and keeps the faster one."""
        best = None
        for dataflow in ("gather_gemm_scatter", "list_driven", "implicit", "offset_groups"):
            total = 0.0
            try:
                for kernel_map in self._tuning_data:
                    if dataflow in ("implicit", "offset_groups") and kernel_map.dense is None:
                        raise RuntimeError("no dense kernel map")
                    if dataflow == "list_driven" and not kernel_map.ensure_row_lists():
                        raise RuntimeError("no row lists for this kernel map")
                    sources = torch.randn(kernel_map.num_sources, self.in_channels,
                                          device=self.kernel.device).to(self.kernel.dtype)
                    order = kernel_map.kernel_map_order
                    if dataflow == "offset_groups":
                        offsets = self._kernel_map_cache._kernel_offsets(
                            (1,) * self.ndim, self.kernel_size, self.dilation)
                        groups = None
                        if (not self.transposed and sources.is_cuda and _C.offset_groups_forward_supported(
                                self.in_channels, self.out_channels, sources.dtype)):
                            groups = _C.kernel_map_offset_groups(kernel_map.dense, offsets)
                        if groups is None:
                            raise RuntimeError("no offset groups for this layer")
                        packed = F.pack_weights(self.kernel.detach())
                        call = lambda: _C.sparse_convolution_forward_groups(
                            sources, self.kernel.detach(), groups, packed_weights=packed)
                    else:
                        call = lambda: F.sparse_convolution_forward(
                            sources=sources, weights=self.kernel, kernel_map=kernel_map,
                            gather_tile_size=self._tunable_config["gather_tile_size"],
                            scatter_tile_size=self._tunable_config["scatter_tile_size"],
                            allow_shortcut_matmul=self._allow_shortcut_matmul and order is not None,
                            threshold=self._tunable_config["threshold"], dataflow=dataflow)
                    call()
                    start = torch.cuda.Event(enable_timing=True)
                    stop = torch.cuda.Event(enable_timing=True)
                    start.record()
                    for _ in range(max(1, self.__NUM_TUNING_ROUNDS__)):
                        call()
                    stop.record()
                    stop.synchronize()
                    total += start.elapsed_time(stop)
            except RuntimeError:
                F.cuda_reset_error()              # shape this dataflow does not offer
                continue
            if best is None or total < best:
                best = total
                self._tunable_config["dataflow"] = dataflow

    # ------------------------------------------------------------- forward ----
    def _packed_kernel(self, pad: int = 0):
        """``(weights, packed)``: the layer's weights (with ``pad`` zero input
        channels appended) and the same in the layout the matrix kernels stage,
        remade only when the parameter has changed (in-place updates bump its
        version counter).  ``packed`` is None while gradients are recorded."""
        kernel = self.kernel
        if torch.is_grad_enabled() and kernel.requires_grad:
            padded = kernel if pad == 0 else torch.nn.functional.pad(kernel, (0, 0, 0, pad))
            return padded, None
        key = (kernel.data_ptr(), kernel._version, kernel.dtype, kernel.device, pad)
        if self._packed is None or self._packed[0] != key:
            with torch.no_grad():
                weights = kernel.detach()
                if pad:
                    weights = torch.nn.functional.pad(weights, (0, 0, 0, pad))
                self._packed = (key, weights, F.pack_weights(weights))
        return self._packed[1], self._packed[2]

    def _row_padding(self, features: torch.Tensor) -> int:
        """Zero input channels to append so that the feature rows of a 16-bit
        layer become ones the single-kernel dataflow takes (4 or 8 bytes under
        a small kernel, else a multiple of 16 bytes); 0 where they already are,
        or where that dataflow is not an option."""
        if (features.dtype == torch.float32 or not features.is_cuda
                or self._tunable_config.get("dataflow", "auto") in ("gather_gemm_scatter", "list_driven",
                                                                     "offset_groups")):
            return 0
        esize = features.element_size()
        row_bytes = self.in_channels * esize
        widths = [b // esize for b in (4, 8) if row_bytes <= b] + [-(-row_bytes // 16) * 16 // esize]
        for width in widths:
            if _C.implicit_forward_supported(width, self.out_channels, features.dtype, self.kernel.shape[0]):
                return width - self.in_channels
        return 0

    def _takes_implicit(self, features: torch.Tensor, pad: int) -> bool:
        """Whether this call runs the single-kernel dataflow: forced by the
        tunable ``dataflow``, or chosen where it is the faster one."""
        dataflow = self._tunable_config.get("dataflow", "auto")
        if dataflow in ("gather_gemm_scatter", "list_driven", "offset_groups") or not features.is_cuda:
            return False
        if features.dtype != self.kernel.dtype:
            return False
        if dataflow == "implicit":
            return True
        return F.prefers_implicit(self.kernel.shape[0], self.in_channels + pad, self.out_channels,
                                  features.dtype)

    def _takes_offset_groups(self, features: torch.Tensor) -> bool:
        """Whether this call multiplies its offsets three at a time (the
        ``offset_groups`` dataflow): forced by the tunable ``dataflow``, or, under
        ``auto``, for the wide 16-bit 3 x 3 x 3 layers that the single-kernel form
        does not take, whose product rows are what bounds them."""
        dataflow = self._tunable_config.get("dataflow", "auto")
        if dataflow not in ("auto", "offset_groups") or not features.is_cuda or self.transposed:
            return False
        if (features.dtype != self.kernel.dtype or self.ndim != 3 or self.kernel.shape[0] != 27
                or not _C.offset_groups_forward_supported(self.in_channels, self.out_channels, features.dtype)):
            return False
        return dataflow == "offset_groups" or self.in_channels * features.element_size() >= 256

    def _pointwise(self, features: torch.Tensor, epilogue: Optional[F.Epilogue]) -> torch.Tensor:
        """1x1x1 kernel, stride 1: a plain ``features @ W`` (reference:
        convolutions.py:452-455).  Where the single-kernel forward takes the
        shape it runs there, as one offset whose kernel map is the identity,
        so that an epilogue costs no extra pass; otherwise ``torch.mm``."""
        weights = self.kernel.view(1, self.in_channels, self.out_channels)
        needs_grad = torch.is_grad_enabled() and (features.requires_grad or weights.requires_grad)
        if (features.is_cuda and not needs_grad
                and self._tunable_config.get("dataflow", "auto") not in ("gather_gemm_scatter", "list_driven")
                and features.dtype == weights.dtype
                and _C.implicit_forward_supported(self.in_channels, self.out_channels, weights.dtype)
                # measured against torch.mm plus a separate epilogue pass up to these widths;
                # wider layers are plain library GEMM territory
                and self.in_channels * weights.dtype.itemsize <= 512 and self.out_channels <= 128):
            rows = features.shape[0]
            identity = self._identity_map
            if identity is None or identity.shape[1] < rows or identity.device != features.device:
                identity = torch.arange(rows, dtype=torch.int32, device=features.device).view(1, rows)
                self._identity_map = identity
            return _C.sparse_convolution_forward_implicit(features, weights, identity[:, :rows],
                                                          epilogue=epilogue,
                                                          packed_weights=self._packed_kernel()[1])
        out = torch.mm(features, weights[0])
        return out if epilogue is None else epilogue.apply(out)

    def forward(self, inputs: SparseTensor,
                epilogue: Optional[F.Epilogue] = None) -> SparseTensor:
        """``epilogue`` (not in the reference, whose layers end at the bias add,
        convolutions.py:446-499) is applied to the output rows in the same pass
        that writes them: ``act(conv(x) * scale + shift + residual)``, with the
        bias, if any, added before the scale."""
        if epilogue is not None and self.bias is not None:
            bias = self.bias.float()
            shift = bias if epilogue.scale is None else bias * epilogue.scale.float()
            if epilogue.shift is not None:
                shift = shift + epilogue.shift.float()
            epilogue = F.Epilogue(epilogue.scale, shift, epilogue.residual, epilogue.activation,
                                  epilogue.negative_slope)
        if self.is_trivial:
            features = self._pointwise(inputs.F, epilogue)
            coordinates, stride, batch_dims = inputs.C, inputs.stride, inputs.batch_dims
        else:
            cache = self._kernel_map_cache
            if cache is None:
                raise ValueError("Kernel map cache must be specified")
            if self._unit_stride and type(inputs.stride) is tuple:
                coordinates, stride, batch_dims = cache.coordinates_at(inputs.C, inputs.stride,
                                                                       inputs.batch_dims)
            else:
                coordinates, stride, batch_dims = cache.get_target_coordinates(
                    transposed=self.transposed, source_coordinates=inputs.C,
                    source_batch_dims=inputs.batch_dims, source_stride=inputs.stride,
                    kernel_stride=self.stride)
            map_args = dict(transposed=self.transposed, source_coordinates=inputs.C,
                            source_stride=inputs.stride, source_batch_dims=inputs.batch_dims,
                            target_coordinates=coordinates, target_stride=stride,
                            target_batch_dims=batch_dims, kernel_size=self.kernel_size,
                            kernel_dilation=self.dilation)
            sources = inputs.F
            # the route depends on the layer, the feature type and the tunable
            # dataflow only: decided once, then looked up
            route_key = (sources.dtype, sources.is_cuda, self._tunable_config.get("dataflow", "auto"))
            route = self._routes.get(route_key)
            if route is None:
                grouped = self._takes_offset_groups(sources)
                pad = 0 if grouped else self._row_padding(sources)
                route = (pad, not grouped and self._takes_implicit(sources, pad), grouped)
                self._routes[route_key] = route
            pad, implicit, grouped = route
            groups = cache.get_offset_groups(**map_args) if grouped and self._tuning_data is None else None
            if groups is not None:
                # offsets multiplied three at a time: needs the dense map and its group tables only
                weights, packed = self._packed_kernel()
                features = _C.sparse_convolution_forward_groups(sources, weights, groups, epilogue=epilogue,
                                                                packed_weights=packed)
            elif implicit and self._tuning_data is None:
                # single-kernel dataflow: the dense map is all it needs
                dense = cache.get_dense_kernel_map(**map_args)
                if pad:
                    sources = torch.nn.functional.pad(sources, (0, pad))
                weights, packed = self._packed_kernel(pad)
                features = _C.sparse_convolution_forward_implicit(sources, weights, dense,
                                                                  epilogue=epilogue,
                                                                  packed_weights=packed)
            else:
                features = self._forward_tables(cache, map_args, sources, epilogue)
        if self.bias is not None and epilogue is None:
            features += self.bias
        if batch_dims is not None and len(batch_dims) <= 2:
            batch_dims = None
        return SparseTensor.like(inputs, features, coordinates, stride, batch_dims)

    def _forward_tables(self, cache, map_args, sources, epilogue):
        """Gather -> GEMM -> Scatter through the rank tables (the reference's
        dataflow, convolutions.py:470-494)."""
        kernel_map = cache.get_kernel_map(**map_args)
        if self._tuning_data is not None:
            self._tuning_data.append(kernel_map)
        dataflow = "gather_gemm_scatter"
        if (self._tunable_config.get("dataflow") == "list_driven" and self._tuning_data is None
                and sources.is_cuda and kernel_map.ensure_row_lists()):
            dataflow = "list_driven"
        weights, packed = self._packed_kernel() if sources.is_cuda else (self.kernel, None)
        return F.sparse_convolution_forward(
            sources=sources, weights=weights, kernel_map=kernel_map,
            gather_tile_size=self._tunable_config["gather_tile_size"],
            scatter_tile_size=self._tunable_config["scatter_tile_size"],
            allow_shortcut_matmul=self._allow_shortcut_matmul,
            threshold=self._tunable_config["threshold"], epilogue=epilogue,
            dataflow=dataflow, packed_weights=packed)


class SparseConv3d(SparseConv):
    """:class:`SparseConv` for 3-D point clouds; never transposed
    (reference: convolutions.py:502-527)."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, dilation=1,
                 bias: bool = False, dtype: Optional[torch.dtype] = None,
                 device: Optional[torch.device] = None):
        super().__init__(ndim=3, in_channels=in_channels, out_channels=out_channels,
                         kernel_size=kernel_size, stride=stride, dilation=dilation, bias=bias,
                         transposed=False, dtype=dtype, device=device)
