"""Gather-GEMM-Scatter forward and its stage timers (mirrors
minuet/nn/functional/convolution.py)."""
from typing import Optional

import torch

from . import _C
from ..kernel_map import KernelMap

__all__ = ["cuda_time_gather", "cuda_time_scatter", "sparse_convolution_forward",
           "cuda_time_gemm", "set_gemm_parallel_level", "Epilogue", "pack_weights",
           "prefers_implicit"]

pack_weights = _C.pack_weights

Epilogue = _C.Epilogue

GEMM_PARALLEL_LEVEL = 4
DATAFLOWS = ("auto", "gather_gemm_scatter", "implicit", "list_driven")


def set_gemm_parallel_level(level: int):
    """Kept for compatibility (reference: convolution.py:15-25).  The reference
    spreads per-bucket GEMMs over this many streams; here all offsets run in
    one grouped launch, so the value has no effect."""
    global GEMM_PARALLEL_LEVEL
    GEMM_PARALLEL_LEVEL = level


def prefers_implicit(num_offsets: int, num_source_features: int, num_target_features: int,
                     dtype: torch.dtype) -> bool:
    """Whether ``dataflow="auto"`` takes the single-kernel form for a layer of
    this shape: it must fit that kernel, and it must be the faster one, which
    measurements say it is for 16-bit features with source rows of up to 128
    bytes and up to 128 output channels, and for rows of up to 256 bytes with up
    to 64 output channels under kernels of more than 8 offsets (beyond that its
    matrix work on empty (offset, target) pairs outweighs the buffer traffic it
    saves).  fp32 matrix work is 16x dearer, so there it only pays where most
    (offset, target) pairs are hits, i.e. for small layers with strided 2^D
    kernels."""
    if not _C.implicit_forward_supported(num_source_features, num_target_features, dtype, num_offsets):
        return False
    if dtype != torch.float32:
        row_bytes = num_source_features * dtype.itemsize
        if row_bytes <= 128:
            return num_target_features <= 128
        return row_bytes <= 256 and num_target_features <= 64 and num_offsets > 8
    return num_offsets <= 8 and num_source_features * num_target_features <= 1024


def cuda_time_gather(weights: torch.Tensor, source_masks: torch.Tensor,
                     target_masks: torch.Tensor, kernel_map_sizes: torch.Tensor,
                     tile_size: int, allow_shortcut_matmul: bool = False,
                     threshold: Optional[float] = 0) -> float:
    """Milliseconds of one Gather with ``tile_size`` feature elements per lane
    (reference: convolution.py:28-53)."""
    return _C.cuda_time_gather(tile_size, allow_shortcut_matmul, threshold, weights,
                               source_masks, target_masks, kernel_map_sizes)


def cuda_time_scatter(weights: torch.Tensor, source_masks: torch.Tensor,
                      target_masks: torch.Tensor, kernel_map_sizes: torch.Tensor,
                      tile_size: int, allow_shortcut_matmul: bool = False,
                      threshold: Optional[float] = 0) -> float:
    """Milliseconds of one Scatter (reference: convolution.py:56-81)."""
    return _C.cuda_time_scatter(tile_size, allow_shortcut_matmul, threshold, weights,
                                source_masks, target_masks, kernel_map_sizes)


def cuda_time_gemm(weights: torch.Tensor, source_masks: torch.Tensor,
                   target_masks: torch.Tensor, kernel_map_sizes: torch.Tensor,
                   allow_shortcut_matmul: bool = False, parallel: Optional[int] = None,
                   threshold: Optional[float] = 0) -> float:
    """Milliseconds of the grouped GEMM (reference: convolution.py:84-107)."""
    if parallel is None:
        parallel = GEMM_PARALLEL_LEVEL
    return _C.cuda_time_gemm(allow_shortcut_matmul, parallel, threshold, weights, source_masks,
                             target_masks, kernel_map_sizes)


def sparse_convolution_forward(sources: torch.Tensor, weights: torch.Tensor,
                               source_masks: Optional[torch.Tensor] = None,
                               target_masks: Optional[torch.Tensor] = None,
                               kernel_map_order: Optional[torch.Tensor] = None,
                               kernel_map_sizes: Optional[torch.Tensor] = None,
                               gather_tile_size: int = 0, scatter_tile_size: int = 0,
                               allow_shortcut_matmul: bool = False,
                               parallel: Optional[int] = None,
                               threshold: Optional[float] = 0,
                               epilogue: Optional[_C.Epilogue] = None,
                               dataflow: str = "auto",
                               packed_weights: Optional[torch.Tensor] = None,
                               kernel_map=None) -> torch.Tensor:
    """Output features ``[N_out, C_out]`` of one sparse convolution
    (reference: convolution.py:110-155).

    The kernel map comes either as the reference's four tensors
    (``source_masks``, ``target_masks``, ``kernel_map_order``,
    ``kernel_map_sizes``; a 4-tuple from ``KernelMapCache.get_kernel_map``
    unpacks into them) or as ``kernel_map=`` a :class:`~minuet_amd.nn.KernelMap`,
    which is what ``KernelMapCache.get_kernel_map`` returns.  With the four
    tensors alone the call behaves like the reference: Gather, grouped GEMM and
    Scatter as separate kernels, and the sizes are read back from the device
    once per call.  A ``KernelMap`` carries host copies of sizes and order, the
    pair lists and the dense map, with which nothing is read back, the Gather
    is folded into the GEMM's operand load and ``dataflow`` has a choice:

    ``"gather_gemm_scatter"`` is the reference's dataflow, ``"implicit"`` the
    single-kernel output-stationary form (needs ``kernel_map.dense`` and
    ``weights`` in their original offset order, as a layer holds them) and
    ``"auto"`` takes the implicit form where it is the faster one: 16-bit
    features whose rows it can stage, and small fp32 layers with 2^D kernels.

    ``"list_driven"`` is Gather-GEMM-Scatter without the rank tables: the GEMM
    reads its rows through the pair list and writes its products in
    target-major order (``KernelMap.row_ptr`` / ``out_pos``, built on first use
    from the dense map), so that Scatter reads them as one stream.  Scatter
    gains what the GEMM's scattered row writes lose, so ``"auto"`` never picks
    it; a layer's autotuner times it beside the other two.  Padding threshold,
    gather tile and the centre-offset shortcut have no meaning there.

    ``epilogue`` (:class:`Epilogue`) is applied to each output row before it is
    rounded to the feature dtype.  ``packed_weights`` (``pack_weights(weights)``,
    kept by the caller while the weights are unchanged) spares the packing pass
    that otherwise starts every call; it needs a ``KernelMap`` when the map is
    reordered (the host copy of the order) and is ignored without."""
    if not sources.is_cuda:
        raise NotImplementedError
    if dataflow not in DATAFLOWS:
        raise ValueError(f"dataflow must be one of {DATAFLOWS}")
    if kernel_map is None and isinstance(source_masks, KernelMap):
        kernel_map, source_masks = source_masks, None
    host_sizes = host_order = gather_index = dense = None
    if kernel_map is not None:
        source_masks, target_masks, kernel_map_order, kernel_map_sizes = kernel_map
        host_sizes, host_order = kernel_map.sizes_host, kernel_map.order_host
        gather_index = kernel_map.in_idx if host_sizes is not None else None
        dense = kernel_map.dense
    if dataflow == "implicit" and dense is None:
        raise ValueError("the implicit dataflow needs a KernelMap with its dense map")
    if dense is not None and dataflow in ("auto", "implicit"):
        if dataflow == "implicit" or prefers_implicit(weights.shape[0], weights.shape[1],
                                                      weights.shape[2], weights.dtype):
            return _C.sparse_convolution_forward_implicit(sources, weights, dense, epilogue=epilogue,
                                                          packed_weights=packed_weights)
    if dataflow == "list_driven":
        if kernel_map is None or gather_index is None or not kernel_map.ensure_row_lists():
            raise ValueError("the list-driven dataflow needs a KernelMap with its dense map and pair lists")
        # list-driven form: Gather folded into the GEMM, products written in
        # target-major order, Scatter streams through them (no rank table read)
        return _C.sparse_convolution_forward_rows(
            sources, weights, host_sizes, host_order, gather_index, kernel_map.out_pos, kernel_map.row_ptr,
            scatter_tile_size=scatter_tile_size, epilogue=epilogue, packed_weights=packed_weights)
    if source_masks is None or target_masks is None or kernel_map_sizes is None:
        raise ValueError("the Gather-GEMM-Scatter dataflow needs the rank tables and sizes of the kernel map")
    if parallel is None:
        parallel = GEMM_PARALLEL_LEVEL
    if gather_index is not None and (kernel_map_order is None or host_order is not None):
        # the map brings host sizes and pair lists: what depends on it alone is checked once per map
        return _C.sparse_convolution_forward_map(
            sources, weights, kernel_map, gather_tile_size, scatter_tile_size, allow_shortcut_matmul,
            parallel, threshold, epilogue=epilogue, packed_weights=packed_weights)
    if kernel_map_order is not None:
        if host_order is None:
            packed_weights = None
        kernel_map_order = kernel_map_order.contiguous()
    return _C.cuda_sparse_convolution_forward(
        gather_tile_size, scatter_tile_size, allow_shortcut_matmul, parallel, threshold,
        sources.contiguous(), weights.contiguous(), source_masks.contiguous(),
        target_masks.contiguous(), kernel_map_order, kernel_map_sizes.contiguous(),
        kernel_map_sizes_host=host_sizes, gather_index=gather_index, epilogue=epilogue,
        packed_weights=packed_weights, kernel_map_order_host=host_order)
