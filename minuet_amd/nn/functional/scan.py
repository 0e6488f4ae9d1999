"""Kernel-map sizes and rank tables (mirrors minuet/nn/functional/scan.py)."""
import torch

from . import _C

__all__ = ["compute_kernel_map_masks", "compute_kernel_map_sizes"]


def compute_kernel_map_sizes(kernel_map: torch.Tensor) -> torch.Tensor:
    """Hits per weight offset of a dense kernel map (reference: scan.py:8-24)."""
    kernel_map = kernel_map.contiguous()
    if not kernel_map.is_cuda:
        raise NotImplementedError
    return _C.cuda_compute_kernel_map_sizes(kernel_map)


def compute_kernel_map_masks(num_sources: int, kernel_map: torch.Tensor,
                             kernel_map_sizes: torch.Tensor):
    """Input and output rank tables ``[N_weight, N_in]`` / ``[N_weight, N_out]``
    of a dense kernel map (reference: scan.py:27-48)."""
    kernel_map = kernel_map.contiguous()
    kernel_map_sizes = kernel_map_sizes.contiguous()
    if not kernel_map.is_cuda:
        raise NotImplementedError
    return _C.cuda_compute_kernel_map_masks(num_sources, kernel_map, kernel_map_sizes)
