"""Module forms of the global pooling functions (mirrors minuet/nn/pooling.py)."""
import torch
from torch.nn import Module

from minuet_amd.nn import functional as F

__all__ = ["GlobalAvgPool", "GlobalMaxPool", "GlobalSumPool"]


class GlobalAvgPool(Module):
    def forward(self, x) -> torch.Tensor:
        return F.global_avg_pool(x)


class GlobalMaxPool(Module):
    def forward(self, x) -> torch.Tensor:
        return F.global_max_pool(x)


class GlobalSumPool(Module):
    def forward(self, x) -> torch.Tensor:
        return F.global_sum_pool(x)
