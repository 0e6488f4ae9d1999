"""Global pooling over each point cloud of a SparseTensor (mirrors
minuet/nn/functional/pooling.py; plain tensor reductions on the features)."""
import torch

__all__ = ["global_avg_pool", "global_max_pool", "global_sum_pool"]


def _per_cloud(x, reduce):
    if x.batch_dims is None:
        return reduce(x.F)
    bounds = x.batch_dims.tolist()
    return torch.stack([reduce(x.F[bounds[k]:bounds[k + 1]]) for k in range(x.batch_size)], dim=0)


def global_avg_pool(x):
    """Mean feature of every point cloud, stacked in batch order."""
    return _per_cloud(x, lambda f: torch.mean(f, dim=0))


def global_sum_pool(x):
    """Feature sum of every point cloud, stacked in batch order."""
    return _per_cloud(x, lambda f: torch.sum(f, dim=0))


def global_max_pool(x):
    """Channel-wise maximum of every point cloud, stacked in batch order."""
    return _per_cloud(x, lambda f: torch.max(f, dim=0)[0])
