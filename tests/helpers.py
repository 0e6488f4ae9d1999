"""Shared input builders for the parity tests."""
import numpy as np
import torch

import minuet_oracle as orc


def random_cloud(n, extent, seed, ndim=3, lo=0, duplicates=0.0, dtype=np.int32):
    """n random rows in [lo, lo+extent)^ndim; a fraction of rows is duplicated."""
    rng = np.random.default_rng(seed)
    c = rng.integers(lo, lo + extent, size=(n, ndim)).astype(dtype)
    if duplicates > 0 and n > 1:
        k = int(n * duplicates)
        src = rng.integers(0, n, size=k)
        dst = rng.integers(0, n, size=k)
        c[dst] = c[src]
    return c


def sorted_unique(coords, batch_dims=None):
    """Oracle-side sort + unique -> (coords, batch_dims)."""
    idx = orc.arg_sort_coordinates(coords, batch_dims)
    c = coords[idx]
    u, uidx = orc.unique_coordinates(c, batch_dims)
    bd = None
    if batch_dims is not None:
        bd = uidx[np.asarray(batch_dims, dtype=np.int64)].astype(np.asarray(batch_dims).dtype)
    return u, bd


def dev(array, device="cuda"):
    return None if array is None else torch.from_numpy(np.ascontiguousarray(array)).to(device)


def host(tensor):
    return None if tensor is None else tensor.detach().cpu().numpy()
