"""Random unique coordinates (mirrors minuet/utils/random.py)."""
import random

import numpy as np

__all__ = ["random_unique_points"]


def random_unique_points(ndim: int, n: int, c_min: int, c_max: int, dtype=np.int32) -> np.ndarray:
    """``n`` distinct points with every coordinate in ``[c_min, c_max]`` (a
    virtual Fisher-Yates shuffle over the cell indices, driven by Python's
    ``random`` module)."""
    side = c_max - c_min + 1
    cells = side ** ndim
    if n > cells:
        raise ValueError(f"Cannot sample {n} points without replacement from a space with only "
                         f"{cells} possible points")
    moved = {}
    points = np.empty((n, ndim), dtype=dtype)
    for i in range(n):
        pick = random.randrange(i, cells)
        value = moved.get(pick, pick)
        moved[pick] = moved.get(i, i)
        for j in range(ndim):
            value, rem = divmod(value, side)
            points[i, j] = rem + c_min
    return points
