"""CPU oracle for the sparse-convolution hot path (Map -> Gather -> GEMM -> Scatter).

THIS IS TEST INFRASTRUCTURE.  It is a NumPy restatement of what the reference
computes, used only as the checker in tests/, in the smoke test and as the
timed ``cpu_baseline`` of the benchmark.  The product never imports it.

Every function names the reference lines it restates (paths relative to the
reference checkout).  The reference has no CPU path, no tests and no golden
vectors, so each function is pinned by independent checks in
``tests/test_oracle.py``:

  generate_kernel_offsets      closed-form known answers (k=2,3,5; stride; layouts)
  arg_sort_coordinates         python ``sorted`` on tuples (stable) + permutation invariants
  unique_coordinates           ``np.unique(axis=0)`` per batch + run-end counting
  target_coordinates           python set of floor-divided tuples (negatives included)
  query_sorted_index           brute force with a python dict over every (offset, target)
  kernel_map_sizes / masks     counting / ranking by plain python loops + invariants
  padding buckets / cumsum     hand cases worked from the reference loop + invariants
  sparse_convolution_forward   dense ``torch.nn.functional.conv3d`` / ``conv_transpose3d``
                               on a densified grid, k=1 -> F @ W, isolated voxel, all-ones

Integer outputs are exact.  Feature outputs are computed in float64 unless a
dtype is requested.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import numpy as np

__all__ = [
    "as_tuple", "generate_kernel_offsets", "arg_sort_coordinates",
    "unique_coordinates", "target_coordinates", "query_sorted_index_with_offsets",
    "compute_kernel_map_sizes", "stable_size_order", "compute_kernel_map_masks",
    "kernel_map_pair_lists", "generate_padding_buckets",
    "cumsum_kernel_padded_sizes", "sparse_convolution_forward",
    "build_kernel_map", "conv_layer",
]


def as_tuple(value, size: int) -> Tuple[int, ...]:
    """Scalar -> repeated tuple; iterable -> tuple of the given size
    (minuet/utils/helpers.py:138-162)."""
    if np.isscalar(value):
        return tuple(int(value) for _ in range(size))
    value = tuple(int(v) for v in value)
    if len(value) != size:
        raise ValueError(f"expected {size} elements but found {len(value)}")
    return value


def generate_kernel_offsets(ndim: int, kernel_size, source_stride=1, dilation=1,
                            layout: str = "minuet") -> np.ndarray:
    """Weight offsets of a sparse convolution (minuet/utils/helpers.py:165-212).

    Per dimension an odd kernel spans ``[-k//2, k//2]`` and an even one
    ``[-k/2+1, k/2]``; rows enumerate the Cartesian product with dimension 0
    slowest ("minuet" layout), then everything is scaled by stride*dilation.
    """
    ks = as_tuple(kernel_size, ndim)
    ss = as_tuple(source_stride, ndim)
    dl = as_tuple(dilation, ndim)
    axes = []
    for k in ks:
        hi = k // 2
        lo = -hi if k % 2 == 1 else -hi + 1
        axes.append(list(range(lo, hi + 1)))
    rows = [[]]
    for axis in axes:                      # dim 0 outermost -> slowest
        rows = [r + [v] for r in rows for v in axis]
    grid = np.asarray(rows, dtype=np.int64).reshape([len(a) for a in axes] + [ndim])
    if layout == "minuet":
        pass
    elif layout == "torchsparse":
        if int(np.prod(ks)) % 2 == 1:
            grid = np.transpose(grid, list(range(ndim - 1, -1, -1)) + [ndim])
    elif layout == "minkowski":
        grid = np.transpose(grid, list(range(ndim - 1, -1, -1)) + [ndim])
    else:
        raise NotImplementedError(layout)
    flat = grid.reshape(-1, ndim)
    return flat * np.asarray(ss, dtype=np.int64) * np.asarray(dl, dtype=np.int64)


def _batch_ids(n: int, batch_dims: Optional[np.ndarray]) -> np.ndarray:
    """Batch id of every row: row i belongs to g with bd[g] <= i < bd[g+1]
    (csrc/minuet/cuda/kernels/load_batch_id_with_permutation.cuh:9)."""
    if batch_dims is None:
        return np.zeros(n, dtype=np.int64)
    bd = np.asarray(batch_dims, dtype=np.int64)
    return np.searchsorted(bd, np.arange(n, dtype=np.int64), side="right") - 1


def arg_sort_coordinates(coords: np.ndarray,
                         batch_dims: Optional[np.ndarray] = None) -> np.ndarray:
    """Stable lexicographic arg-sort, dimension 0 most significant, batch-major
    (csrc/minuet/cuda/functions/arg_sort_coodrinates.cu:273-360,362-469;
    comparison order csrc/minuet/common/functions.h:94-105).  Ties keep input
    order because every radix pass of the reference is stable."""
    coords = np.asarray(coords)
    n, ndim = coords.shape
    keys = [coords[:, d] for d in range(ndim - 1, -1, -1)]   # last key = primary
    keys.append(_batch_ids(n, batch_dims))
    return np.lexsort(keys).astype(np.int64)                  # lexsort is stable


def unique_coordinates(sorted_coords: np.ndarray,
                       batch_dims: Optional[np.ndarray] = None):
    """Run-length unique of SORTED rows
    (csrc/minuet/cuda/functions/unique_coordinates.cu:16-46,57-70 and
    kernels/fill_unique_coordinate.cuh:13-19).

    ``idx[0] = 0`` and ``idx[i+1] = idx[i] + [row i ends a run]`` where a run
    also ends at the last row of a batch; the representative of a run is
    written at ``idx[i]``.  Returns ``(unique_rows, idx)`` with ``idx`` of
    length N+1 (int64), so ``idx[batch_dims]`` are the new batch boundaries.
    """
    c = np.asarray(sorted_coords)
    n = c.shape[0]
    ends = np.ones(n, dtype=bool)
    if n > 1:
        ends[:-1] = np.any(c[:-1] != c[1:], axis=1)
    if batch_dims is not None:
        bd = np.asarray(batch_dims, dtype=np.int64)
        inner = bd[(bd >= 1) & (bd <= n)] - 1
        ends[inner] = True
    idx = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(ends, out=idx[1:])
    return c[ends].copy(), idx


def target_coordinates(source_coords: np.ndarray, batch_dims: Optional[np.ndarray],
                       target_stride):
    """Output voxel set of a strided convolution
    (minuet/nn/convolutions.py:84-99): floor-divide by the target stride,
    multiply back, sort, unique.  Returns ``(coords, target_batch_dims)``."""
    c = np.asarray(source_coords)
    ts = np.asarray(as_tuple(target_stride, c.shape[1]), dtype=c.dtype)
    t = np.floor_divide(c, ts) * ts
    order = arg_sort_coordinates(t, batch_dims)
    t = t[order]
    uniq, idx = unique_coordinates(t, batch_dims)
    tbd = None
    if batch_dims is not None:
        bd = np.asarray(batch_dims)
        tbd = idx[bd.astype(np.int64)].astype(bd.dtype)
    return uniq, tbd


def _row_keys(rows: np.ndarray, lo: np.ndarray, span: np.ndarray):
    """Mixed-radix key, dimension 0 most significant
    (csrc/minuet/cuda/kernels/flatten_coordinates.cuh:18-38).  Python ints
    when the product of spans does not fit int64."""
    total = 1
    for s in span:
        total *= int(s)
    if total < (1 << 62):
        key = np.zeros(rows.shape[0], dtype=np.int64)
        for d in range(rows.shape[1]):
            key = key * int(span[d]) + (rows[:, d].astype(np.int64) - int(lo[d]))
        return key
    key = np.zeros(rows.shape[0], dtype=object)
    for d in range(rows.shape[1]):
        key = key * int(span[d]) + (rows[:, d].astype(object) - int(lo[d]))
    return key


def query_sorted_index_with_offsets(sources: np.ndarray, targets: np.ndarray,
                                    offsets: np.ndarray,
                                    source_batch_dims: Optional[np.ndarray] = None,
                                    target_batch_dims: Optional[np.ndarray] = None,
                                    dtype=None) -> np.ndarray:
    """Dense kernel map ``M[o, t] = j`` with ``sources[j] == targets[t] + offsets[o]``
    in every dimension (and the same batch), else -1
    (csrc/minuet/cuda/kernels/query_sorted_index_with_offsets.cuh:36-77,
    batched: multi_query_sorted_index_with_offsets.cuh:38-91 which searches
    only the sources of the target's own batch).

    Restated as one ``searchsorted`` per offset over mixed-radix keys whose
    per-dimension span leaves room for the offset, so a shifted target can
    never alias into a neighbouring row.
    """
    s = np.asarray(sources)
    t = np.asarray(targets)
    off = np.asarray(offsets).astype(np.int64)
    num_s, ndim = s.shape
    num_t = t.shape[0]
    num_o = off.shape[0]
    if dtype is None:
        dtype = s.dtype if source_batch_dims is None else np.asarray(source_batch_dims).dtype
    out = np.full((num_o, num_t), -1, dtype=dtype)
    if num_s == 0 or num_t == 0 or num_o == 0:
        return out
    sb = _batch_ids(num_s, source_batch_dims)
    tb = _batch_ids(num_t, target_batch_dims)
    s64 = np.concatenate([sb[:, None], s.astype(np.int64)], axis=1)
    t64 = np.concatenate([tb[:, None], t.astype(np.int64)], axis=1)
    omin = np.concatenate([[0], off.min(axis=0)])
    omax = np.concatenate([[0], off.max(axis=0)])
    lo = np.minimum(s64.min(axis=0), t64.min(axis=0) + omin)
    hi = np.maximum(s64.max(axis=0), t64.max(axis=0) + omax)
    span = hi - lo + 1
    skeys = _row_keys(s64, lo, span)
    # sources are sorted (batch-major, lexicographic) => keys are non-decreasing
    for o in range(num_o):
        shifted = t64.copy()
        shifted[:, 1:] += off[o]
        q = _row_keys(shifted, lo, span)
        pos = np.searchsorted(skeys, q, side="left")
        pos_c = np.minimum(pos, num_s - 1)
        hit = (pos < num_s) & (skeys[pos_c] == q)
        out[o, hit] = pos_c[hit]
    return out


def compute_kernel_map_sizes(kernel_map: np.ndarray) -> np.ndarray:
    """``sizes[o] = #{t : M[o,t] != -1}``
    (csrc/minuet/cuda/functions/scan.cu:220-290)."""
    m = np.asarray(kernel_map)
    return (m != -1).sum(axis=1).astype(m.dtype)


def stable_size_order(sizes: np.ndarray) -> np.ndarray:
    """Ascending order of the offsets by hit count
    (minuet/nn/convolutions.py:157-161).  The reference calls an UNSTABLE
    device sort, so its tie order is not a function of the input; the stable
    order is the canonical choice made here."""
    return np.argsort(np.asarray(sizes), kind="stable").astype(np.int64)


def compute_kernel_map_masks(num_sources: int, kernel_map: np.ndarray,
                             sizes: Optional[np.ndarray] = None):
    """Rank tables (csrc/minuet/cuda/functions/scan.cu:292-365 and
    kernels/generate_masks_from_kernel_map.cuh:20-29): hits are enumerated
    row-major (offset, then target); the rank of a hit is its position minus
    the number of hits of earlier offsets.  ``source_masks[o, M[o,t]] = rank``
    and ``target_masks[o, t] = rank``; everything else is -1."""
    m = np.asarray(kernel_map)
    num_o, num_t = m.shape
    hit = m != -1
    rank = np.cumsum(hit, axis=1) - 1
    tmask = np.where(hit, rank, -1).astype(m.dtype)
    smask = np.full((num_o, num_sources), -1, dtype=m.dtype)
    oo, tt = np.nonzero(hit)
    smask[oo, m[oo, tt]] = rank[oo, tt]
    return smask, tmask


def kernel_map_pair_lists(kernel_map: np.ndarray):
    """Per-offset (in_idx, out_idx) lists in rank order — the inverse of the
    two mask tables.  Returns ``(in_idx[nnz], out_idx[nnz], sizes[O])`` with the
    offsets concatenated in row order of ``kernel_map``."""
    m = np.asarray(kernel_map)
    oo, tt = np.nonzero(m != -1)
    return (m[oo, tt].astype(np.int32), tt.astype(np.int32),
            (m != -1).sum(axis=1).astype(np.int64))


def generate_padding_buckets(sizes: Sequence[int], threshold: Optional[float]):
    """Greedy grouping of size-ascending offsets into GEMM batches
    (csrc/minuet/cuda/functions/sparse_convolution.cu:16-43).

    A bucket is extended while ``(max*count - sum)/sum <= threshold``;
    ``threshold < 0`` gives singletons, ``None`` one bucket.  With ``sum == 0``
    the reference's ratio is 0/0 = NaN, which compares false against the
    threshold, so empty offsets are always merged; that is kept explicit here.
    """
    sizes = [int(v) for v in sizes]
    n = len(sizes)
    buckets = [0]
    i = 0
    while i < n:
        j = i
        actual = sizes[i]
        summit = sizes[i]
        while i + 1 < n:
            actual += sizes[i + 1]
            summit = max(summit, sizes[i + 1])
            padded = summit * ((i + 1) - j + 1)
            if threshold is not None:
                if threshold < 0:
                    break
                if actual > 0 and (padded - actual) / actual > threshold:
                    break
            i += 1
        buckets.append(i + 1)
        i += 1
    return buckets


def cumsum_kernel_padded_sizes(sizes: Sequence[int], buckets: Sequence[int]):
    """Every offset of a bucket gets ``max size in the bucket`` rows; prefix sum
    (csrc/minuet/cuda/functions/sparse_convolution.cu:272-292)."""
    sizes = [int(v) for v in sizes]
    cum = [0] * (len(sizes) + 1)
    for b in range(len(buckets) - 1):
        lo, hi = buckets[b], buckets[b + 1]
        summit = max(sizes[lo:hi]) if hi > lo else 0
        for j in range(lo, hi):
            cum[j + 1] = cum[j] + summit
    return cum


def sparse_convolution_forward(sources: np.ndarray, weights: np.ndarray,
                               source_masks: np.ndarray, target_masks: np.ndarray,
                               kernel_map_order: Optional[np.ndarray],
                               kernel_map_sizes: np.ndarray,
                               acc_dtype=np.float64) -> np.ndarray:
    """Gather -> per-offset GEMM -> target-stationary scatter
    (csrc/minuet/cuda/functions/sparse_convolution.cu:504-661;
    kernels/padded_gather_warp_optimized.cuh:43-59,
    kernels/padded_scatter_warp_optimized.cuh:33-52).

    ``buf[rank] = F[s]`` for ``source_masks[o,s] = rank``;
    ``cbuf = buf @ W[order[o]]``; ``out[t] += cbuf[target_masks[o,t]]`` with the
    offsets visited in row order.  The centre-offset shortcut of the reference
    adds the same term, so it is not a separate case here."""
    f = np.asarray(sources).astype(acc_dtype)
    w = np.asarray(weights).astype(acc_dtype)
    sm = np.asarray(source_masks)
    tm = np.asarray(target_masks)
    num_o, num_t = tm.shape
    out = np.zeros((num_t, w.shape[2]), dtype=acc_dtype)
    for o in range(num_o):
        size = int(kernel_map_sizes[o])
        if size == 0:
            continue
        wo = w[int(kernel_map_order[o])] if kernel_map_order is not None else w[o]
        src = np.nonzero(sm[o] != -1)[0]
        buf = np.zeros((size, f.shape[1]), dtype=acc_dtype)
        buf[sm[o, src]] = f[src]
        cbuf = buf @ wo
        tgt = np.nonzero(tm[o] != -1)[0]
        out[tgt] += cbuf[tm[o, tgt]]
    return out


def build_kernel_map(source_coords, source_batch_dims, target_coords,
                     target_batch_dims, offsets, reorder: bool = True,
                     index_dtype=np.int32):
    """What ``KernelMapCache.get_kernel_map`` computes on a miss
    (minuet/nn/convolutions.py:147-170) with the stable tie order."""
    m = query_sorted_index_with_offsets(source_coords, target_coords, offsets,
                                        source_batch_dims, target_batch_dims,
                                        dtype=index_dtype)
    sizes = compute_kernel_map_sizes(m)
    order = None
    if reorder:
        order = stable_size_order(sizes)
        sizes = sizes[order]
        m = m[order]
        order = order.astype(sizes.dtype)
    smask, tmask = compute_kernel_map_masks(source_coords.shape[0], m, sizes)
    return smask, tmask, order, sizes, m


def conv_layer(coords, batch_dims, feats, weights, kernel_size, stride=1,
               dilation=1, source_stride=1, transposed_from=None, bias=None,
               acc_dtype=np.float64):
    """One ``SparseConv.forward`` (minuet/nn/convolutions.py:446-499) for the
    non-transposed case, or — when ``transposed_from=(fine_coords,
    fine_batch_dims, fine_stride)`` — the transposed layer that reuses the
    kernel map of the matching forward layer with the two mask tables
    swapped (convolutions.py:123-140).  Returns ``(out_feats, out_coords,
    out_batch_dims, out_stride)``."""
    coords = np.asarray(coords)
    ndim = coords.shape[1]
    ks = as_tuple(kernel_size, ndim)
    st = as_tuple(stride, ndim)
    dl = as_tuple(dilation, ndim)
    ss = as_tuple(source_stride, ndim)
    if all(k == 1 for k in ks) and all(s == 1 for s in st) and all(d == 1 for d in dl):
        out = np.asarray(feats).astype(acc_dtype) @ np.asarray(weights).astype(acc_dtype)[0]
        if bias is not None:
            out = out + np.asarray(bias).astype(acc_dtype)
        return out, coords, batch_dims, ss
    if transposed_from is None:
        ts = tuple(a * b for a, b in zip(ss, st))
        if ts == ss:
            tc, tbd = coords, batch_dims
        else:
            tc, tbd = target_coordinates(coords, batch_dims, ts)
        offsets = generate_kernel_offsets(ndim, ks, ss, dl)
        smask, tmask, order, sizes, _ = build_kernel_map(coords, batch_dims, tc, tbd, offsets)
        out = sparse_convolution_forward(feats, weights, smask, tmask, order, sizes, acc_dtype)
        out_c, out_bd, out_s = tc, tbd, ts
    else:
        fc, fbd, fs = transposed_from
        fs = as_tuple(fs, ndim)
        offsets = generate_kernel_offsets(ndim, ks, fs, dl)
        smask, tmask, order, sizes, _ = build_kernel_map(fc, fbd, coords, batch_dims, offsets)
        out = sparse_convolution_forward(feats, weights, tmask, smask, order, sizes, acc_dtype)
        out_c, out_bd, out_s = np.asarray(fc), fbd, fs
    if bias is not None:
        out = out + np.asarray(bias).astype(acc_dtype)
    return out, out_c, out_bd, out_s
