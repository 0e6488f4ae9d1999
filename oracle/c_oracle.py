"""ctypes loader of the plain-C oracle (test infrastructure, see oracle_c.c)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_build", "liboracle_c.so")
_lib = None

_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_i64p = np.ctypeslib.ndpointer(dtype=np.int64, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")


def build():
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            build()
        lib = ctypes.CDLL(_PATH)
        i64, vp = ctypes.c_int64, ctypes.c_void_p
        lib.orc_num_threads.restype = ctypes.c_int
        lib.orc_arg_sort.restype = ctypes.c_int
        lib.orc_arg_sort.argtypes = [_i32p, i64, ctypes.c_int, _i64p, vp]
        lib.orc_query.restype = ctypes.c_int
        lib.orc_query.argtypes = [_i32p, i64, _i32p, i64, _i32p, i64, ctypes.c_int, _i32p]
        lib.orc_sizes.restype = None
        lib.orc_sizes.argtypes = [_i32p, i64, i64, _i64p]
        lib.orc_masks.restype = None
        lib.orc_masks.argtypes = [_i32p, i64, i64, i64, vp, _i32p, _i32p]
        lib.orc_pair_lists.restype = i64
        lib.orc_pair_lists.argtypes = [_i32p, i64, i64, _i32p, _i32p]
        lib.orc_conv_forward.restype = None
        lib.orc_conv_forward.argtypes = [_f32p, _f32p, _i32p, _i32p, vp, _i64p, i64, i64, i64, i64,
                                         i64, _f32p]
        _lib = lib
    return _lib


def num_threads():
    return int(load().orc_num_threads())


def arg_sort(coords):
    coords = np.ascontiguousarray(coords, dtype=np.int32)
    n, ndim = coords.shape
    idx = np.empty(n, dtype=np.int64)
    out = np.empty_like(coords)
    if load().orc_arg_sort(coords, n, ndim, idx, out.ctypes.data_as(ctypes.c_void_p)):
        raise ValueError("coordinate range does not fit a 64-bit key")
    return idx, out


def query(sources, targets, offsets):
    sources = np.ascontiguousarray(sources, dtype=np.int32)
    targets = np.ascontiguousarray(targets, dtype=np.int32)
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    out = np.empty((offsets.shape[0], targets.shape[0]), dtype=np.int32)
    if load().orc_query(sources, sources.shape[0], targets, targets.shape[0], offsets,
                        offsets.shape[0], sources.shape[1], out):
        raise ValueError("coordinate range does not fit a 64-bit key")
    return out


def sizes(kernel_map):
    out = np.empty(kernel_map.shape[0], dtype=np.int64)
    load().orc_sizes(kernel_map, kernel_map.shape[0], kernel_map.shape[1], out)
    return out


def masks(kernel_map, num_sources, order=None):
    num_o, num_t = kernel_map.shape
    sm = np.empty((num_o, num_sources), dtype=np.int32)
    tm = np.empty((num_o, num_t), dtype=np.int32)
    order_arr = None if order is None else np.ascontiguousarray(order, dtype=np.int64)
    load().orc_masks(kernel_map, num_o, num_sources, num_t,
                     None if order_arr is None else order_arr.ctypes.data_as(ctypes.c_void_p),
                     sm, tm)
    return sm, tm


def pair_lists(kernel_map):
    cap = int((kernel_map != -1).sum())
    a = np.empty(cap, dtype=np.int32)
    b = np.empty(cap, dtype=np.int32)
    n = load().orc_pair_lists(kernel_map, kernel_map.shape[0], kernel_map.shape[1], a, b)
    assert n == cap
    return a, b


def map_step(coords, offsets):
    """The benchmarked Map step on the CPU: unsorted unique voxels -> sorted
    coordinates, dense map, sizes and per-offset pair lists."""
    idx, sorted_coords = arg_sort(coords)
    m = query(sorted_coords, sorted_coords, offsets)
    sz = sizes(m)
    a, b = pair_lists(m)
    return idx, sorted_coords, m, sz, a, b


def conv_forward(features, weights, source_masks, target_masks, order, sizes_):
    features = np.ascontiguousarray(features, dtype=np.float32)
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    num_o, num_s = source_masks.shape
    num_t = target_masks.shape[1]
    out = np.empty((num_t, weights.shape[2]), dtype=np.float32)
    order_arr = None if order is None else np.ascontiguousarray(order, dtype=np.int64)
    load().orc_conv_forward(features, weights, np.ascontiguousarray(source_masks, dtype=np.int32),
                            np.ascontiguousarray(target_masks, dtype=np.int32),
                            None if order_arr is None else order_arr.ctypes.data_as(ctypes.c_void_p),
                            np.ascontiguousarray(sizes_, dtype=np.int64), num_s, num_t, num_o,
                            features.shape[1], weights.shape[2], out)
    return out
