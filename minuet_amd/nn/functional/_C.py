"""Bridge between torch tensors and libminuet_hip.so (ctypes, C ABI).

Mirrors the function table of the reference's pybind module
``minuet.nn.functional._C`` (registered with MINUET_TORCH_REGISTER in
csrc/minuet/torch/*.cu): same names, same argument order, same result shapes
and dtypes, same validation.  Every function here allocates its outputs with
torch, hands raw device pointers plus torch's current stream to the library
and raises ``RuntimeError`` with the library's message when a call fails.
There is no CPU or eager fallback: without the built library nothing works.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

_LIB_PATH = os.environ.get("MINUET_AMD_LIBRARY") or os.path.join(
    os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))), "lib",
    "libminuet_hip.so")
_lib = None

_INT = {torch.int32: 0, torch.int64: 1}
_FLOAT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

_c = ctypes
_vp, _i64, _int, _dbl, _sz = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_double, _c.c_size_t
_pi64 = _c.POINTER(_c.c_int64)
_pf = _c.POINTER(_c.c_float)

# name -> (restype, argtypes); the single place that states the ABI on the
# Python side.  tests/test_abi.py checks it against include/minuet_hip.h.
SIGNATURES = {
    "mnt_abi_version": (_int, []),
    "mnt_last_error": (_c.c_char_p, []),
    "mnt_buffer_preallocate": (_int, [_vp, _sz]),
    "mnt_buffer_free": (_int, [_vp]),
    "mnt_buffer_set_growth": (_int, [_vp, _c.c_float]),
    "mnt_buffer_set_page_size": (_int, [_vp, _sz]),
    "mnt_buffer_total_size": (_sz, [_vp]),
    "mnt_buffer_used_size": (_sz, [_vp]),
    "mnt_reset_error": (_int, []),
    "mnt_device_reset": (_int, []),
    "mnt_stream_acquire": (_int, [_vp]),
    "mnt_stream_release": (_int, [_vp]),
    "mnt_host_wait_stats": (_int, [_pi64, _pi64, _int]),
    "mnt_lookahead_start": (_int, [_vp, _i64, _int, _int, _vp, _i64, _int, _pi64, _vp, _int, _int, _pi64,
                                   _vp, _vp]),
    "mnt_lookahead_wait": (_int, [_int, _vp, _pi64]),
    "mnt_lookahead_finish": (_int, [_vp]),
    "mnt_arg_sort_coordinates": (_int, [_vp, _i64, _int, _int, _vp, _i64, _int, _vp, _vp, _pi64, _vp]),
    "mnt_unique_coordinates": (_int, [_vp, _i64, _int, _int, _vp, _i64, _int, _vp, _pi64, _vp]),
    "mnt_fill_unique_coordinates": (_int, [_vp, _i64, _int, _int, _vp, _int, _vp, _vp]),
    "mnt_target_coordinates_count": (_int, [_vp, _i64, _int, _int, _pi64, _vp, _i64, _int, _pi64, _pi64,
                                            _vp]),
    "mnt_target_coordinates_fill": (_int, [_vp, _vp, _vp]),
    "mnt_target_coordinates": (_int, [_vp, _i64, _int, _int, _pi64, _vp, _i64, _int, _pi64, _vp, _i64,
                                      _vp, _pi64, _vp]),
    "mnt_query_sorted_index_with_offsets": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _int, _int,
                                                   _vp, _vp, _i64, _int, _vp, _int, _vp]),
    "mnt_compute_kernel_map_sizes": (_int, [_vp, _i64, _i64, _int, _vp, _vp]),
    "mnt_compute_kernel_map_sizes_static": (_int, [_vp, _i64, _i64, _int, _vp, _vp]),
    "mnt_compute_kernel_map_masks": (_int, [_vp, _i64, _i64, _i64, _int, _vp, _vp, _vp]),
    "mnt_kernel_map_query": (_int, [_vp, _i64, _vp, _i64, _pi64, _i64, _int, _int, _vp, _vp, _i64,
                                    _int, _int, _pi64, _pi64, _pi64, _vp, _pi64, _pi64, _vp]),
    "mnt_kernel_map_emit": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mnt_kernel_map_build": (_int, [_vp, _i64, _vp, _i64, _pi64, _i64, _int, _int, _vp, _vp, _i64,
                                    _int, _int, _pi64, _pi64, _pi64, _vp, _vp, _vp, _vp, _vp, _i64,
                                    _vp, _vp, _pi64, _pi64, _vp]),
    "mnt_kernel_map_lists": (_int, [_vp, _i64, _vp, _i64, _pi64, _i64, _int, _int, _vp, _vp, _i64,
                                    _int, _int, _pi64, _pi64, _pi64, _vp, _vp, _i64, _vp, _vp, _pi64,
                                    _pi64, _vp]),
    # host arrays are passed as plain addresses here (the call sits on a hot path)
    "mnt_sorted_kernel_map_lists": (_int, [_vp, _i64, _int, _int, _vp, _i64, _int, _vp, _vp, _vp, _vp,
                                           _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mnt_kernel_map_row_lists": (_int, [_vp, _i64, _i64, _pi64, _pi64, _vp, _vp, _vp]),
    "mnt_kernel_map_dense": (_int, [_vp, _i64, _vp, _i64, _vp, _i64, _int, _int, _vp, _vp, _i64, _int,
                                    _vp, _vp, _vp, _vp, _vp]),
    "mnt_kernel_map_tables": (_int, [_vp, _i64, _i64, _i64, _int, _pi64, _pi64, _vp]),
    "mnt_kernel_map_pair_lists": (_int, [_vp, _i64, _i64, _pi64, _vp, _vp, _vp]),
    "mnt_generate_padding_buckets": (_int, [_pi64, _i64, _int, _dbl, _pi64, _pi64]),
    "mnt_cumsum_kernel_padded_sizes": (_int, [_pi64, _i64, _pi64, _i64, _pi64]),
    "mnt_sparse_convolution_forward": (_int, [_i64, _i64, _int, _i64, _int, _dbl, _vp, _vp, _vp, _vp,
                                              _vp, _vp, _pi64, _i64, _i64, _i64, _i64, _i64, _int,
                                              _int, _vp, _vp, _vp]),
    "mnt_sparse_convolution_forward_fused": (_int, [_i64, _i64, _int, _i64, _int, _dbl, _vp, _vp, _vp,
                                                    _vp, _vp, _vp, _pi64, _i64, _i64, _i64, _i64,
                                                    _i64, _int, _int, _vp, _vp, _vp, _vp, _int,
                                                    _c.c_float, _vp, _pi64, _vp, _vp]),
    "mnt_sparse_convolution_forward_rows": (_int, [_i64, _vp, _vp, _pi64, _pi64, _vp, _vp, _vp, _i64, _i64,
                                                   _i64, _i64, _i64, _int, _vp, _vp, _vp, _int, _c.c_float,
                                                   _vp, _vp, _vp]),
    "mnt_kernel_map_offset_groups": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "mnt_sparse_convolution_forward_groups": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int,
                                                     _vp, _vp, _vp, _int, _c.c_float, _vp, _vp]),
    "mnt_pack_weights": (_int, [_vp, _i64, _i64, _i64, _int, _vp, _vp]),
    "mnt_sparse_convolution_forward_implicit": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                                       _int, _vp, _vp, _vp, _int, _c.c_float, _vp,
                                                       _vp, _vp]),
    "mnt_kernel_map_invert": (_int, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "mnt_time_gather": (_int, [_i64, _int, _int, _dbl, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int,
                               _int, _pf, _vp]),
    "mnt_time_scatter": (_int, [_i64, _int, _int, _dbl, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int,
                                _int, _pf, _vp]),
    "mnt_time_gemm": (_int, [_int, _i64, _int, _dbl, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int,
                             _int, _pf, _vp]),
    "mnt_time_memory": (_int, [_int, _sz, _int, _pf, _vp]),
    "mnt_device_facts": (_int, [_pi64, _int]),
    "mnt_timer_repeats": (_int, [_int]),
    "mnt_profile_enable": (_int, [_int]),
    "mnt_profile_read": (_int, [_int, _pf, _c.c_char_p, _int, _c.POINTER(_c.c_int)]),
}


def library_path() -> str:
    return _LIB_PATH


def load_library():
    """Load (once) the HIP library; build it first only when no build exists."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        from minuet_amd.build import build_library
        build_library(verbose=False)
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    # a look-ahead session still running when the interpreter goes down would have
    # the library's worker thread inside the GPU runtime while that is torn down
    import atexit
    atexit.register(lambda: lib.mnt_lookahead_finish(None))
    return lib


def _check(status: int):
    if status != 0:
        message = load_library().mnt_last_error().decode("utf-8", "replace")
        raise RuntimeError(message or f"[Minuet] native call failed with status {status}")


def _fail(message: str):
    raise RuntimeError(f"[Minuet] {message}")


def _ptr(tensor: Optional[torch.Tensor]):
    """Device address as a plain int (what a ``c_void_p`` parameter accepts),
    None for a missing or empty tensor's null pointer."""
    if tensor is None:
        return None
    return tensor.data_ptr() or None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device: torch.device):
    """Handle of torch's current stream on ``device`` (an int; 0 / None is the
    default stream)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index) or None
    return torch.cuda.current_stream(device).cuda_stream or None


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on(device: torch.device):
    """Context that makes ``device`` current; free when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _ensure_ndim(name: str, tensor: torch.Tensor, ndim: int):
    if tensor.dim() != ndim:
        _fail(f"Tensor {name} is expected to have {ndim} dimension(s) but found "
              f"{tensor.dim()} dimension(s)")


def _ensure_dim(name: str, tensor: torch.Tensor, dim: int, size: int):
    if tensor.size(dim) != size:
        _fail(f"The dimension {dim} of Tensor {name} is expected to be {size} but found "
              f"{tensor.size(dim)}")


def _common_device(tensors: Sequence[torch.Tensor]) -> torch.device:
    device = tensors[0].device
    for t in tensors:
        if t.device != device:
            _fail(f"Found tensors on two different device ({device} != {t.device})")
    if device.type != "cuda":
        _fail(f"tensors must live on a GPU but found device {device}")
    return device


def _common_dtype(tensors: Sequence[torch.Tensor]) -> torch.dtype:
    dtype = tensors[0].dtype
    for t in tensors:
        if t.dtype != dtype:
            _fail(f"Found tensors with two different scalar types ({dtype} != {t.dtype})")
    return dtype


def _int_code(dtype: torch.dtype, what: str, fn: str) -> int:
    if dtype not in _INT:
        _fail(f"Cannot find implementation of {fn} for {what} data type {dtype}")
    return _INT[dtype]


def _float_code(dtype: torch.dtype, fn: str) -> int:
    if dtype not in _FLOAT:
        _fail(f"Cannot find implementation of {fn} for feature data type {dtype}")
    return _FLOAT[dtype]


def _check_ndim_supported(ndim: int, fn: str, dtype):
    if not 1 <= ndim <= 4:
        _fail(f"Cannot find implementation of {fn} for coordinate data type {dtype} of with ndim={ndim}")


# ----------------------------------------------------------------- sorting ----

def cuda_arg_sort_coordinates(coordinates: torch.Tensor, enable_flattening: bool = True) -> torch.Tensor:
    """csrc/minuet/torch/cuda_arg_sort_coordinates.cu:8-34.  ``enable_flattening``
    only selects an algorithm in the reference; the result is the same either way."""
    _ensure_ndim("coordinates", coordinates, 2)
    device = _common_device([coordinates])
    n, ndim = coordinates.shape
    ccode = _int_code(coordinates.dtype, "coordinate", "CUDAArgSortCoordinates")
    _check_ndim_supported(ndim, "CUDAArgSortCoordinates", coordinates.dtype)
    itype = torch.int32 if n <= 2 ** 31 - 1 else torch.int64
    indices = torch.empty((n,), dtype=itype, device=device)
    with _on(device):
        _check(load_library().mnt_arg_sort_coordinates(
            _ptr(coordinates), n, ndim, ccode, None, 1, _INT[itype], _ptr(indices), None, None,
            _stream(device)))
    return indices


def cuda_multi_arg_sort_coordinates(coordinates: torch.Tensor, batch_dims: torch.Tensor,
                                    enable_flattening: bool = True) -> torch.Tensor:
    """csrc/minuet/torch/cuda_arg_sort_coordinates.cu:36-66."""
    _ensure_ndim("coordinates", coordinates, 2)
    _ensure_ndim("batch_dims", batch_dims, 1)
    device = _common_device([coordinates, batch_dims])
    n, ndim = coordinates.shape
    ccode = _int_code(coordinates.dtype, "coordinate", "CUDAMultiArgSortCoordinates")
    icode = _int_code(batch_dims.dtype, "index", "CUDAMultiArgSortCoordinates")
    _check_ndim_supported(ndim, "CUDAMultiArgSortCoordinates", coordinates.dtype)
    indices = torch.empty((n,), dtype=batch_dims.dtype, device=device)
    with _on(device):
        _check(load_library().mnt_arg_sort_coordinates(
            _ptr(coordinates), n, ndim, ccode, _ptr(batch_dims), batch_dims.numel() - 1, icode,
            _ptr(indices), None, None, _stream(device)))
    return indices


def sort_coordinates(coordinates: torch.Tensor, batch_dims: Optional[torch.Tensor] = None,
                     return_bounds: bool = False):
    """Arg-sort and the sorted rows in one library call (int32 indices unless
    ``batch_dims`` says otherwise).  With ``return_bounds`` a third result holds
    the per-dimension coordinate minima [0..3] and maxima [4..7] (numpy int64),
    which ``kernel_map_build`` accepts to skip its own reduction."""
    _ensure_ndim("coordinates", coordinates, 2)
    device = _common_device([coordinates] + ([batch_dims] if batch_dims is not None else []))
    n, ndim = coordinates.shape
    ccode = _int_code(coordinates.dtype, "coordinate", "sort_coordinates")
    itype = batch_dims.dtype if batch_dims is not None else torch.int32
    indices = torch.empty((n,), dtype=itype, device=device)
    out = torch.empty_like(coordinates)
    bounds = np.zeros(8, dtype=np.int64)
    with _on(device):
        _check(load_library().mnt_arg_sort_coordinates(
            _ptr(coordinates), n, ndim, ccode, _ptr(batch_dims),
            batch_dims.numel() - 1 if batch_dims is not None else 1, _INT[itype], _ptr(indices),
            _ptr(out), bounds.ctypes.data_as(_pi64), _stream(device)))
    if return_bounds:
        return indices, out, bounds
    return indices, out


# ------------------------------------------------------------------ unique ----

def _unique(coordinates: torch.Tensor, batch_dims: Optional[torch.Tensor], fn: str):
    _ensure_ndim("coordinates", coordinates, 2)
    if batch_dims is not None:
        _ensure_ndim("batch_dims", batch_dims, 1)
    device = _common_device([coordinates] + ([batch_dims] if batch_dims is not None else []))
    n, ndim = coordinates.shape
    ccode = _int_code(coordinates.dtype, "coordinate", fn)
    _check_ndim_supported(ndim, fn, coordinates.dtype)
    itype = torch.int64 if batch_dims is None else batch_dims.dtype
    icode = _int_code(itype, "index", fn)
    indices = torch.empty((n + 1,), dtype=itype, device=device)
    count = ctypes.c_int64(0)
    lib = load_library()
    with _on(device):
        # the reference passes len(batch_dims) as the batch count
        # (cuda_unique_coordinates.cu:51); results are the same with B
        _check(lib.mnt_unique_coordinates(
            _ptr(coordinates), n, ndim, ccode, _ptr(batch_dims),
            batch_dims.numel() - 1 if batch_dims is not None else 1, icode, _ptr(indices),
            ctypes.byref(count), _stream(device)))
        targets = torch.empty((count.value, ndim), dtype=coordinates.dtype, device=device)
        _check(lib.mnt_fill_unique_coordinates(
            _ptr(coordinates), n, ndim, ccode, _ptr(indices), icode, _ptr(targets), _stream(device)))
    return targets, indices


def cuda_unique_coordinates(coordinates: torch.Tensor):
    """csrc/minuet/torch/cuda_unique_coordinates.cu:8-43 -> (unique rows, idx[N+1] int64)."""
    return _unique(coordinates, None, "CUDAUniqueCoordinates")


def cuda_multi_unique_coordinates(coordinates: torch.Tensor, batch_dims: torch.Tensor):
    """csrc/minuet/torch/cuda_unique_coordinates.cu:45-81 -> (unique rows, idx[N+1])."""
    return _unique(coordinates, batch_dims, "CUDAMultiUniqueCoordinates")


def target_coordinates(coordinates: torch.Tensor, batch_dims: Optional[torch.Tensor],
                       target_stride: Sequence[int], source_bounds=None):
    """floor(c / stride) * stride, sorted and unique, plus the new batch
    boundaries — the tensor expression of minuet/nn/convolutions.py:84-99 as two
    library calls.  ``source_bounds`` (8 int64: per-dimension minima, then
    maxima of ``coordinates``) spares their reduction on the device."""
    _ensure_ndim("coordinates", coordinates, 2)
    if batch_dims is not None and batch_dims.numel() <= 2:
        # one cloud carrying its boundaries: the library runs it as unbatched and
        # writes no boundaries, so they are put together here
        # (minuet/nn/convolutions.py:92-96 returns [0, count] for it)
        out, _ = target_coordinates(coordinates, None, target_stride, source_bounds)
        ends = [0, out.shape[0]][:batch_dims.numel()]
        return out, torch.tensor(ends, dtype=batch_dims.dtype, device=batch_dims.device)
    known = None if source_bounds is None else np.ascontiguousarray(source_bounds, dtype=np.int64)
    device = _common_device([coordinates] + ([batch_dims] if batch_dims is not None else []))
    n, ndim = coordinates.shape
    ccode = _int_code(coordinates.dtype, "coordinate", "target_coordinates")
    itype = batch_dims.dtype if batch_dims is not None else torch.int32
    icode = _int_code(itype, "index", "target_coordinates")
    stride = (ctypes.c_int64 * ndim)(*[int(s) for s in target_stride])
    count = ctypes.c_int64(0)
    lib = load_library()
    num_batches = batch_dims.numel() - 1 if batch_dims is not None else 1
    known_arg = None if known is None else known.ctypes.data_as(_pi64)
    if n > 0:
        # room for the worst case (no two sources share a target): the rows are
        # written while the host waits for their number, in one call
        with _on(device):
            room = torch.empty((n, ndim), dtype=coordinates.dtype, device=device)
            out_dims = torch.empty_like(batch_dims) if batch_dims is not None else None
            _check(lib.mnt_target_coordinates(
                _ptr(coordinates), n, ndim, ccode, stride, _ptr(batch_dims), num_batches, icode,
                known_arg, _ptr(room), n, _ptr(out_dims), ctypes.byref(count), _stream(device)))
        return room[:count.value], out_dims
    with _on(device):
        _check(lib.mnt_target_coordinates_count(
            _ptr(coordinates), n, ndim, ccode, stride, _ptr(batch_dims),
            batch_dims.numel() - 1 if batch_dims is not None else 1, icode,
            None if known is None else known.ctypes.data_as(_pi64), ctypes.byref(count),
            _stream(device)))
        out = torch.empty((count.value, ndim), dtype=coordinates.dtype, device=device)
        out_dims = torch.empty_like(batch_dims) if batch_dims is not None else None
        _check(lib.mnt_target_coordinates_fill(_ptr(out), _ptr(out_dims), _stream(device)))
    return out, out_dims


# ------------------------------------------------------------------- query ----

def cuda_query_sorted_index_with_offsets(sources: torch.Tensor, targets: torch.Tensor,
                                         offsets: torch.Tensor) -> torch.Tensor:
    """csrc/minuet/torch/cuda_sparse_convolution_mapping.cu:9-47 -> M[O,T] of the
    coordinate dtype."""
    fn = "CUDAQuerySortedIndexWithOffsets"
    _ensure_ndim("sources", sources, 2)
    _ensure_ndim("targets", targets, 2)
    _ensure_ndim("offsets", offsets, 2)
    ndim = offsets.size(1)
    _ensure_dim("sources", sources, 1, ndim)
    _ensure_dim("targets", targets, 1, ndim)
    ctype = _common_dtype([sources, targets, offsets])
    device = _common_device([sources, targets, offsets])
    ccode = _int_code(ctype, "coordinate", fn)
    _check_ndim_supported(ndim, fn, ctype)
    out = torch.empty((offsets.size(0), targets.size(0)), dtype=ctype, device=device)
    with _on(device):
        _check(load_library().mnt_query_sorted_index_with_offsets(
            _ptr(sources), sources.size(0), _ptr(targets), targets.size(0), _ptr(offsets),
            offsets.size(0), ndim, ccode, None, None, 1, 0, _ptr(out), ccode, _stream(device)))
    return out


def cuda_multi_query_sorted_index_with_offsets(source_batch_dims: torch.Tensor,
                                               target_batch_dims: torch.Tensor,
                                               sources: torch.Tensor, targets: torch.Tensor,
                                               offsets: torch.Tensor) -> torch.Tensor:
    """csrc/minuet/torch/cuda_sparse_convolution_mapping.cu:49-93 -> M[O,T] of the
    batch_dims dtype."""
    fn = "CUDAMultiQuerySortedIndexWithOffsets"
    _ensure_ndim("sources", sources, 2)
    _ensure_ndim("targets", targets, 2)
    _ensure_ndim("offsets", offsets, 2)
    _ensure_ndim("source_batch_dims", source_batch_dims, 1)
    _ensure_ndim("target_batch_dims", target_batch_dims, 1)
    ndim = offsets.size(1)
    _ensure_dim("sources", sources, 1, ndim)
    _ensure_dim("targets", targets, 1, ndim)
    ctype = _common_dtype([sources, targets, offsets])
    itype = _common_dtype([source_batch_dims, target_batch_dims])
    if source_batch_dims.size(0) <= 1:
        _fail(f"Tensor source_batch_dims should be at least length 2 but found "
              f"{source_batch_dims.size(0)} <= 1")
    if target_batch_dims.size(0) != source_batch_dims.size(0):
        _fail(f"Tensor target_batch_dims must have the same length as source_batch_dims but found "
              f"{target_batch_dims.size(0)} != {source_batch_dims.size(0)}")
    device = _common_device([sources, targets, offsets, source_batch_dims, target_batch_dims])
    ccode = _int_code(ctype, "coordinate", fn)
    icode = _int_code(itype, "index", fn)
    _check_ndim_supported(ndim, fn, ctype)
    out = torch.empty((offsets.size(0), targets.size(0)), dtype=itype, device=device)
    with _on(device):
        _check(load_library().mnt_query_sorted_index_with_offsets(
            _ptr(sources), sources.size(0), _ptr(targets), targets.size(0), _ptr(offsets),
            offsets.size(0), ndim, ccode, _ptr(source_batch_dims), _ptr(target_batch_dims),
            source_batch_dims.size(0) - 1, icode, _ptr(out), icode, _stream(device)))
    return out


def cuda_compute_kernel_map_sizes(kernel_map: torch.Tensor) -> torch.Tensor:
    """csrc/minuet/torch/cuda_sparse_convolution_mapping.cu:95-121."""
    _ensure_ndim("kernel_map", kernel_map, 2)
    device = _common_device([kernel_map])
    icode = _int_code(kernel_map.dtype, "tensor", "CUDAComputeKernelMapSizes")
    sizes = torch.empty((kernel_map.size(0),), dtype=kernel_map.dtype, device=device)
    with _on(device):
        _check(load_library().mnt_compute_kernel_map_sizes(
            _ptr(kernel_map), kernel_map.size(0), kernel_map.size(1), icode, _ptr(sizes),
            _stream(device)))
    return sizes


STATIC_SCRATCH_WORDS = 1 << 20


def compute_kernel_map_sizes_static(kernel_map: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """:func:`cuda_compute_kernel_map_sizes` through the entry point that
    allocates nothing: ``out`` ([O], dtype of ``kernel_map``) is written in
    place and the counts live in the library's static device array, so maps
    beyond ``O * (ceil(T / 512) + 1) <= STATIC_SCRATCH_WORDS`` are refused."""
    _ensure_ndim("kernel_map", kernel_map, 2)
    device = _common_device([kernel_map, out])
    icode = _int_code(_common_dtype([kernel_map, out]), "tensor", "compute_kernel_map_sizes_static")
    if not kernel_map.is_contiguous() or not out.is_contiguous() or out.numel() != kernel_map.size(0):
        _fail("compute_kernel_map_sizes_static needs contiguous tensors and one output entry per offset")
    with _on(device):
        _check(load_library().mnt_compute_kernel_map_sizes_static(
            _ptr(kernel_map), kernel_map.size(0), kernel_map.size(1), icode, _ptr(out),
            _stream(device)))
    return out


def cuda_compute_kernel_map_masks(num_sources: int, kernel_map: torch.Tensor,
                                  kernel_map_sizes: torch.Tensor):
    """csrc/minuet/torch/cuda_sparse_convolution_mapping.cu:123-156.  The ranks are
    recomputed from ``kernel_map``; ``kernel_map_sizes`` is only validated."""
    _ensure_ndim("kernel_map", kernel_map, 2)
    device = _common_device([kernel_map, kernel_map_sizes])
    icode = _int_code(kernel_map.dtype, "tensor", "CUDAComputeKernelMapMasks")
    num_offsets, num_targets = kernel_map.shape
    source_masks = torch.empty((num_offsets, num_sources), dtype=kernel_map.dtype, device=device)
    target_masks = torch.empty((num_offsets, num_targets), dtype=kernel_map.dtype, device=device)
    with _on(device):
        _check(load_library().mnt_compute_kernel_map_masks(
            _ptr(kernel_map), num_offsets, int(num_sources), num_targets, icode,
            _ptr(source_masks), _ptr(target_masks), _stream(device)))
    return source_masks, target_masks


# Pair lists are allocated for their worst case (and the call spared a launch
# after its wait) while both lists together stay below this many bytes.
PAIR_LIST_SLACK_BYTES = 256 << 20


def kernel_map_build(sources: torch.Tensor, targets: torch.Tensor, offsets_host: np.ndarray,
                     source_batch_dims: Optional[torch.Tensor],
                     target_batch_dims: Optional[torch.Tensor], reorder: bool,
                     want_masks: bool = True, want_lists: bool = False,
                     want_dense: bool = False, source_bounds=None, target_bounds=None):
    """Fused kernel-map build: query + sizes + stable size order + rank tables
    and/or per-offset pair lists.  Returns a dict with ``sizes_host``,
    ``order_host`` (numpy int64), ``sizes``/``order`` (int32 device), ``bounds``
    (numpy int64 [16]: coordinate minima / maxima of sources then targets) and
    the requested tensors (``source_masks``, ``target_masks``, ``in_idx``,
    ``out_idx``, ``kernel_map``).  ``source_bounds`` / ``target_bounds`` (8
    int64 each) skip the device-side bounds reduction when already known."""
    _ensure_ndim("sources", sources, 2)
    _ensure_ndim("targets", targets, 2)
    ndim = sources.size(1)
    _ensure_dim("targets", targets, 1, ndim)
    ctype = _common_dtype([sources, targets])
    tensors = [sources, targets]
    if (source_batch_dims is None) != (target_batch_dims is None):
        raise ValueError("source_batch_dims and target_batch_dims must be both provided or "
                         "neither provided")
    bcode = 0
    if source_batch_dims is not None:
        tensors += [source_batch_dims, target_batch_dims]
        bcode = _int_code(_common_dtype([source_batch_dims, target_batch_dims]), "index",
                          "kernel_map_build")
    device = _common_device(tensors)
    ccode = _int_code(ctype, "coordinate", "kernel_map_build")
    offs = np.ascontiguousarray(np.asarray(offsets_host, dtype=np.int64).reshape(-1, ndim))
    num_offsets = offs.shape[0]
    num_sources, num_targets = sources.size(0), targets.size(0)
    lists_only = want_lists and not want_masks and not want_dense
    dense = None if lists_only else torch.empty((num_offsets, num_targets), dtype=torch.int32, device=device)
    sizes_host = np.zeros(num_offsets, dtype=np.int64)
    order_host = np.zeros(num_offsets, dtype=np.int64)
    bounds = np.zeros(16, dtype=np.int64)
    sb = None if source_bounds is None else np.ascontiguousarray(source_bounds, dtype=np.int64)
    tb = None if target_bounds is None else np.ascontiguousarray(target_bounds, dtype=np.int64)
    lib = load_library()
    result = {}
    # everything whose size is known goes before the query: the host then has
    # less to do between the wait for the sizes and the second launch
    smask = tmask = in_idx = out_idx = None
    if want_masks:
        smask = torch.empty((num_offsets, num_sources), dtype=torch.int32, device=device)
        tmask = torch.empty((num_offsets, num_targets), dtype=torch.int32, device=device)
    sizes_dev = torch.empty((num_offsets,), dtype=torch.int32, device=device)
    order_dev = torch.empty((num_offsets,), dtype=torch.int32, device=device)
    num_batches = source_batch_dims.numel() - 1 if source_batch_dims is not None else 1
    # Pair lists whose worst case (every (offset, target) pair a hit) is small
    # are handed over before their length is known: the tables are then written
    # while the host waits for the sizes, in one call.
    capacity = num_offsets * num_targets
    one_call = (num_sources > 0 and num_targets > 0 and num_offsets > 0
                and (not want_lists or capacity * 8 <= PAIR_LIST_SLACK_BYTES))
    with _on(device):
        stream = _stream(device)
        if lists_only and not one_call:
            dense = torch.empty((num_offsets, num_targets), dtype=torch.int32, device=device)
        if one_call and lists_only:
            # the lists alone: the dense map is neither written nor read back
            both = torch.empty((2, capacity), dtype=torch.int32, device=device)
            _check(lib.mnt_kernel_map_lists(
                _ptr(sources), num_sources, _ptr(targets), num_targets,
                offs.ctypes.data_as(_pi64), num_offsets, ndim, ccode, _ptr(source_batch_dims),
                _ptr(target_batch_dims), num_batches, bcode, 1 if reorder else 0,
                None if sb is None else sb.ctypes.data_as(_pi64),
                None if tb is None else tb.ctypes.data_as(_pi64), bounds.ctypes.data_as(_pi64),
                _ptr(both[0]), _ptr(both[1]), capacity, _ptr(sizes_dev), _ptr(order_dev),
                sizes_host.ctypes.data_as(_pi64), order_host.ctypes.data_as(_pi64), stream))
            nnz = int(sizes_host.sum())
            result.update(sizes_host=sizes_host, order_host=order_host, sizes=sizes_dev, order=order_dev,
                          bounds=bounds, source_masks=None, target_masks=None, in_idx=both[0, :nnz],
                          out_idx=both[1, :nnz])
            return result
        if one_call:
            if want_lists:
                both = torch.empty((2, capacity), dtype=torch.int32, device=device)
            _check(lib.mnt_kernel_map_build(
                _ptr(sources), num_sources, _ptr(targets), num_targets,
                offs.ctypes.data_as(_pi64), num_offsets, ndim, ccode, _ptr(source_batch_dims),
                _ptr(target_batch_dims), num_batches, bcode, 1 if reorder else 0,
                None if sb is None else sb.ctypes.data_as(_pi64),
                None if tb is None else tb.ctypes.data_as(_pi64), bounds.ctypes.data_as(_pi64),
                _ptr(dense), _ptr(smask), _ptr(tmask),
                _ptr(both[0]) if want_lists else None, _ptr(both[1]) if want_lists else None, capacity,
                _ptr(sizes_dev), _ptr(order_dev), sizes_host.ctypes.data_as(_pi64),
                order_host.ctypes.data_as(_pi64), stream))
            if want_lists:
                nnz = int(sizes_host.sum())
                in_idx, out_idx = both[0, :nnz], both[1, :nnz]
            result.update(sizes_host=sizes_host, order_host=order_host, sizes=sizes_dev, order=order_dev,
                          bounds=bounds, source_masks=smask, target_masks=tmask, in_idx=in_idx,
                          out_idx=out_idx)
            if want_dense:
                result["kernel_map"] = dense
            return result
        _check(lib.mnt_kernel_map_query(
            _ptr(sources), num_sources, _ptr(targets), num_targets,
            offs.ctypes.data_as(_pi64), num_offsets, ndim, ccode, _ptr(source_batch_dims),
            _ptr(target_batch_dims), num_batches, bcode,
            1 if reorder else 0,
            None if sb is None else sb.ctypes.data_as(_pi64),
            None if tb is None else tb.ctypes.data_as(_pi64), bounds.ctypes.data_as(_pi64),
            _ptr(dense), sizes_host.ctypes.data_as(_pi64), order_host.ctypes.data_as(_pi64),
            stream))
        if want_lists:
            nnz = int(sizes_host.sum())
            both = torch.empty((2, nnz), dtype=torch.int32, device=device)
            in_idx, out_idx = both[0], both[1]
        _check(lib.mnt_kernel_map_emit(_ptr(smask), _ptr(tmask), _ptr(in_idx), _ptr(out_idx),
                                       _ptr(sizes_dev), _ptr(order_dev), stream))
    result.update(sizes_host=sizes_host, order_host=order_host, sizes=sizes_dev, order=order_dev,
                  bounds=bounds,
                  source_masks=smask, target_masks=tmask, in_idx=in_idx, out_idx=out_idx)
    if want_dense:
        result["kernel_map"] = dense
    return result


class SortedMapLists:
    """What :func:`sorted_kernel_map_lists` returns: the sorted cloud and the pair
    lists of its kernel map.  All int32 results live in one device allocation;
    the tensors handed out (``indices``, ``coordinates``, ``in_idx``, ``out_idx``,
    ``sizes``, ``order``) are views of it, made when first asked for.  Reads like
    the dict of :func:`kernel_map_build` (``built["in_idx"]``, ``"sizes_host"``,
    ``"order_host"``, ``"bounds"`` ...)."""
    __slots__ = ("_store", "_coords", "_raw_host", "_n", "_ndim", "_num_offsets", "_views")

    def __init__(self, store, coords, host, n, ndim, num_offsets):
        # host: a ctypes int64 array (bounds [8], sizes [O], order [O]) that the
        # library filled; its NumPy view is made when first asked for
        self._store, self._coords, self._raw_host = store, coords, host
        self._n, self._ndim, self._num_offsets = n, ndim, num_offsets
        self._views = {}

    @property
    def _host(self):
        host = self._views.get("_host")
        if host is None:
            host = self._views["_host"] = np.frombuffer(self._raw_host, dtype=np.int64)
        return host

    @property
    def sizes_host(self):
        return self._host[8:8 + self._num_offsets]

    @property
    def order_host(self):
        return self._host[8 + self._num_offsets:]

    @property
    def nnz(self) -> int:
        return int(self.sizes_host.sum())

    def _view(self, key):
        n, no = self._n, self._num_offsets
        cap = no * n
        lists = n if self._coords is not None else n * (1 + self._ndim)
        if key == "indices":
            return self._store[:n]
        if key == "coordinates":
            return self._coords if self._coords is not None else self._store[n:lists].view(n, self._ndim)
        if key == "in_idx":
            return self._store[lists:lists + self.nnz]
        if key == "out_idx":
            return self._store[lists + cap:lists + cap + self.nnz]
        if key == "sizes":
            return self._store[lists + 2 * cap:lists + 2 * cap + no]
        if key == "order":
            return self._store[lists + 2 * cap + no:lists + 2 * cap + 2 * no]
        if key == "sizes_host":
            return self.sizes_host
        if key == "order_host":
            return self.order_host
        if key == "bounds":
            return np.concatenate([self._host[:8], self._host[:8]])
        if key in ("source_masks", "target_masks"):
            return None
        raise KeyError(key)

    def __getitem__(self, key):
        if key not in self._views:
            self._views[key] = self._view(key)
        return self._views[key]

    def __contains__(self, key):
        return key in ("indices", "coordinates", "in_idx", "out_idx", "sizes", "order", "sizes_host",
                       "order_host", "bounds", "source_masks", "target_masks")


_ADDRESSES = {}


def _host_address(array: np.ndarray) -> int:
    """Address of a NumPy array's data, remembered per array object (asking
    NumPy for it costs a microsecond, which a call on a hot path feels)."""
    hit = _ADDRESSES.get(id(array))
    if hit is not None and hit[0] is array:
        return hit[1]
    if len(_ADDRESSES) > 64:
        _ADDRESSES.clear()
    address = array.ctypes.data
    _ADDRESSES[id(array)] = (array, address)
    return address


def sorted_kernel_map_lists(coordinates: torch.Tensor, offsets_host: np.ndarray, reorder: bool = True,
                            result_only: bool = False):
    """The Map step of a stride-1 layer on an unsorted cloud (one batch) in one
    library call: ``sort_coordinates`` then the lists-only ``kernel_map_build``
    of the sorted cloud onto itself.  Returns ``(indices int32 [n], sorted
    coordinates, built)`` with ``built`` a :class:`SortedMapLists` that reads
    like the dict :func:`kernel_map_build` returns for ``want_masks=False,
    want_lists=True`` (``bounds`` holds the 8 bounds of the cloud twice:
    sources, then targets) and also holds ``"indices"`` and ``"coordinates"``;
    ``result_only=True`` returns ``built`` alone, whose tensors are views made
    when first asked for."""
    if coordinates.dim() != 2:
        _ensure_ndim("coordinates", coordinates, 2)
    device = coordinates.device
    if device.type != "cuda":
        _common_device([coordinates])
    n, ndim = coordinates.shape
    ccode = _INT.get(coordinates.dtype)
    if ccode is None:
        _int_code(coordinates.dtype, "coordinate", "sorted_kernel_map_lists")
    if not 1 <= ndim <= 4:
        _check_ndim_supported(ndim, "sorted_kernel_map_lists", coordinates.dtype)
    offs = offsets_host
    if not (isinstance(offs, np.ndarray) and offs.dtype == np.int64 and offs.ndim == 2
            and offs.shape[1] == ndim and offs.flags.c_contiguous):
        offs = np.ascontiguousarray(np.asarray(offsets_host, dtype=np.int64).reshape(-1, ndim))
    num_offsets = offs.shape[0]
    if n == 0 or num_offsets == 0:
        indices, out = sort_coordinates(coordinates)
        built = kernel_map_build(out, out, offs, None, None, reorder, want_masks=False, want_lists=True)
        if result_only:
            built = dict(built, indices=indices, coordinates=out)
            return built
        return indices, out, built
    if not coordinates.is_contiguous():
        coordinates = coordinates.contiguous()
    capacity = num_offsets * n
    narrow = ccode == 0
    lists = n * (1 + ndim) if narrow else n
    store = torch.empty((lists + 2 * capacity + 2 * num_offsets,), dtype=torch.int32, device=device)
    coords_out = None if narrow else torch.empty_like(coordinates)
    host = (ctypes.c_int64 * (8 + 2 * num_offsets))()
    base = store.data_ptr()
    hbase = ctypes.addressof(host)
    with _on(device):
        status = load_library().mnt_sorted_kernel_map_lists(
            coordinates.data_ptr(), n, ndim, ccode, _host_address(offs), num_offsets,
            1 if reorder else 0, base, base + 4 * n if narrow else coords_out.data_ptr(),
            base + 4 * lists, base + 4 * (lists + capacity), capacity,
            base + 4 * (lists + 2 * capacity), base + 4 * (lists + 2 * capacity + num_offsets),
            hbase, hbase + 64, hbase + 64 + 8 * num_offsets, _stream(device))
    if status != 0:
        _check(status)
    built = SortedMapLists(store, coords_out, host, n, ndim, num_offsets)
    if result_only:
        return built
    return built["indices"], built["coordinates"], built


def kernel_map_dense(sources: torch.Tensor, targets: torch.Tensor, offsets_host: np.ndarray,
                     source_batch_dims: Optional[torch.Tensor],
                     target_batch_dims: Optional[torch.Tensor], source_bounds=None,
                     target_bounds=None):
    """The query alone: ``(kernel_map [O, T] int32, bounds)``.  Nothing is read
    back when both bounds are given, so the call returns without waiting for
    the device."""
    if sources.dim() != 2:
        _ensure_ndim("sources", sources, 2)
    if targets.dim() != 2:
        _ensure_ndim("targets", targets, 2)
    ndim = sources.shape[1]
    if targets.shape[1] != ndim:
        _ensure_dim("targets", targets, 1, ndim)
    ctype = sources.dtype
    if targets.dtype != ctype:
        _common_dtype([sources, targets])
    if (source_batch_dims is None) != (target_batch_dims is None):
        raise ValueError("source_batch_dims and target_batch_dims must be both provided or "
                         "neither provided")
    device = sources.device
    if device.type != "cuda" or targets.device != device:
        _common_device([sources, targets])
    bcode = 0
    num_batches = 1
    if source_batch_dims is not None:
        if source_batch_dims.device != device or target_batch_dims.device != device:
            _common_device([sources, source_batch_dims, target_batch_dims])
        bcode = _int_code(_common_dtype([source_batch_dims, target_batch_dims]), "index",
                          "kernel_map_dense")
        num_batches = source_batch_dims.numel() - 1
    ccode = _INT.get(ctype)
    if ccode is None:
        _int_code(ctype, "coordinate", "kernel_map_dense")
    offs = offsets_host
    if not (isinstance(offs, np.ndarray) and offs.dtype == np.int64 and offs.ndim == 2
            and offs.shape[1] == ndim and offs.flags.c_contiguous):
        offs = np.ascontiguousarray(np.asarray(offsets_host, dtype=np.int64).reshape(-1, ndim))
    num_offsets = offs.shape[0]
    dense = torch.empty((num_offsets, targets.shape[0]), dtype=torch.int32, device=device)
    bounds = np.zeros(16, dtype=np.int64)
    sb = None if source_bounds is None else np.ascontiguousarray(source_bounds, dtype=np.int64)
    tb = None if target_bounds is None else np.ascontiguousarray(target_bounds, dtype=np.int64)
    with _on(device):
        status = load_library().mnt_kernel_map_dense(
            _ptr(sources), sources.shape[0], _ptr(targets), targets.shape[0],
            _host_address(offs), num_offsets, ndim, ccode, _ptr(source_batch_dims),
            _ptr(target_batch_dims), num_batches, bcode,
            None if sb is None else sb.ctypes.data, None if tb is None else tb.ctypes.data,
            bounds.ctypes.data, _ptr(dense), _stream(device))
    if status != 0:
        _check(status)
    return dense, bounds


def kernel_map_tables(kernel_map: torch.Tensor, num_sources: int, reorder: bool,
                      want_lists: bool = True):
    """Sizes, stable size order, rank tables and (optionally) pair lists of a
    dense int32 kernel map made earlier by :func:`kernel_map_dense`: the rest
    of what :func:`kernel_map_build` returns."""
    _ensure_ndim("kernel_map", kernel_map, 2)
    if kernel_map.dtype != torch.int32:
        _fail("kernel_map_tables expects an int32 kernel map")
    device = _common_device([kernel_map])
    kernel_map = kernel_map.contiguous()
    num_offsets, num_targets = kernel_map.shape
    sizes_host = np.zeros(num_offsets, dtype=np.int64)
    order_host = np.zeros(num_offsets, dtype=np.int64)
    lib = load_library()
    with _on(device):
        stream = _stream(device)
        _check(lib.mnt_kernel_map_tables(_ptr(kernel_map), num_sources, num_targets, num_offsets,
                                         1 if reorder else 0, sizes_host.ctypes.data_as(_pi64),
                                         order_host.ctypes.data_as(_pi64), stream))
        smask = torch.empty((num_offsets, num_sources), dtype=torch.int32, device=device)
        tmask = torch.empty((num_offsets, num_targets), dtype=torch.int32, device=device)
        in_idx = out_idx = None
        if want_lists:
            nnz = int(sizes_host.sum())
            in_idx = torch.empty((nnz,), dtype=torch.int32, device=device)
            out_idx = torch.empty((nnz,), dtype=torch.int32, device=device)
        sizes_dev = torch.empty((num_offsets,), dtype=torch.int32, device=device)
        order_dev = torch.empty((num_offsets,), dtype=torch.int32, device=device)
        _check(lib.mnt_kernel_map_emit(_ptr(smask), _ptr(tmask), _ptr(in_idx), _ptr(out_idx),
                                       _ptr(sizes_dev), _ptr(order_dev), stream))
    return dict(sizes_host=sizes_host, order_host=order_host, sizes=sizes_dev, order=order_dev,
                source_masks=smask, target_masks=tmask, in_idx=in_idx, out_idx=out_idx,
                kernel_map=kernel_map)


MAX_ROW_LIST_OFFSETS = 1024


def kernel_map_row_lists(kernel_map: torch.Tensor, sizes_host, order_host=None):
    """``(row_ptr [T + 1], out_pos [nnz])`` (int32) of a dense int32 kernel map
    whose pair lists are numbered by ``sizes_host`` / ``order_host`` (as
    :func:`kernel_map_build` returns them): the target-major row lists that
    :func:`sparse_convolution_forward_rows` is driven by.  Waits for nothing."""
    _ensure_ndim("kernel_map", kernel_map, 2)
    device = _common_device([kernel_map])
    if kernel_map.dtype != torch.int32:
        _fail("kernel_map_row_lists expects an int32 kernel map")
    kernel_map = kernel_map.contiguous()
    num_offsets, num_targets = kernel_map.shape
    sizes = np.ascontiguousarray(sizes_host, dtype=np.int64)
    order = None if order_host is None else np.ascontiguousarray(order_host, dtype=np.int64)
    if sizes.shape[0] != num_offsets or (order is not None and order.shape[0] != num_offsets):
        _fail("sizes_host / order_host need one entry per offset")
    row_ptr = torch.empty((num_targets + 1,), dtype=torch.int32, device=device)
    out_pos = torch.empty((int(sizes.sum()),), dtype=torch.int32, device=device)
    with _on(device):
        _check(load_library().mnt_kernel_map_row_lists(
            _ptr(kernel_map), num_offsets, num_targets, sizes.ctypes.data_as(_pi64),
            None if order is None else order.ctypes.data_as(_pi64), _ptr(row_ptr), _ptr(out_pos),
            _stream(device)))
    return row_ptr, out_pos


def kernel_map_pair_lists(kernel_map: torch.Tensor, sizes_host: Sequence[int]):
    """Per-offset (in_idx, out_idx) lists of an int32 dense kernel map."""
    _ensure_ndim("kernel_map", kernel_map, 2)
    device = _common_device([kernel_map])
    if kernel_map.dtype != torch.int32:
        _fail("kernel_map_pair_lists expects an int32 kernel map")
    num_offsets, num_targets = kernel_map.shape
    cum = np.zeros(num_offsets + 1, dtype=np.int64)
    cum[1:] = np.cumsum(np.asarray(sizes_host, dtype=np.int64))
    in_idx = torch.empty((int(cum[-1]),), dtype=torch.int32, device=device)
    out_idx = torch.empty_like(in_idx)
    with _on(device):
        _check(load_library().mnt_kernel_map_pair_lists(
            _ptr(kernel_map), num_offsets, num_targets, cum.ctypes.data_as(_pi64), _ptr(in_idx),
            _ptr(out_idx), _stream(device)))
    return in_idx, out_idx


# ------------------------------------------------------------ padding plan ----

def generate_padding_buckets(sizes: Sequence[int], threshold: Optional[float]):
    """GeneratePaddingBuckets, csrc/minuet/cuda/functions/sparse_convolution.cu:16-43."""
    arr = np.ascontiguousarray(np.asarray(sizes, dtype=np.int64))
    out = np.zeros(arr.shape[0] + 1, dtype=np.int64)
    count = ctypes.c_int64(0)
    _check(load_library().mnt_generate_padding_buckets(
        arr.ctypes.data_as(_pi64), arr.shape[0], 0 if threshold is None else 1,
        0.0 if threshold is None else float(threshold), out.ctypes.data_as(_pi64),
        ctypes.byref(count)))
    return out[:count.value].tolist()


def cumsum_kernel_padded_sizes(sizes: Sequence[int], buckets: Sequence[int]):
    """ComputeCumsumKernelPaddedSizes, sparse_convolution.cu:272-292."""
    arr = np.ascontiguousarray(np.asarray(sizes, dtype=np.int64))
    bks = np.ascontiguousarray(np.asarray(buckets, dtype=np.int64))
    out = np.zeros(arr.shape[0] + 1, dtype=np.int64)
    _check(load_library().mnt_cumsum_kernel_padded_sizes(
        arr.ctypes.data_as(_pi64), arr.shape[0], bks.ctypes.data_as(_pi64), bks.shape[0],
        out.ctypes.data_as(_pi64)))
    return out.tolist()


# ----------------------------------------------------------------- forward ----

def _conv_shapes(weights, source_masks, target_masks, kernel_map_sizes):
    _ensure_ndim("weights", weights, 3)
    _ensure_ndim("source_masks", source_masks, 2)
    _ensure_ndim("target_masks", target_masks, 2)
    _ensure_ndim("kernel_map_sizes", kernel_map_sizes, 1)
    num_offsets = target_masks.size(0)
    _ensure_dim("kernel_map_sizes", kernel_map_sizes, 0, num_offsets)
    _ensure_dim("source_masks", source_masks, 0, num_offsets)
    return (source_masks.size(1), target_masks.size(1), num_offsets, weights.size(1),
            weights.size(2))


ACTIVATION_CODES = {None: 0, "relu": 1, "leaky_relu": 2, "relu6": 3}


class Epilogue:
    """What the forward applies to each summed output row before rounding:
    ``act(row * scale + shift + residual)``.  ``scale`` / ``shift``: fp32
    ``[C_out]``; ``residual``: ``[N_out, C_out]`` of the feature dtype;
    ``activation``: ``None``, ``"relu"``, ``"leaky_relu"`` or ``"relu6"``."""

    __slots__ = ("scale", "shift", "residual", "activation", "negative_slope")

    def __init__(self, scale: Optional[torch.Tensor] = None, shift: Optional[torch.Tensor] = None,
                 residual: Optional[torch.Tensor] = None, activation: Optional[str] = None,
                 negative_slope: float = 0.01):
        if activation not in ACTIVATION_CODES:
            raise ValueError(f"unknown activation {activation!r}")
        self.scale, self.shift, self.residual = scale, shift, residual
        self.activation, self.negative_slope = activation, negative_slope

    def checked(self, num_targets: int, channels: int, dtype: torch.dtype, device) -> "Epilogue":
        """Copy with operands validated and laid out the way the kernel reads them
        (the object itself when nothing needs changing)."""
        scale, shift, residual = self.scale, self.shift, self.residual
        f32 = torch.float32
        if ((scale is None or (scale.dtype == f32 and scale.device == device and scale.dim() == 1
                               and scale.shape[0] == channels and scale.is_contiguous()))
                and (shift is None or (shift.dtype == f32 and shift.device == device and shift.dim() == 1
                                       and shift.shape[0] == channels and shift.is_contiguous()))
                and (residual is None or (residual.dtype == dtype and residual.device == device
                                          and residual.dim() == 2 and residual.shape[0] == num_targets
                                          and residual.shape[1] == channels and residual.is_contiguous()
                                          and residual.data_ptr() % 16 == 0))):
            return self

        def vector(name, t):
            if t is None:
                return None
            if t.shape != (channels,) or t.device != device:
                _fail(f"epilogue {name} must be a [{channels}] tensor on the device of the features")
            if t.dtype == torch.float32 and t.is_contiguous():
                return t
            return t.to(torch.float32).contiguous()
        residual = self.residual
        if residual is not None:
            if residual.shape != (num_targets, channels) or residual.dtype != dtype or \
                    residual.device != device:
                _fail(f"epilogue residual must be a [{num_targets}, {channels}] {dtype} tensor on "
                      "the device of the features")
            residual = residual.contiguous()
            if residual.data_ptr() % 16:
                residual = residual.clone()
        return Epilogue(vector("scale", self.scale), vector("shift", self.shift), residual,
                        self.activation, self.negative_slope)

    def apply(self, features: torch.Tensor) -> torch.Tensor:
        """The same arithmetic with tensor expressions (fp32, one rounding), for
        paths that do not go through Scatter."""
        value = features.float()
        if self.scale is not None:
            value = value * self.scale.float()
        if self.shift is not None:
            value = value + self.shift.float()
        if self.residual is not None:
            value = value + self.residual.float()
        if self.activation == "relu":
            value = torch.relu(value)
        elif self.activation == "leaky_relu":
            value = torch.nn.functional.leaky_relu(value, self.negative_slope)
        elif self.activation == "relu6":
            value = torch.nn.functional.relu6(value)
        return value.to(features.dtype)


def _host_sizes_arg(sizes_host, num_offsets):
    if sizes_host is None:
        return None, None
    if type(sizes_host) is np.ndarray and sizes_host.dtype == np.int64 and sizes_host.flags.c_contiguous:
        arr = sizes_host
    else:
        arr = np.ascontiguousarray(np.asarray(sizes_host, dtype=np.int64))
    if arr.shape[0] != num_offsets:
        _fail("host copy of kernel_map_sizes has the wrong length")
    return arr, ctypes.cast(arr.__array_interface__["data"][0], _pi64)


def cuda_sparse_convolution_forward(gather_tile_size: int, scatter_tile_size: int,
                                    allow_shortcut_matmul: bool, parallel: int,
                                    threshold: Optional[float], sources: torch.Tensor,
                                    weights: torch.Tensor, source_masks: torch.Tensor,
                                    target_masks: torch.Tensor,
                                    kernel_map_order: Optional[torch.Tensor],
                                    kernel_map_sizes: torch.Tensor,
                                    kernel_map_sizes_host=None,
                                    gather_index: Optional[torch.Tensor] = None,
                                    epilogue: Optional["Epilogue"] = None,
                                    packed_weights: Optional[torch.Tensor] = None,
                                    kernel_map_order_host=None) -> torch.Tensor:
    """csrc/minuet/torch/cuda_sparse_convolution_forward.cu:136-213.  The extra
    ``kernel_map_sizes_host`` spares the device read-back of the sizes;
    ``gather_index`` (int32, the kernel map's source row per buffer row) folds
    the Gather step into the GEMM; ``epilogue`` is applied to every output row
    before it is rounded to the feature dtype; ``packed_weights``
    (:func:`pack_weights` of ``weights``) spares the packing pass and needs
    ``kernel_map_order_host`` whenever there is a ``kernel_map_order``."""
    fn = "CUDASparseConvolutionForward"
    _ensure_ndim("sources", sources, 2)
    S, T, O, K, N = _conv_shapes(weights, source_masks, target_masks, kernel_map_sizes)
    if kernel_map_order is not None:
        _ensure_dim("kernel_map_order", kernel_map_order, 0, O)
    _ensure_dim("weights", weights, 0, O)
    _ensure_dim("sources", sources, 1, K)
    _ensure_dim("sources", sources, 0, S)
    index_tensors = [source_masks, target_masks, kernel_map_sizes]
    if kernel_map_order is not None:
        index_tensors.append(kernel_map_order)
    device = _common_device([sources, weights] + index_tensors)
    itype = _common_dtype(index_tensors)
    if sources.dtype != weights.dtype:
        _fail(f"Found tensors with two different scalar types ({sources.dtype} != {weights.dtype})")
    fcode = _float_code(weights.dtype, fn)
    icode = _int_code(itype, "index", fn)
    out = torch.empty((T, N), dtype=weights.dtype, device=device)
    keep, sizes_ptr = _host_sizes_arg(kernel_map_sizes_host, O)
    if gather_index is not None:
        if gather_index.dtype != torch.int32 or gather_index.device != device:
            _fail("gather_index must be an int32 tensor on the device of the features")
        if kernel_map_sizes_host is None or gather_index.numel() != int(np.sum(kernel_map_sizes_host)):
            _fail("gather_index needs the host sizes and one entry per kernel map hit")
        gather_index = gather_index.contiguous()
    ep = Epilogue() if epilogue is None else epilogue.checked(T, N, weights.dtype, device)
    keep_order = order_ptr = None
    if packed_weights is not None:
        _check_packed(packed_weights, weights)
        if kernel_map_order is not None:
            if kernel_map_order_host is None:
                _fail("packed weights need the host copy of kernel_map_order")
            keep_order, order_ptr = _host_sizes_arg(kernel_map_order_host, O)
    with _on(device):
        _check(load_library().mnt_sparse_convolution_forward_fused(
            int(gather_tile_size), int(scatter_tile_size), 1 if allow_shortcut_matmul else 0,
            int(parallel), 0 if threshold is None else 1,
            0.0 if threshold is None else float(threshold), _ptr(sources), _ptr(weights),
            _ptr(source_masks), _ptr(target_masks), _ptr(kernel_map_order),
            _ptr(kernel_map_sizes), sizes_ptr, S, T, O, K, N, icode, fcode, _ptr(gather_index),
            _ptr(ep.scale), _ptr(ep.shift), _ptr(ep.residual), ACTIVATION_CODES[ep.activation],
            float(ep.negative_slope), _ptr(packed_weights), order_ptr, _ptr(out), _stream(device)))
    del keep, keep_order
    return out


def sparse_convolution_forward_map(sources: torch.Tensor, weights: torch.Tensor, kernel_map,
                                   gather_tile_size: int = 0, scatter_tile_size: int = 0,
                                   allow_shortcut_matmul: bool = False, parallel: int = 4,
                                   threshold: Optional[float] = 0, epilogue: Optional["Epilogue"] = None,
                                   packed_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`cuda_sparse_convolution_forward` for a
    :class:`~minuet_amd.nn.KernelMap` that carries host sizes and pair lists:
    the same library call, with everything that depends on the map alone
    (shapes, dtypes, devices, pointers) checked and worked out once per map
    instead of once per forward."""
    prepared = kernel_map.prepared
    if prepared is None:
        source_masks, target_masks, order, sizes = kernel_map
        _conv_shapes(torch.empty((sizes.shape[0], 1, 1), device="meta"), source_masks, target_masks, sizes)
        tensors = [source_masks, target_masks, sizes] + ([order] if order is not None else [])
        device = _common_device(tensors + [kernel_map.in_idx])
        icode = _int_code(_common_dtype(tensors), "index", "CUDASparseConvolutionForward")
        O = target_masks.size(0)
        if order is not None:
            _ensure_dim("kernel_map_order", order, 0, O)
        if kernel_map.in_idx.dtype != torch.int32 or kernel_map.in_idx.numel() != int(np.sum(kernel_map.sizes_host)):
            _fail("gather_index needs the host sizes and one entry per kernel map hit")
        keep = [t.contiguous() for t in (source_masks, target_masks, sizes, kernel_map.in_idx)]
        keep_order = None if order is None else order.contiguous()
        sizes_host, sizes_ptr = _host_sizes_arg(kernel_map.sizes_host, O)
        order_host, order_ptr = ((None, None) if kernel_map.order_host is None
                                 else _host_sizes_arg(kernel_map.order_host, O))
        if order is not None and order_host is None:
            _fail("packed weights need the host copy of kernel_map_order")
        prepared = kernel_map.prepared = (
            source_masks.size(1), target_masks.size(1), O, icode, device, _ptr(keep[0]), _ptr(keep[1]),
            _ptr(keep_order), _ptr(keep[2]), sizes_ptr, order_ptr, _ptr(keep[3]),
            (keep, keep_order, sizes_host, order_host))
    S, T, O, icode, device, p_sm, p_tm, p_order, p_sizes, sizes_ptr, order_ptr, p_gather, _ = prepared
    dtype = weights.dtype
    if not (sources.dim() == 2 and weights.dim() == 3 and sources.shape[0] == S and weights.shape[0] == O
            and sources.shape[1] == weights.shape[1] and sources.dtype == dtype and sources.device == device
            and weights.device == device and dtype in _FLOAT):
        source_masks, target_masks, order, sizes = kernel_map           # the checks one by one, for the message
        return cuda_sparse_convolution_forward(
            gather_tile_size, scatter_tile_size, allow_shortcut_matmul, parallel, threshold, sources, weights,
            source_masks, target_masks, order, sizes, kernel_map_sizes_host=kernel_map.sizes_host,
            gather_index=kernel_map.in_idx, epilogue=epilogue, packed_weights=packed_weights,
            kernel_map_order_host=kernel_map.order_host)
    K, N = weights.shape[1], weights.shape[2]
    if not sources.is_contiguous():
        sources = sources.contiguous()
    if not weights.is_contiguous():
        weights = weights.contiguous()
    out = torch.empty((T, N), dtype=dtype, device=device)
    ep = Epilogue() if epilogue is None else epilogue.checked(T, N, dtype, device)
    if packed_weights is not None:
        _check_packed(packed_weights, weights)
    with _on(device):
        _check(load_library().mnt_sparse_convolution_forward_fused(
            int(gather_tile_size), int(scatter_tile_size), 1 if allow_shortcut_matmul else 0,
            int(parallel), 0 if threshold is None else 1,
            0.0 if threshold is None else float(threshold), _ptr(sources), _ptr(weights), p_sm, p_tm, p_order,
            p_sizes, sizes_ptr, S, T, O, K, N, icode, _FLOAT[dtype], p_gather, _ptr(ep.scale), _ptr(ep.shift),
            _ptr(ep.residual), ACTIVATION_CODES[ep.activation], float(ep.negative_slope),
            _ptr(packed_weights), order_ptr if packed_weights is not None else None, _ptr(out),
            _stream(device)))
    return out


def sparse_convolution_forward_rows(sources: torch.Tensor, weights: torch.Tensor, sizes_host, order_host,
                                    in_idx: torch.Tensor, out_pos: torch.Tensor, row_ptr: torch.Tensor,
                                    scatter_tile_size: int = 0, epilogue: Optional["Epilogue"] = None,
                                    packed_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The list-driven Gather-GEMM-Scatter (mnt_sparse_convolution_forward_rows):
    ``in_idx`` / ``out_pos`` [nnz] and ``row_ptr`` [T + 1] int32 on the device,
    ``sizes_host`` / ``order_host`` int64 on the host (``order_host`` None: rows
    in offset order), ``weights`` [O, Cin, Cout] in the layer's offset order."""
    _ensure_ndim("sources", sources, 2)
    _ensure_ndim("weights", weights, 3)
    device = _common_device([sources, weights, in_idx, out_pos, row_ptr])
    fcode = _float_code(_common_dtype([sources, weights]), "sparse_convolution_forward_rows")
    S, K = sources.shape
    O, K2, N = weights.shape
    if K2 != K:
        _fail(f"The dimension 1 of Tensor weights is expected to be {K} but found {K2}")
    T = row_ptr.numel() - 1
    for name, tensor in (("in_idx", in_idx), ("out_pos", out_pos), ("row_ptr", row_ptr)):
        if tensor.dtype != torch.int32 or not tensor.is_contiguous():
            _fail(f"{name} must be a contiguous int32 tensor")
    keep, sizes_ptr = _host_sizes_arg(sizes_host, O)
    keep_order, order_ptr = (None, None) if order_host is None else _host_sizes_arg(order_host, O)
    if in_idx.numel() != out_pos.numel() or in_idx.numel() != int(np.asarray(keep).sum()):
        _fail("in_idx / out_pos need one entry per kernel map hit")
    ep = Epilogue() if epilogue is None else epilogue.checked(T, N, sources.dtype, device)
    if packed_weights is not None:
        _check_packed(packed_weights, weights)
    sources, weights = sources.contiguous(), weights.contiguous()
    out = torch.empty((T, N), dtype=sources.dtype, device=device)
    with _on(device):
        _check(load_library().mnt_sparse_convolution_forward_rows(
            int(scatter_tile_size), _ptr(sources), _ptr(weights), sizes_ptr, order_ptr, _ptr(in_idx),
            _ptr(out_pos), _ptr(row_ptr), S, T, O, K, N, fcode, _ptr(ep.scale), _ptr(ep.shift),
            _ptr(ep.residual), ACTIVATION_CODES[ep.activation], float(ep.negative_slope),
            _ptr(packed_weights), _ptr(out), _stream(device)))
    del keep, keep_order
    return out


def offset_group_table(offsets_host: np.ndarray) -> Optional[np.ndarray]:
    """For a kernel of 27 offsets that form a 3 x 3 x 3 grid (any dilation, any
    order): int32 ``[3, 9, 3]``, the offset index of member m of group j along
    axis a, where the groups along an axis are the triples of offsets that
    differ along that axis only.  None for any other kernel."""
    offsets = np.asarray(offsets_host, dtype=np.int64)
    if offsets.shape != (27, 3):
        return None
    key = offsets.tobytes()
    if key in _GROUP_TABLES:
        return _GROUP_TABLES[key]
    table = _offset_group_table(offsets)
    if len(_GROUP_TABLES) > 64:
        _GROUP_TABLES.clear()
    _GROUP_TABLES[key] = table
    return table


_GROUP_TABLES = {}


def _offset_group_table(offsets: np.ndarray) -> Optional[np.ndarray]:
    table = np.zeros((3, 9, 3), dtype=np.int32)
    for axis in range(3):
        others = [a for a in range(3) if a != axis]
        rest = offsets[:, others]
        keys, group_of = np.unique(rest, axis=0, return_inverse=True)
        group_of = np.asarray(group_of).reshape(-1)
        if keys.shape[0] != 9:
            return None
        for j in range(9):
            members = np.nonzero(group_of == j)[0]
            if members.shape[0] != 3 or np.unique(offsets[members, axis]).shape[0] != 3:
                return None
            table[axis, j] = members[np.argsort(offsets[members, axis], kind="stable")]
    return np.ascontiguousarray(table)


class OffsetGroups:
    """The offset-group tables of one dense kernel map (mnt_kernel_map_offset_groups):
    ``rank`` int32 [9, T], ``src`` int32 [9 * T, 4], ``head`` int32 [16] on the
    device and the host table ``offsets`` int32 [3, 9, 3] they were built with."""

    def __init__(self, rank, src, head, offsets, num_targets):
        self.rank, self.src, self.head, self.offsets, self.num_targets = rank, src, head, offsets, num_targets
        self._offsets_address = offsets.ctypes.data


def kernel_map_offset_groups(kernel_map: torch.Tensor, offsets_host: np.ndarray) -> Optional[OffsetGroups]:
    """Offset groups of a dense int32 kernel map ``[27, T]`` whose offsets form a
    3 x 3 x 3 grid; None for other kernels.  Waits for nothing on the device."""
    table = offset_group_table(offsets_host)
    if table is None or kernel_map.dim() != 2 or kernel_map.shape[0] != 27:
        return None
    if kernel_map.dtype != torch.int32:
        _fail("kernel_map_offset_groups expects an int32 kernel map")
    device = _common_device([kernel_map])
    kernel_map = kernel_map.contiguous()
    T = kernel_map.shape[1]
    table = np.ascontiguousarray(table)
    store = torch.empty((9 * T * 5 + 16,), dtype=torch.int32, device=device)
    src, rank, head = store[:36 * T].view(9 * T, 4), store[36 * T:45 * T].view(9, T), store[45 * T:]
    with _on(device):
        _check(load_library().mnt_kernel_map_offset_groups(
            _ptr(kernel_map), T, table.ctypes.data, _ptr(rank), _ptr(src), _ptr(head), _stream(device)))
    return OffsetGroups(rank, src, head, table, T)


def offset_groups_forward_supported(in_channels: int, out_channels: int, dtype: torch.dtype) -> bool:
    """Whether mnt_sparse_convolution_forward_groups takes these widths."""
    return (dtype in (torch.float16, torch.bfloat16) and (in_channels * 2) % 128 == 0
            and out_channels % 8 == 0)


def sparse_convolution_forward_groups(sources: torch.Tensor, weights: torch.Tensor, groups: OffsetGroups,
                                      epilogue: Optional["Epilogue"] = None,
                                      packed_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The forward pass over offset groups (mnt_sparse_convolution_forward_groups):
    ``weights`` [27, Cin, Cout] in the layer's own offset order (``packed_weights``:
    their :func:`pack_weights` form, made here when missing)."""
    _ensure_ndim("sources", sources, 2)
    _ensure_ndim("weights", weights, 3)
    device = _common_device([sources, weights, groups.rank])
    fcode = _float_code(_common_dtype([sources, weights]), "sparse_convolution_forward_groups")
    S, K = sources.shape
    O, K2, N = weights.shape
    if K2 != K or O != 27:
        _fail(f"weights are expected to be [27, {K}, C_out] but found {tuple(weights.shape)}")
    if not offset_groups_forward_supported(K, N, sources.dtype):
        _fail(f"the offset-group forward does not take {K} -> {N} channels of {sources.dtype}")
    T = groups.num_targets
    ep = Epilogue() if epilogue is None else epilogue.checked(T, N, sources.dtype, device)
    if packed_weights is None:
        packed_weights = pack_weights(weights.contiguous())
    else:
        _check_packed(packed_weights, weights)
    sources = sources.contiguous()
    out = torch.empty((T, N), dtype=sources.dtype, device=device)
    with _on(device):
        _check(load_library().mnt_sparse_convolution_forward_groups(
            _ptr(sources), _ptr(packed_weights), _ptr(groups.rank), _ptr(groups.src), _ptr(groups.head),
            groups._offsets_address, S, T, K, N, fcode, _ptr(ep.scale), _ptr(ep.shift), _ptr(ep.residual),
            ACTIVATION_CODES[ep.activation], float(ep.negative_slope), _ptr(out), _stream(device)))
    return out


def packed_weights_shape(weights: torch.Tensor):
    """Shape of :func:`pack_weights`'s result for ``weights [O, C_in, C_out]``."""
    O, K, N = weights.shape
    per_chunk = 128 // weights.dtype.itemsize
    return (O, (N + 31) // 32 * 32, (K + per_chunk - 1) // per_chunk * per_chunk)


def pack_weights(weights: torch.Tensor) -> torch.Tensor:
    """``weights [O, C_in, C_out]`` in the transposed, padded layout the matrix
    kernels stage (offset order unchanged).  A layer keeps the result for as
    long as its weights do not change and hands it to the forward functions."""
    _ensure_ndim("weights", weights, 3)
    device = _common_device([weights])
    fcode = _float_code(weights.dtype, "pack_weights")
    weights = weights.contiguous()
    packed = torch.empty(packed_weights_shape(weights), dtype=weights.dtype, device=device)
    O, K, N = weights.shape
    with _on(device):
        _check(load_library().mnt_pack_weights(_ptr(weights), O, K, N, fcode, _ptr(packed),
                                               _stream(device)))
    return packed


def _check_packed(packed: torch.Tensor, weights: torch.Tensor):
    if (tuple(packed.shape) != packed_weights_shape(weights) or packed.dtype != weights.dtype
            or packed.device != weights.device or not packed.is_contiguous()):
        _fail("packed_weights does not belong to these weights (shape, dtype, device or layout)")


def kernel_map_invert(kernel_map: torch.Tensor, num_sources: int) -> torch.Tensor:
    """``[O, num_sources]`` int32 map with ``inverse[o, m] = t`` wherever
    ``kernel_map[o, t] = m`` and -1 elsewhere: the dense kernel map of the
    transposed layer that shares this map."""
    _ensure_ndim("kernel_map", kernel_map, 2)
    if kernel_map.dtype != torch.int32:
        _fail("kernel_map_invert expects an int32 kernel map")
    device = _common_device([kernel_map])
    kernel_map = kernel_map.contiguous()
    num_offsets, num_targets = kernel_map.shape
    inverse = torch.empty((num_offsets, num_sources), dtype=torch.int32, device=device)
    with _on(device):
        _check(load_library().mnt_kernel_map_invert(_ptr(kernel_map), num_offsets, num_targets,
                                                    num_sources, _ptr(inverse), _stream(device)))
    return inverse


IMPLICIT_MAX_TARGET_FEATURES = 512
IMPLICIT_MAX_SOURCE_ROW_BYTES = 2048


IMPLICIT_NARROW_LDS_BYTES = 64 * 1024
_IMPLICIT_TURN_BYTES = 4 * 32 * (32 * 4 + 16)


def implicit_forward_supported(num_source_features: int, num_target_features: int,
                               dtype: torch.dtype, num_offsets: Optional[int] = None) -> bool:
    """Shapes ``sparse_convolution_forward_implicit`` accepts: source rows of a
    multiple of 16 bytes, or, for 16-bit features, rows of 4 or 8 bytes (a
    stem's 2 or 4 input channels) under a kernel of ``num_offsets`` offsets
    small enough for its weights to sit in LDS as a whole."""
    row_bytes = num_source_features * dtype.itemsize
    if (num_target_features % 4 != 0 or num_target_features > IMPLICIT_MAX_TARGET_FEATURES
            or row_bytes > IMPLICIT_MAX_SOURCE_ROW_BYTES):
        return False
    if row_bytes % 16 == 0:
        return row_bytes > 0
    if dtype.itemsize != 2 or row_bytes not in (4, 8) or num_offsets is None or num_target_features > 128:
        return False
    steps = -(-num_offsets * num_source_features // 16)
    blocks = -(-num_target_features // 32)
    return steps * blocks * 1024 + _IMPLICIT_TURN_BYTES <= IMPLICIT_NARROW_LDS_BYTES


def sparse_convolution_forward_implicit(sources: torch.Tensor, weights: torch.Tensor,
                                        kernel_map: torch.Tensor,
                                        epilogue: Optional[Epilogue] = None,
                                        packed_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Output-stationary forward from the dense kernel map ``[O, N_out]`` (int32,
    original offset order): one kernel, no gather / GEMM-output buffers."""
    fn = "sparse_convolution_forward_implicit"
    device = sources.device
    dtype = weights.dtype
    if not (sources.dim() == 2 and weights.dim() == 3 and kernel_map.dim() == 2
            and kernel_map.shape[0] == weights.shape[0] and sources.shape[1] == weights.shape[1]
            and weights.device == device and kernel_map.device == device and device.type == "cuda"
            and kernel_map.dtype == torch.int32 and sources.dtype == dtype and dtype in _FLOAT):
        # something is off: the checks one by one, for the message
        _ensure_ndim("sources", sources, 2)
        _ensure_ndim("weights", weights, 3)
        _ensure_ndim("kernel_map", kernel_map, 2)
        _ensure_dim("kernel_map", kernel_map, 0, weights.shape[0])
        _ensure_dim("sources", sources, 1, weights.shape[1])
        _common_device([sources, weights, kernel_map])
        if kernel_map.dtype != torch.int32:
            _fail("the implicit forward expects an int32 kernel map")
        if sources.dtype != dtype:
            _fail(f"Found tensors with two different scalar types ({sources.dtype} != {dtype})")
    O, K, N = weights.shape
    fcode = _float_code(dtype, fn)
    S, T = sources.shape[0], kernel_map.shape[1]
    if not sources.is_contiguous():
        sources = sources.contiguous()
    if not weights.is_contiguous():
        weights = weights.contiguous()
    if not kernel_map.is_contiguous():
        kernel_map = kernel_map.contiguous()
    if sources.data_ptr() % 16:
        sources = sources.clone()
    out = torch.empty((T, N), dtype=weights.dtype, device=device)
    ep = Epilogue() if epilogue is None else epilogue.checked(T, N, weights.dtype, device)
    if packed_weights is not None:
        _check_packed(packed_weights, weights)
    with _on(device):
        _check(load_library().mnt_sparse_convolution_forward_implicit(
            _ptr(sources), _ptr(weights), _ptr(kernel_map), S, T, O, K, N, fcode, _ptr(ep.scale),
            _ptr(ep.shift), _ptr(ep.residual), ACTIVATION_CODES[ep.activation],
            float(ep.negative_slope), _ptr(packed_weights), _ptr(out), _stream(device)))
    return out


def _time_stage(name, lead_args, threshold, mask, weights, source_masks, target_masks,
                kernel_map_sizes, pass_weights):
    S, T, O, K, N = _conv_shapes(weights, source_masks, target_masks, kernel_map_sizes)
    device = _common_device([weights, source_masks, target_masks, kernel_map_sizes])
    itype = _common_dtype([source_masks, target_masks, kernel_map_sizes])
    fcode = _float_code(weights.dtype, name)
    icode = _int_code(itype, "index", name)
    ms = ctypes.c_float(0.0)
    first = weights if pass_weights else mask
    with _on(device):
        _check(getattr(load_library(), name)(
            *lead_args, 0 if threshold is None else 1,
            0.0 if threshold is None else float(threshold), _ptr(first), _ptr(kernel_map_sizes),
            S, T, O, K, N, icode, fcode, ctypes.byref(ms), _stream(device)))
    return float(ms.value)


def cuda_time_gather(tile_size, allow_shortcut_matmul, threshold, weights, source_masks,
                     target_masks, kernel_map_sizes) -> float:
    """csrc/minuet/torch/cuda_sparse_convolution_forward.cu:50-91."""
    return _time_stage("mnt_time_gather", (int(tile_size), 1 if allow_shortcut_matmul else 0),
                       threshold, source_masks, weights, source_masks, target_masks,
                       kernel_map_sizes, False)


def cuda_time_scatter(tile_size, allow_shortcut_matmul, threshold, weights, source_masks,
                      target_masks, kernel_map_sizes) -> float:
    """csrc/minuet/torch/cuda_sparse_convolution_forward.cu:93-134."""
    return _time_stage("mnt_time_scatter", (int(tile_size), 1 if allow_shortcut_matmul else 0),
                       threshold, target_masks, weights, source_masks, target_masks,
                       kernel_map_sizes, False)


def cuda_time_gemm(allow_shortcut_matmul, parallel, threshold, weights, source_masks,
                   target_masks, kernel_map_sizes) -> float:
    """csrc/minuet/torch/cuda_sparse_convolution_forward.cu:7-48."""
    return _time_stage("mnt_time_gemm", (1 if allow_shortcut_matmul else 0, int(parallel)),
                       threshold, None, weights, source_masks, target_masks, kernel_map_sizes, True)


# ------------------------------------------------------------------ memory ----

def _current_stream():
    if not torch.cuda.is_available():
        _fail("no GPU is available")
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def cuda_preallocate_buffer(size: int):
    _check(load_library().mnt_buffer_preallocate(_current_stream(), int(size)))


def cuda_free_buffers():
    _check(load_library().mnt_buffer_free(_current_stream()))


def cuda_set_buffer_growth(growth: float):
    _check(load_library().mnt_buffer_set_growth(_current_stream(), float(growth)))


def cuda_set_buffer_page_size(page_size: int):
    _check(load_library().mnt_buffer_set_page_size(_current_stream(), int(page_size)))


def cuda_buffer_used_size() -> int:
    return int(load_library().mnt_buffer_used_size(_current_stream()))


def cuda_buffer_total_size() -> int:
    return int(load_library().mnt_buffer_total_size(_current_stream()))


def cuda_reset_error():
    load_library().mnt_reset_error()


_device_resets = 0


def device_reset_count() -> int:
    """How often :func:`cuda_device_reset` has run in this process (what holds
    addresses of the library's scratch memory checks it before using them)."""
    return _device_resets


def cuda_device_reset():
    """csrc/minuet/torch/cuda_memory_buffer.cu:38,47.  Frees everything the library
    holds on the current device (every stream's arena); unlike the reference's
    cudaDeviceReset() it leaves the context, and with it every torch tensor, alone.
    Passes captured with ``minuet.capture_forward`` before the reset refuse to
    replay after it (their kernels point into the freed scratch memory)."""
    global _device_resets
    _device_resets += 1
    _check(load_library().mnt_device_reset())


def stream_acquire(stream=None):
    """Keeps the library's state of ``stream`` (a raw handle; None = the null
    stream) for the calling thread until :func:`stream_release`: calls of other
    threads on that stream fail meanwhile.  One caller thread per stream at a
    time is the library's threading contract (ctypes releases the interpreter
    lock during a call, so two Python threads can be inside the library at once;
    the reference's pybind module holds the lock, csrc/minuet/torch/common.h:17-21)."""
    _check(load_library().mnt_stream_acquire(stream))


def stream_release(stream=None):
    _check(load_library().mnt_stream_release(stream))


def host_wait_stats(reset: bool = False):
    """``(waits, seconds)``: how often and for how long library calls of this
    process have made the host wait for the device since the tally was last
    reset (each wait polls one completion flag in pinned memory)."""
    waits, ns = ctypes.c_int64(0), ctypes.c_int64(0)
    _check(load_library().mnt_host_wait_stats(ctypes.byref(waits), ctypes.byref(ns), 1 if reset else 0))
    return waits.value, ns.value * 1e-9


AHEAD_COORDS, AHEAD_DENSE, AHEAD_TABLES, AHEAD_INVERT = 0, 1, 2, 3


class LookaheadItem(ctypes.Structure):
    """``mnt_lookahead_item`` of include/minuet_hip.h."""
    _fields_ = [("kind", ctypes.c_int32), ("source_level", ctypes.c_int32),
                ("target_level", ctypes.c_int32), ("dense_item", ctypes.c_int32),
                ("reorder", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("stride", ctypes.c_int64 * 4), ("offsets", ctypes.c_void_p),
                ("num_offsets", ctypes.c_int64), ("capacity", ctypes.c_int64),
                ("out0", ctypes.c_void_p), ("out1", ctypes.c_void_p), ("out2", ctypes.c_void_p),
                ("out3", ctypes.c_void_p), ("out4", ctypes.c_void_p), ("out5", ctypes.c_void_p),
                ("host0", ctypes.c_void_p), ("host1", ctypes.c_void_p)]


def lookahead_start(coordinates: torch.Tensor, batch_dims: Optional[torch.Tensor], bounds,
                    items, num_levels: int):
    """Hands ``items`` (a ctypes array of :class:`LookaheadItem`) to the
    library's worker thread, which builds them for the sorted cloud
    ``coordinates`` on a stream of its own; returns at once."""
    device = coordinates.device
    n, ndim = coordinates.shape
    known = None if bounds is None else np.ascontiguousarray(bounds, dtype=np.int64)
    with _on(device):
        _check(load_library().mnt_lookahead_start(
            coordinates.data_ptr(), n, ndim, _INT[coordinates.dtype], _ptr(batch_dims),
            batch_dims.numel() - 1 if batch_dims is not None else 1,
            _INT[batch_dims.dtype] if batch_dims is not None else 0,
            None if known is None else known.ctypes.data_as(_pi64), ctypes.addressof(items),
            len(items), num_levels, None, None, _stream(device)))


def lookahead_wait(item: int, device: torch.device) -> int:
    """Blocks until ``item`` is built, orders the current stream after the
    kernels that wrote it and returns its size."""
    size = ctypes.c_int64(0)
    with _on(device):
        _check(load_library().mnt_lookahead_wait(item, _stream(device), ctypes.byref(size)))
    return size.value


def lookahead_finish(device: torch.device):
    """Waits for the worker to go idle and orders the current stream after all
    it enqueued; a no-op without a session."""
    with _on(device):
        _check(load_library().mnt_lookahead_finish(_stream(device)))


def time_memory(kind: str, nbytes: int, repeats: int = 10, device=None) -> float:
    """Milliseconds one plain streaming kernel takes for ``nbytes`` of device
    memory: ``kind`` "copy" (reads and writes that many bytes), "read" or "write"."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    ms = ctypes.c_float(0.0)
    with _on(device):
        _check(load_library().mnt_time_memory({"copy": 0, "read": 1, "write": 2}[kind], nbytes, repeats,
                                              ctypes.byref(ms), _stream(device)))
    return float(ms.value)


def device_facts():
    """Compute units, clocks, bus width, L2 and memory size of the current device."""
    facts = (ctypes.c_int64 * 6)()
    _check(load_library().mnt_device_facts(facts, 6))
    return {"compute_units": int(facts[0]), "engine_clock_mhz": facts[1] / 1e3,
            "memory_clock_mhz": facts[2] / 1e3, "memory_bus_bits": int(facts[3]),
            "l2_bytes": int(facts[4]), "memory_bytes": int(facts[5])}


def timer_repeats(repeats: int):
    """Launches per run of the ``cuda_time_*`` stage timers (1 = the reference's
    protocol; more = back-to-back launches, time of one)."""
    _check(load_library().mnt_timer_repeats(int(repeats)))


def profile_enable(on: bool):
    load_library().mnt_profile_enable(1 if on else 0)


def profile_read():
    """Stage intervals recorded since the last read: list of (name, ms)."""
    capacity, stride = 4096, 32
    ms = (ctypes.c_float * capacity)()
    labels = ctypes.create_string_buffer(capacity * stride)
    count = ctypes.c_int(0)
    _check(load_library().mnt_profile_read(capacity, ms, labels, stride, ctypes.byref(count)))
    raw = labels.raw
    out = []
    for i in range(count.value):
        name = raw[i * stride:(i + 1) * stride].split(b"\0", 1)[0].decode()
        out.append((name, float(ms[i])))
    return out
