"""Scratch-arena knobs (mirrors minuet/nn/functional/memory.py)."""
from . import _C

__all__ = ["cuda_buffer_total_size", "cuda_buffer_used_size", "cuda_free_buffers",
           "cuda_set_buffer_growth", "cuda_set_buffer_page_size", "cuda_preallocate_buffer",
           "cuda_reset_error", "cuda_device_reset"]


def cuda_buffer_total_size() -> int:
    """Bytes held by the scratch arena of the current stream."""
    return _C.cuda_buffer_total_size()


def cuda_buffer_used_size() -> int:
    """Bytes of the arena currently lent out (the reference's wrapper returns the
    total here by mistake, memory.py:14-15)."""
    return _C.cuda_buffer_used_size()


def cuda_free_buffers():
    return _C.cuda_free_buffers()


def cuda_preallocate_buffer(size: int):
    return _C.cuda_preallocate_buffer(size)


def cuda_set_buffer_growth(growth: float):
    return _C.cuda_set_buffer_growth(growth)


def cuda_set_buffer_page_size(page_size: int):
    return _C.cuda_set_buffer_page_size(page_size)


def cuda_reset_error():
    _C.cuda_reset_error()


def cuda_device_reset():
    """Gives back all scratch memory the library holds on the current device
    (every stream's arena) and clears its error state."""
    _C.cuda_device_reset()
