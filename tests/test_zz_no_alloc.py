"""The allocation-free sizes entry point (static device scratch) against the
arena-backed one it is a variant of, through the C ABI."""
import numpy as np
import pytest
import torch

from minuet_amd.nn.functional import _C

pytestmark = pytest.mark.gpu


def _random_map(num_offsets, num_targets, density, seed, dtype):
    rng = np.random.default_rng(seed)
    dense = rng.integers(0, max(1, num_targets), size=(num_offsets, num_targets))
    dense[rng.random(size=dense.shape) >= density] = -1
    return torch.from_numpy(dense.astype(np.int64)).to("cuda").to(dtype)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_static_scratch_sizes_match_arena_sizes(dtype):
    # two calls in a row on the shared array, the second with a smaller map:
    # nothing of the first call's counts may leak into the second result
    first = _random_map(27, 70_001, 0.3, 1, dtype)
    second = _random_map(8, 1_337, 0.6, 2, dtype)
    for kernel_map in (first, second):
        expect = _C.cuda_compute_kernel_map_sizes(kernel_map)
        out = torch.full((kernel_map.size(0),), -7, dtype=dtype, device="cuda")
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        assert _C.compute_kernel_map_sizes_static(kernel_map, out) is out
        torch.cuda.synchronize()
        # neither torch's allocator nor the library's arena took device memory
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(out, expect)
        assert torch.equal(out.cpu(), (kernel_map != -1).sum(dim=1).cpu().to(dtype))
    # an empty target set is all zeros, written by a kernel
    empty = torch.empty((5, 0), dtype=dtype, device="cuda")
    out = torch.full((5,), 9, dtype=dtype, device="cuda")
    assert torch.equal(_C.compute_kernel_map_sizes_static(empty, out).cpu(), torch.zeros(5, dtype=dtype))


def test_static_scratch_rejects_maps_beyond_its_size():
    # 2048 offsets x 513 tiles exceed the 2^20 words; the map itself is never read
    tiles = _C.STATIC_SCRATCH_WORDS // 2048 + 1
    kernel_map = torch.empty((2048, tiles * 512), dtype=torch.int32, device="cuda")
    out = torch.empty((2048,), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="static array holds"):
        _C.compute_kernel_map_sizes_static(kernel_map, out)
    _C.cuda_reset_error()
