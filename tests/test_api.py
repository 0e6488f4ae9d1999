"""Host-side API behaviour that needs no GPU: SparseTensor validation, helper
functions, module construction, tunable-config round trips, the drop-in alias."""
import json

import numpy as np
import pytest
import torch

import minuet_amd as minuet
from minuet_amd.utils.helpers import as_tuple


def test_alias_package_points_at_the_same_objects():
    import minuet as alias
    import minuet.nn.functional as AF
    from minuet.nn import SparseConv3d, KernelMapCache
    from minuet.utils.helpers import generate_kernel_offsets
    assert alias.SparseTensor is minuet.SparseTensor
    assert SparseConv3d is minuet.nn.SparseConv3d and KernelMapCache is minuet.nn.KernelMapCache
    assert AF.sparse_convolution_forward is minuet.nn.functional.sparse_convolution_forward
    assert generate_kernel_offsets is minuet.utils.helpers.generate_kernel_offsets
    for name in ("set_kernel_map_cache", "autotune", "load_tunable_config", "dump_tunable_config",
                 "set_gemm_parallel_level"):
        assert getattr(alias, name) is getattr(minuet, name)
    for name in ("arg_sort_coordinates", "build_sorted_index", "query_sorted_index_with_offsets",
                 "unique_coordinates", "compute_kernel_map_masks", "compute_kernel_map_sizes",
                 "cuda_time_gather", "cuda_time_scatter", "cuda_time_gemm", "sparse_convolution_forward",
                 "set_gemm_parallel_level", "cuda_buffer_total_size", "cuda_buffer_used_size",
                 "cuda_free_buffers", "cuda_set_buffer_growth", "cuda_set_buffer_page_size",
                 "cuda_preallocate_buffer", "cuda_reset_error", "global_avg_pool", "global_max_pool",
                 "global_sum_pool", "cat"):
        assert hasattr(AF, name), name


def test_as_tuple():
    assert as_tuple(2) == (2, 2, 2)
    assert as_tuple((1, 2), size=2) == (1, 2)
    assert as_tuple([3, 4, 5]) == (3, 4, 5)
    with pytest.raises(ValueError, match="kernel_size must be a scalar or a iterable of size 3"):
        as_tuple((1, 2), size=3, name="kernel_size")


def test_sparse_tensor_validation_and_properties():
    f = torch.randn(5, 4)
    c = torch.zeros((5, 3), dtype=torch.int32)
    x = minuet.SparseTensor(f, c, stride=2, batch_dims=torch.tensor([0, 2, 5]))
    assert x.stride == (2, 2, 2) and x.batch_size == 2 and x.n == 5 and x.ndim == 3
    assert x.num_features == 4 and x.shape == (5, 4) and x.dtype == torch.float32
    assert minuet.SparseTensor(f, c, batch_dims=torch.tensor([0, 5])).batch_dims is None
    assert minuet.SparseTensor(f, c).batch_size == 1
    with pytest.raises(ValueError, match="must be a 2-D tensor"):
        minuet.SparseTensor(f, c[:, 0])
    with pytest.raises(ValueError, match="features tensor indicate 5 coordinates but expected 4"):
        minuet.SparseTensor(f, c[:4])
    with pytest.raises(ValueError, match="must be int32 or int64"):
        minuet.SparseTensor(f, c.float())
    with pytest.raises(ValueError, match="strides must be a scalar"):
        minuet.SparseTensor(f, c, stride=(1, 2))
    with pytest.raises(ValueError, match="different from expected"):
        x.F = torch.randn(4, 4)
    x.F = torch.ones(5, 4)
    assert x.half().dtype == torch.float16 and x.half().C is x.C
    y = x.clone()
    assert y.C is not x.C and torch.equal(y.C, x.C) and torch.equal(y.batch_dims, x.batch_dims)
    z = x.to(dtype=torch.float64, copy=True)
    assert z.dtype == torch.float64 and z.C.dtype == torch.int32 and x.dtype == torch.float32
    assert x.detach().F.requires_grad is False
    assert x.contiguous() is x and x.cpu() is x


def test_conv_module_construction():
    conv = minuet.nn.SparseConv3d(8, 16, 3, bias=True)
    assert conv.kernel.shape == (27, 8, 16) and conv.bias.shape == (16,)
    bound = 1.0 / np.sqrt(8 * 27)
    assert conv.kernel.abs().max() <= bound and conv.bias.abs().max() <= bound
    assert conv.tunable_config == {"threshold": -1, "gather_tile_size": 0, "scatter_tile_size": 0,
                                   "dataflow": "auto"}
    assert repr(conv) == "SparseConv3d(8, 16, kernel_size=(3, 3, 3))"
    up = minuet.nn.SparseConv(3, 8, 4, 2, stride=2, transposed=True)
    assert "stride=(2, 2, 2)" in repr(up) and "transposed=True" in repr(up) and "bias=False" in repr(up)
    assert up.kernel.abs().max() <= 1.0 / np.sqrt(4 * 8)          # transposed: fan = out_channels
    assert minuet.nn.SparseConv3d(4, 4, 1).is_trivial and not conv.is_trivial
    assert set(conv.state_dict()) == {"kernel", "bias"}
    d = minuet.nn.SparseConv3d(4, 4, 3, dilation=2)
    assert "dilation=(2, 2, 2)" in repr(d)
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cpu")
    for m in (conv, d, minuet.nn.SparseConv3d(4, 4, 3, stride=2)):
        m.set_kernel_map_cache(cache)
    assert conv._allow_shortcut_matmul and not d._allow_shortcut_matmul
    x = minuet.SparseTensor(torch.randn(3, 8), torch.zeros((3, 3), dtype=torch.int32))
    with pytest.raises(ValueError, match="Kernel map cache must be specified"):
        minuet.nn.SparseConv3d(8, 8, 3)(x)


def test_trivial_conv_and_wrappers_on_cpu():
    x = minuet.SparseTensor(torch.randn(6, 4), torch.arange(18, dtype=torch.int32).view(6, 3),
                            batch_dims=torch.tensor([0, 2, 6]))
    conv = minuet.nn.SparseConv3d(4, 5, 1, bias=True)
    with torch.no_grad():
        y = conv(x)
    torch.testing.assert_close(y.F, x.F @ conv.kernel[0] + conv.bias)
    assert y.C is x.C and y.batch_dims is x.batch_dims
    r = minuet.nn.ReLU()(x)
    assert (r.F >= 0).all() and r.C is x.C
    assert minuet.nn.LeakyReLU(0.1)(x).F.shape == x.F.shape and minuet.nn.ReLU6()(x).F.max() <= 6
    bn = minuet.nn.BatchNorm(4).eval()
    torch.testing.assert_close(bn(x).F, x.F / np.sqrt(1 + 1e-5), rtol=1e-5, atol=1e-6)
    both = minuet.nn.functional.cat([x, r])
    assert both.F.shape == (6, 8) and both.C is x.C
    avg = minuet.nn.GlobalAvgPool()(x)
    torch.testing.assert_close(avg, torch.stack([x.F[:2].mean(0), x.F[2:].mean(0)]))
    torch.testing.assert_close(minuet.nn.GlobalSumPool()(x)[1], x.F[2:].sum(0))
    torch.testing.assert_close(minuet.nn.GlobalMaxPool()(x)[0], x.F[:2].max(0)[0])
    single = minuet.SparseTensor(x.F, x.C)
    torch.testing.assert_close(minuet.nn.GlobalAvgPool()(single), x.F.mean(0))


def test_tunable_config_round_trip(tmp_path):
    net = torch.nn.Sequential(minuet.nn.SparseConv3d(4, 8, 3), minuet.nn.ReLU(),
                              torch.nn.Sequential(minuet.nn.SparseConv3d(8, 8, 3)))
    cfg = minuet.dump_tunable_config(net)
    assert set(cfg) == {"0", "1", "2"} and cfg["1"] == {} and set(cfg["2"]) == {"0"}
    cfg = json.loads(json.dumps(cfg))
    cfg["0"]["threshold"] = 0.25
    cfg["2"]["0"]["gather_tile_size"] = 4
    other = torch.nn.Sequential(minuet.nn.SparseConv3d(4, 8, 3), minuet.nn.ReLU(),
                                torch.nn.Sequential(minuet.nn.SparseConv3d(8, 8, 3)))
    minuet.load_tunable_config(other, cfg)
    assert other[0].tunable_config["threshold"] == 0.25
    assert other[2][0].tunable_config["gather_tile_size"] == 4
    path = tmp_path / "cfg.json"
    path.write_text(json.dumps(cfg))
    again = torch.nn.Sequential(minuet.nn.SparseConv3d(4, 8, 3), minuet.nn.ReLU(),
                                torch.nn.Sequential(minuet.nn.SparseConv3d(8, 8, 3)))
    minuet.autotune(again, None, [], cache_path=str(path))        # existing file: load, never run
    assert again[0].tunable_config["threshold"] == 0.25


def test_set_kernel_map_cache_is_recursive():
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cpu")
    net = torch.nn.Sequential(minuet.nn.SparseConv3d(4, 8, 3),
                              torch.nn.Sequential(minuet.nn.ReLU(), minuet.nn.SparseConv3d(8, 8, 3)))
    assert minuet.set_kernel_map_cache(net, cache) is net
    assert net[0]._kernel_map_cache is cache and net[1][1]._kernel_map_cache is cache


def test_random_unique_points():
    from minuet_amd.utils.random import random_unique_points
    pts = random_unique_points(3, 200, -2, 4)
    assert pts.shape == (200, 3) and pts.min() >= -2 and pts.max() <= 4
    assert len({tuple(p) for p in pts.tolist()}) == 200
    with pytest.raises(ValueError):
        random_unique_points(2, 10, 0, 2)
    assert len({tuple(p) for p in random_unique_points(2, 9, 0, 2).tolist()}) == 9


def test_auto_dataflow_rule():
    """Which layer shapes ``dataflow="auto"`` sends to the single-kernel form:
    16-bit rows of up to 128 bytes with up to 128 output channels, rows of up
    to 256 bytes with up to 64 output channels under kernels of more than 8
    offsets, and small fp32 layers with 2^D kernels."""
    prefers = minuet.nn.functional.prefers_implicit
    half, single = torch.float16, torch.float32
    assert prefers(27, 32, 32, half) and prefers(27, 64, 128, half) and prefers(8, 64, 128, torch.bfloat16)
    assert not prefers(27, 64, 256, half)                 # too many output channels
    assert prefers(27, 128, 64, half) and not prefers(27, 128, 128, half)
    assert not prefers(8, 128, 64, half)                  # strided 2^3 kernel: one hit in eight
    assert not prefers(27, 256, 64, half)                 # 512-byte rows
    assert not prefers(27, 30, 32, half)                  # rows not a multiple of 16 bytes
    assert prefers(8, 32, 32, single) and not prefers(27, 32, 32, single) and not prefers(8, 64, 64, single)


def test_lookahead_layout_places_every_output():
    """The plan of a look-ahead session (no GPU needed): every output of every
    recipe entry gets a 256-byte aligned place of its own inside one allocation,
    entries that need a level or map nobody builds are refused."""
    import torch
    from minuet_amd.nn.functional import _C
    from minuet_amd.nn.lookahead import AheadLayout
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cpu")
    one, two = (1, 1, 1), (2, 2, 2)
    sub = (one, one, (3, 3, 3), one)
    down = (one, two, (2, 2, 2), one)
    recipe = (("dense", sub), ("coords", one, two), ("dense", down), ("tables", down, True), ("invert", down))
    layout = AheadLayout(recipe, cache._kernel_offsets, one, 1 << 14, 3, torch.int32, torch.int32, 2)
    assert layout.num_levels == 2 and len(layout.items) == 5
    assert [item.kind for item in layout.items] == [_C.AHEAD_DENSE, _C.AHEAD_COORDS, _C.AHEAD_DENSE,
                                                    _C.AHEAD_TABLES, _C.AHEAD_INVERT]
    assert layout.items[3].dense_item == 2 and layout.items[4].dense_item == 2 and layout.items[3].reorder == 1
    assert layout.items[0].num_offsets == 27 and layout.items[2].num_offsets == 8
    spans = []
    for places, (_, _, _, sizes) in zip(layout.places, layout.plan):
        for place, size in zip(places, sizes):
            if size:
                assert place % 256 == 0
                spans.append((place, place + size))
    spans.sort()
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])) and spans[-1][1] <= layout.total
    layout.bind(1 << 20)
    assert layout.items[0].out0 == (1 << 20) + layout.places[0][0]
    assert layout.items[1].out1 == (1 << 20) + layout.places[1][1]          # batch boundaries of the new level
    for bad in ((("tables", sub, True),), (("coords", two, (4, 4, 4)),), (("dense", down),), ()):
        with pytest.raises(ValueError):
            AheadLayout(bad, cache._kernel_offsets, one, 1 << 14, 3, torch.int32, None, 1)
