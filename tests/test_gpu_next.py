"""The pieces around the hot path: scratch-arena knobs, alternate offset
layouts through the kernel-map cache, pooling / activation modules on the GPU
and the ResNet-style classifier against a float64 replay."""
import numpy as np
import pytest
import torch

import minuet_oracle as orc
import minuet_amd as minuet
from helpers import dev, host, random_cloud, sorted_unique
from minuet_amd.nn import functional as F
from minuet_amd.resnet import SparseResNet
from minuet_amd.synthetic import make_cloud
from test_gpu_unet import Ref, ref_forward, build_input

pytestmark = pytest.mark.gpu

MIB = 1 << 20


def _one_layer(channels=32, n=6000):
    c, _ = sorted_unique(random_cloud(n, 24, seed=6))
    conv = minuet.nn.SparseConv3d(channels, channels, 3, dtype=torch.float16, device="cuda")
    conv.set_kernel_map_cache(minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda"))
    conv.tunable_config["dataflow"] = "gather_gemm_scatter"          # the dataflow with scratch buffers
    x = minuet.SparseTensor(torch.randn(c.shape[0], channels, device="cuda").half(), dev(c))
    return conv, x


def test_scratch_arena_knobs():
    """cuda_preallocate_buffer / free_buffers / set_buffer_page_size / set_buffer_growth /
    buffer_total_size / buffer_used_size act on the arena of the current stream
    (reference: csrc/minuet/cuda/buffer_pool.cu:100-216)."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream), torch.no_grad():
        F.cuda_free_buffers()
        assert F.cuda_buffer_total_size() == 0 and F.cuda_buffer_used_size() == 0
        # preallocate rounds up to whole pages (8 MiB by default) and is kept
        F.cuda_preallocate_buffer(3 * MIB)
        assert F.cuda_buffer_total_size() == 8 * MIB and F.cuda_buffer_used_size() == 0
        F.cuda_preallocate_buffer(5 * MIB)                           # already there: nothing new
        assert F.cuda_buffer_total_size() == 8 * MIB
        F.cuda_preallocate_buffer(20 * MIB)                          # a page of its own
        assert F.cuda_buffer_total_size() == 8 * MIB + 24 * MIB
        # a forward borrows from the arena and hands everything back
        conv, x = _one_layer()
        y = conv(x)
        stream.synchronize()
        assert F.cuda_buffer_used_size() == 0
        total = F.cuda_buffer_total_size()
        assert total >= 32 * MIB
        y2 = conv(x)                                                  # the second pass grows nothing
        stream.synchronize()
        assert F.cuda_buffer_total_size() == total and torch.equal(y.F, y2.F)
        # free gives everything back
        F.cuda_free_buffers()
        assert F.cuda_buffer_total_size() == 0
        # page size: the next page is a multiple of it
        F.cuda_set_buffer_page_size(2 * MIB)
        F.cuda_preallocate_buffer(1)
        assert F.cuda_buffer_total_size() == 2 * MIB
        F.cuda_free_buffers()
        # growth: a request beyond every page allocates (1 + growth) times its size, in whole pages
        F.cuda_set_buffer_page_size(1 * MIB)
        F.cuda_set_buffer_growth(1.0)
        conv(x)
        stream.synchronize()
        doubled = F.cuda_buffer_total_size()
        F.cuda_free_buffers()
        F.cuda_set_buffer_growth(0.0)
        conv(x)
        stream.synchronize()
        tight = F.cuda_buffer_total_size()
        assert 0 < tight < doubled
        F.cuda_free_buffers()
        F.cuda_set_buffer_page_size(8 * MIB)
        F.cuda_set_buffer_growth(1.0)
        # arenas are per stream: the default stream's arena never saw these calls
    other = F.cuda_buffer_total_size()
    with torch.cuda.stream(stream):
        F.cuda_preallocate_buffer(1)
        assert F.cuda_buffer_total_size() == 8 * MIB
    assert F.cuda_buffer_total_size() == other
    # device reset: everything the library holds on the device goes, tensors stay
    keep = torch.arange(10, device="cuda")
    F.cuda_device_reset()
    with torch.cuda.stream(stream):
        assert F.cuda_buffer_total_size() == 0
    assert F.cuda_buffer_total_size() == 0 and keep.sum().item() == 45
    conv, x = _one_layer()
    with torch.no_grad():
        assert torch.isfinite(conv(x).F).all()                       # and the library works on


@pytest.mark.parametrize("layout", ["minuet", "torchsparse", "minkowski"])
@pytest.mark.parametrize("kernel,stride", [(3, 1), (2, 2), ((3, 1, 2), 1)])
@pytest.mark.parametrize("flow", ["gather_gemm_scatter", "implicit"])
def test_layer_through_every_offset_layout(layout, kernel, stride, flow):
    """KernelMapCache(layout=...) only permutes the offset rows, so that weights
    laid out for another engine load as they are (reference: helpers.py:196-210):
    a layer's output equals the oracle's with the offsets of that layout."""
    rng = np.random.default_rng(3)
    c, _ = sorted_unique(random_cloud(5000, 20, seed=12, lo=-6))
    offsets = orc.generate_kernel_offsets(3, kernel, 1, 1, layout=layout)
    feats = rng.normal(size=(c.shape[0], 16))
    conv = minuet.nn.SparseConv3d(16, 32, kernel, stride=stride, dtype=torch.float32, device="cuda")
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda", layout=layout)
    conv.set_kernel_map_cache(cache)
    conv.tunable_config["dataflow"] = flow
    with torch.no_grad():
        y = conv(minuet.SparseTensor(dev(feats).float(), dev(c)))
    weights = host(conv.kernel.detach().double())
    tgt, _ = (c, None) if stride == 1 else orc.target_coordinates(c, None, (stride,) * 3)
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(c, None, tgt, None, offsets, reorder=True)
    ref = orc.sparse_convolution_forward(feats.astype(np.float32).astype(np.float64), weights, esm, etm,
                                         eorder, esizes)
    np.testing.assert_array_equal(host(y.C), tgt)
    err = np.abs(host(y.F.double()) - ref).max()
    assert err <= 1e-5 * np.abs(ref).max(), err
    if layout != "minuet" and np.prod(np.atleast_1d(kernel)) > 1 and not (
            layout == "torchsparse" and int(np.prod(orc.as_tuple(kernel, 3))) % 2 == 0):
        # the layouts differ for this kernel: the default order gives another result
        base = orc.generate_kernel_offsets(3, kernel, 1, 1)
        assert not np.array_equal(base, offsets)


def test_state_dict_names_and_shapes():
    conv = minuet.nn.SparseConv3d(8, 16, 3, bias=True, device="cuda")
    state = conv.state_dict()
    assert list(state) == ["kernel", "bias"]
    assert state["kernel"].shape == (27, 8, 16) and state["bias"].shape == (16,)
    other = minuet.nn.SparseConv3d(8, 16, 3, bias=True, device="cuda")
    other.load_state_dict(state)
    assert torch.equal(other.kernel, conv.kernel) and torch.equal(other.bias, conv.bias)


@pytest.mark.parametrize("batched", [False, True])
def test_pooling_and_activation_modules_on_the_gpu(batched):
    rng = np.random.default_rng(8)
    n = 3000
    feats = rng.normal(size=(n, 24)).astype(np.float32)
    c, bd = sorted_unique(random_cloud(n, 30, seed=4), np.array([0, 1000, 1700, n], dtype=np.int32) if batched else None)
    feats = feats[:c.shape[0]]
    x = minuet.SparseTensor(dev(feats), dev(c), batch_dims=dev(bd))
    spans = [(0, c.shape[0])] if bd is None else list(zip(bd[:-1], bd[1:]))
    for module, reduce in ((minuet.nn.GlobalAvgPool(), np.mean), (minuet.nn.GlobalSumPool(), np.sum),
                           (minuet.nn.GlobalMaxPool(), np.max)):
        got = host(module(x))
        expect = np.stack([reduce(feats[a:b].astype(np.float64), axis=0) for a, b in spans])
        if not batched:
            expect = expect[0]
        np.testing.assert_allclose(got, expect, rtol=1e-5, atol=1e-5)
    for module, fn in ((minuet.nn.ReLU(), lambda v: np.maximum(v, 0)),
                       (minuet.nn.ReLU6(), lambda v: np.clip(v, 0, 6)),
                       (minuet.nn.LeakyReLU(0.2), lambda v: np.where(v > 0, v, 0.2 * v))):
        y = module(minuet.SparseTensor(dev(feats * 4), dev(c), batch_dims=dev(bd)))
        assert torch.equal(y.C, x.C) and y.stride == x.stride
        np.testing.assert_allclose(host(y.F), fn(feats * 4), rtol=1e-6, atol=1e-6)


def _ref_resnet(net, x, levels):
    x = ref_forward(net.stem, x, levels)
    for down, stage in zip(net.down, net.stages):
        x = ref_forward(stage, ref_forward(down, x, levels), levels)
    spans = [(0, x.c.shape[0])] if x.bd is None else list(zip(x.bd[:-1], x.bd[1:]))
    pooled = np.stack([x.f[a:b].mean(axis=0) for a, b in spans])
    weight = host(net.head.weight.detach().double())
    bias = host(net.head.bias.detach().double())
    return pooled @ weight.T + bias


@pytest.mark.parametrize("kind", ["fp32", "fp16"])
def test_resnet_classifier_matches_float64_replay(kind):
    """Stem, three stride-2 stages of two residual blocks, global average pool,
    linear head, on two clouds of the configuration-4 generator at 2 % of their
    size, against the layer-by-layer float64 replay."""
    torch.manual_seed(1)
    dtype = torch.float32 if kind == "fp32" else torch.float16
    coords, bd = build_input(0.02)
    rng = np.random.default_rng(2)
    feats = rng.normal(size=(coords.shape[0], 4))
    net = SparseResNet(4, 10, stem=16, stages=(32, 64, 128), dtype=dtype, device="cuda").eval()
    with torch.no_grad():
        for m in net.modules():
            if isinstance(m, minuet.nn.BatchNorm):
                m.running_mean.uniform_(-0.2, 0.2)
                m.running_var.uniform_(0.5, 1.5)
                m.weight.uniform_(0.8, 1.2)
                m.bias.uniform_(-0.1, 0.1)
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    minuet.set_kernel_map_cache(net, cache)
    x = minuet.SparseTensor(dev(feats).to(dtype), dev(coords), batch_dims=dev(bd))
    with torch.no_grad():
        logits = net(x)
    assert logits.shape == (2, 10)
    ref = _ref_resnet(net, Ref(host(x.F.double()), coords, bd, (1, 1, 1)), {(1, 1, 1): (coords, bd)})
    err = np.abs(host(logits.double()) - ref).max()
    if kind == "fp32":
        assert err <= 1e-5 * np.abs(ref).max(), err
    else:
        assert err <= 2e-2 * np.sqrt(np.mean(ref ** 2)), err
    assert cache.num_coordinate_builds == 3 and cache.num_map_builds == 7
