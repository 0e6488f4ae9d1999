"""GPU parity of Gather -> grouped GEMM -> Scatter and of the module API
against the CPU oracle (fp64).  Tolerances (from the task statement):
fp32: max-abs error <= 1e-5 x max|reference| (relative 1e-5);
fp16 / bf16: max-abs error <= 2e-2 x RMS(reference)."""
import numpy as np
import pytest
import torch

import minuet_oracle as orc
from helpers import dev, host, random_cloud, sorted_unique
import minuet_amd as minuet
from minuet_amd.nn import functional as F
from minuet_amd.nn.functional import _C

pytestmark = pytest.mark.gpu

TORCH = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


def assert_features_close(got, ref, kind):
    got = host(got.float()).astype(np.float64)
    err = np.abs(got - ref).max() if ref.size else 0.0
    if kind == "fp32":
        bound = 1e-5 * max(np.abs(ref).max(), 1e-30)
    else:
        bound = 2e-2 * max(np.sqrt(np.mean(ref ** 2)), 1e-30)
    assert err <= bound, f"{kind}: max-abs error {err:.3e} exceeds {bound:.3e}"


def quantise(array, kind):
    """Round inputs to the feature dtype first so the oracle sees what the GPU sees."""
    return host(torch.from_numpy(array).to(TORCH[kind]).float()).astype(np.float64)


def make_layer_case(seed, n, extent, kernel, cin, cout, kind, stride=1, batched=False):
    rng = np.random.default_rng(seed)
    bd = np.array([0, n // 2, n], dtype=np.int32) if batched else None
    src, sbd = sorted_unique(random_cloud(n, extent, seed=seed, lo=-extent // 2), bd)
    if stride == 1:
        tgt, tbd = src, sbd
    else:
        tgt, tbd = orc.target_coordinates(src, sbd, stride)
    off = orc.generate_kernel_offsets(3, kernel, 1, 1)
    feats = quantise(rng.normal(size=(src.shape[0], cin)), kind)
    k3 = off.shape[0]
    weights = quantise(rng.normal(size=(k3, cin, cout)) / np.sqrt(k3 * cin), kind)
    return src, sbd, tgt, tbd, off, feats, weights


def kernel_map_of(source_masks, target_masks, order, sizes):
    """A KernelMap on the device from the oracle's tables: host copies of sizes
    and order plus the pair list of source rows (buffer row -> source row),
    derived here from the rank table itself."""
    start = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    index = np.full(int(start[-1]), -1, dtype=np.int32)
    for j in range(source_masks.shape[0]):
        hit = np.nonzero(source_masks[j] >= 0)[0]
        index[start[j] + source_masks[j, hit]] = hit
    assert (index >= 0).all()
    return minuet.nn.KernelMap(dev(source_masks), dev(target_masks), dev(order), dev(sizes),
                               sizes_host=sizes, order_host=order, in_idx=dev(index))


@pytest.mark.parametrize("kind", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("kernel,stride,cin,cout,n,extent", [
    (3, 1, 32, 32, 20000, 60), (3, 1, 64, 64, 6000, 25), (2, 2, 64, 128, 20000, 50),
    (3, 1, 4, 32, 5000, 20), (3, 1, 96, 48, 4000, 20), (5, 1, 16, 16, 3000, 16),
    (3, 1, 256, 256, 3000, 16), (3, 1, 24, 40, 2000, 12), (3, 1, 3, 5, 2000, 12),
])
def test_forward_functional(kind, kernel, stride, cin, cout, n, extent):
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(3, n, extent, kernel, cin, cout, kind, stride)
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    dtype = TORCH[kind]
    for shortcut in (False, True):
        for threshold in (-1, 0.3, None):
            out = F.sparse_convolution_forward(
                sources=dev(feats).to(dtype), weights=dev(weights).to(dtype),
                source_masks=dev(esm), target_masks=dev(etm), kernel_map_order=dev(eorder),
                kernel_map_sizes=dev(esizes), gather_tile_size=0, scatter_tile_size=0,
                allow_shortcut_matmul=shortcut and stride == 1, threshold=threshold)
            assert out.dtype == dtype and out.shape == (tgt.shape[0], cout)
            assert_features_close(out, ref, kind)
            # Gather folded into the GEMM: same products, same summation order
            kernel_map = kernel_map_of(esm, etm, eorder, esizes)
            fused = F.sparse_convolution_forward(
                sources=dev(feats).to(dtype), weights=dev(weights).to(dtype), kernel_map=kernel_map,
                gather_tile_size=0, scatter_tile_size=0,
                allow_shortcut_matmul=shortcut and stride == 1, threshold=threshold)
            assert torch.equal(fused, out)
            # weights packed ahead of time (in the layer's own offset order)
            w_dev = dev(weights).to(dtype)
            ahead = F.sparse_convolution_forward(
                sources=dev(feats).to(dtype), weights=w_dev, kernel_map=kernel_map,
                gather_tile_size=0, scatter_tile_size=0,
                allow_shortcut_matmul=shortcut and stride == 1, threshold=threshold,
                packed_weights=F.pack_weights(w_dev))
            assert torch.equal(ahead, out)


@pytest.mark.parametrize("kind", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("activation", [None, "relu", "leaky_relu", "relu6"])
def test_forward_epilogue(kind, activation):
    """act(conv * scale + shift + residual) applied inside Scatter equals the
    same arithmetic on the float64 convolution output."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(11, 6000, 24, 3, 32, 48, kind)
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    conv = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    rng = np.random.default_rng(12)
    scale = rng.uniform(0.5, 1.5, size=48).astype(np.float32)
    shift = rng.uniform(-0.5, 0.5, size=48).astype(np.float32)
    residual = quantise(rng.normal(size=conv.shape), kind)
    dtype = TORCH[kind]
    for use_scale, use_shift, use_residual in [(True, True, True), (False, True, False),
                                               (True, False, False), (False, False, True)]:
        ref = conv.copy()
        if use_scale:
            ref = ref * scale.astype(np.float64)
        if use_shift:
            ref = ref + shift.astype(np.float64)
        if use_residual:
            ref = ref + residual
        if activation == "relu":
            ref = np.maximum(ref, 0.0)
        elif activation == "leaky_relu":
            ref = np.where(ref > 0, ref, ref * 0.2)
        elif activation == "relu6":
            ref = np.clip(ref, 0.0, 6.0)
        epilogue = F.Epilogue(dev(scale) if use_scale else None, dev(shift) if use_shift else None,
                              dev(residual).to(dtype) if use_residual else None, activation, 0.2)
        for shortcut in (False, True):
            out = F.sparse_convolution_forward(
                sources=dev(feats).to(dtype), weights=dev(weights).to(dtype),
                source_masks=dev(esm), target_masks=dev(etm), kernel_map_order=dev(eorder),
                kernel_map_sizes=dev(esizes), gather_tile_size=0, scatter_tile_size=0,
                allow_shortcut_matmul=shortcut, threshold=0, epilogue=epilogue)
            assert_features_close(out, ref, kind)


@pytest.mark.parametrize("kind", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("kernel,stride,cin,cout,n,extent", [
    (3, 1, 32, 32, 20000, 60), (3, 1, 64, 64, 6000, 25), (2, 2, 64, 128, 20000, 50),
    (3, 1, 8, 32, 5000, 20), (3, 1, 24, 48, 4000, 20), (5, 1, 16, 16, 3000, 16),
    (3, 1, 32, 100, 3000, 16), (3, 1, 56, 40, 2000, 12), (1, 1, 32, 12, 999, 12),
    (7, 1, 16, 8, 1500, 10),
    # rows wider than one pipeline stage (chunks of 128 bytes) and more
    # than 128 output channels (channel groups, the last one narrower)
    (3, 1, 128, 128, 4000, 20), (3, 1, 256, 64, 3000, 16), (2, 2, 128, 256, 6000, 30),
    (3, 1, 160, 32, 2000, 12), (3, 1, 96, 200, 2000, 12), (3, 1, 72, 300, 1500, 12),
])
def test_forward_implicit(kind, kernel, stride, cin, cout, n, extent):
    """The single-kernel output-stationary forward against the float64 oracle:
    dense kernel map in the original offset order, no rank tables."""
    if not _C.implicit_forward_supported(cin, cout, TORCH[kind]):
        pytest.skip("a shape this form does not take")
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(4, n, extent, kernel, cin, cout, kind, stride)
    kmap = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd)
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    conv = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    dtype = TORCH[kind]
    assert _C.implicit_forward_supported(cin, cout, dtype)
    out = _C.sparse_convolution_forward_implicit(dev(feats).to(dtype), dev(weights).to(dtype), dev(kmap))
    assert out.dtype == dtype and out.shape == (tgt.shape[0], cout)
    assert_features_close(out, conv, kind)
    w_dev = dev(weights).to(dtype)
    assert torch.equal(out, _C.sparse_convolution_forward_implicit(
        dev(feats).to(dtype), w_dev, dev(kmap), packed_weights=F.pack_weights(w_dev)))
    rng = np.random.default_rng(5)
    scale = rng.uniform(0.5, 1.5, size=cout).astype(np.float32)
    shift = rng.uniform(-0.5, 0.5, size=cout).astype(np.float32)
    residual = quantise(rng.normal(size=conv.shape), kind)
    ref = np.maximum(conv * scale.astype(np.float64) + shift.astype(np.float64) + residual, 0.0)
    out = _C.sparse_convolution_forward_implicit(
        dev(feats).to(dtype), dev(weights).to(dtype), dev(kmap),
        epilogue=F.Epilogue(dev(scale), dev(shift), dev(residual).to(dtype), "relu"))
    assert_features_close(out, ref, kind)


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("kernel,stride,cin,cout,n,extent", [
    (3, 1, 4, 32, 20000, 60), (3, 1, 2, 32, 5000, 20), (3, 1, 8, 32, 6000, 25), (3, 1, 4, 16, 3000, 16),
    (3, 1, 4, 64, 4000, 20), (3, 1, 4, 100, 2000, 12), (2, 2, 4, 128, 6000, 30), (5, 1, 4, 32, 3000, 16),
    (5, 1, 2, 48, 2500, 14), (1, 1, 4, 12, 999, 12), ((3, 1, 2), 1, 8, 24, 3000, 16), (3, 1, 4, 32, 31, 4),
])
def test_forward_implicit_narrow_rows(kind, kernel, stride, cin, cout, n, extent):
    """Source rows of 4, 8 or 16 bytes (the offsets side by side along K, the
    weights in LDS as they are) against the float64 oracle."""
    dtype = TORCH[kind]
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(6, n, extent, kernel, cin, cout, kind, stride)
    assert _C.implicit_forward_supported(cin, cout, dtype, off.shape[0])
    kmap = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd)
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    conv = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    _C.profile_enable(True)
    out = _C.sparse_convolution_forward_implicit(dev(feats).to(dtype), dev(weights).to(dtype), dev(kmap))
    stages = [name for name, _ in _C.profile_read()]
    _C.profile_enable(False)
    assert "pack_weights" not in stages               # the short-row kernel reads the weights as they are
    assert out.dtype == dtype and out.shape == (tgt.shape[0], cout)
    assert_features_close(out, conv, kind)
    rng = np.random.default_rng(5)
    scale = rng.uniform(0.5, 1.5, size=cout).astype(np.float32)
    shift = rng.uniform(-0.5, 0.5, size=cout).astype(np.float32)
    residual = quantise(rng.normal(size=conv.shape), kind)
    ref = conv * scale.astype(np.float64) + shift.astype(np.float64) + residual
    # (no ReLU for bf16: it halves the RMS the bound is taken from, and rounding
    # an output of five times that RMS to 8 bits then exceeds the bound by itself)
    activation = "relu" if kind == "fp16" else None
    if activation == "relu":
        ref = np.maximum(ref, 0.0)
    out = _C.sparse_convolution_forward_implicit(
        dev(feats).to(dtype), dev(weights).to(dtype), dev(kmap),
        epilogue=F.Epilogue(dev(scale), dev(shift), dev(residual).to(dtype), activation))
    assert_features_close(out, ref, kind)


def test_forward_implicit_rejects_unsupported_shapes():
    assert not _C.implicit_forward_supported(4, 32, torch.float16)       # 8-byte rows, kernel unknown
    assert _C.implicit_forward_supported(4, 32, torch.float16, 27)
    assert not _C.implicit_forward_supported(4, 128, torch.float16, 125)  # weights beyond LDS
    assert not _C.implicit_forward_supported(3, 32, torch.float16, 27)    # 6-byte rows
    assert not _C.implicit_forward_supported(1, 32, torch.float32, 27)
    assert not _C.implicit_forward_supported(32, 30, torch.float16)
    assert not _C.implicit_forward_supported(32, 516, torch.float16)
    assert not _C.implicit_forward_supported(1032, 32, torch.float16)    # rows beyond 2048 bytes
    assert _C.implicit_forward_supported(128, 256, torch.float16)
    assert _C.implicit_forward_supported(64, 32, torch.float32)
    kmap = torch.full((27, 10), -1, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="Unsupported channel counts"):
        _C.sparse_convolution_forward_implicit(torch.zeros(10, 4, device="cuda").half(),
                                               torch.zeros(125, 4, 128, device="cuda").half(),
                                               torch.full((125, 10), -1, dtype=torch.int32, device="cuda"))
    with pytest.raises(RuntimeError, match="Unsupported channel counts"):
        _C.sparse_convolution_forward_implicit(torch.zeros(10, 3, device="cuda").half(),
                                               torch.zeros(27, 3, 32, device="cuda").half(), kmap)
    out = _C.sparse_convolution_forward_implicit(torch.ones(10, 8, device="cuda").half(),
                                                 torch.ones(27, 8, 32, device="cuda").half(), kmap)
    assert torch.count_nonzero(out).item() == 0                        # no hits: all zero


def test_packed_weights_follow_the_parameter():
    """A layer repacks its weights when (and only when) the parameter changes."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(2, 3000, 16, 3, 32, 32, "fp16")
    conv = minuet.nn.SparseConv3d(32, 32, 3, dtype=torch.float16, device="cuda")
    conv.set_kernel_map_cache(minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda"))
    x = minuet.SparseTensor(dev(feats).half(), dev(src))
    with torch.no_grad():
        for flow in ("gather_gemm_scatter", "implicit"):
            conv.tunable_config["dataflow"] = flow
            a = conv(x).F.clone()
            first = conv._packed[2]
            assert conv(x).F.equal(a) and conv._packed[2] is first
            conv.kernel.mul_(2.0)                      # in place: same storage, new version
            b = conv(x).F
            assert conv._packed[2] is not first
            assert (b.float() - 2 * a.float()).abs().max().item() <= 2e-2 * a.float().pow(2).mean().sqrt().item()
            conv.kernel.mul_(0.5)
    with pytest.raises(RuntimeError, match="does not belong"):
        F.sparse_convolution_forward(
            sources=x.F, weights=conv.kernel, source_masks=None, target_masks=None, kernel_map_order=None,
            kernel_map_sizes=None, gather_tile_size=0, scatter_tile_size=0, dataflow="gather_gemm_scatter",
            packed_weights=torch.zeros(3, device="cuda").half()) if False else _C._check_packed(
                torch.zeros(3, device="cuda").half(), conv.kernel)


@pytest.mark.parametrize("cin", [1, 3, 4, 5, 12])
def test_narrow_rows_are_padded_for_the_single_kernel_form(cin):
    """16-bit layers whose rows are not a multiple of 16 bytes (stems) still
    take the implicit dataflow: rows of 4 or 8 bytes as they are, others
    through zero channels appended on the fly."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(13, 4000, 18, 3, cin, 32, "fp16")
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    conv = minuet.nn.SparseConv3d(cin, 32, 3, dtype=torch.float16, device="cuda")
    conv.kernel.data.copy_(dev(weights).half())
    conv.set_kernel_map_cache(minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda"))
    x = minuet.SparseTensor(dev(feats).half(), dev(src))
    with torch.no_grad():
        _C.profile_enable(True)
        y = conv(x)
        stages = [name for name, _ in _C.profile_read()]
        _C.profile_enable(False)
    assert "implicit" in stages and "scatter" not in stages
    assert_features_close(y.F, ref, "fp16")


def test_layers_on_empty_and_tiny_clouds():
    """No voxels, one voxel, and a batch with an empty cloud, through both
    dataflows of the module."""
    for flow in ("gather_gemm_scatter", "implicit"):
        conv = minuet.nn.SparseConv3d(16, 32, 3, dtype=torch.float16, device="cuda")
        down = minuet.nn.SparseConv3d(16, 16, 2, stride=2, dtype=torch.float16, device="cuda")
        for m in (conv, down):
            m.tunable_config["dataflow"] = flow
        with torch.no_grad():
            for coords, bd in ((np.zeros((0, 3), dtype=np.int32), None),
                               (np.array([[3, -2, 7]], dtype=np.int32), None),
                               (np.array([[0, 0, 0], [0, 0, 1], [5, 5, 5]], dtype=np.int32),
                                np.array([0, 0, 2, 3], dtype=np.int32))):
                cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
                conv.set_kernel_map_cache(cache)
                down.set_kernel_map_cache(cache)
                n = coords.shape[0]
                feats = torch.ones(n, 16, device="cuda").half()
                x = minuet.SparseTensor(feats, dev(coords), batch_dims=dev(bd))
                y = conv(x)
                assert y.F.shape == (n, 32) and torch.equal(y.C, x.C)
                if n:
                    w = host(conv.kernel.detach().float()).astype(np.float64)
                    ref, _, _, _ = orc.conv_layer(coords, bd, np.ones((n, 16)), w, 3)
                    assert_features_close(y.F, ref, "fp16")
                z = down(x)
                expect, ebd = orc.target_coordinates(coords, bd, 2) if n else (coords, bd)
                np.testing.assert_array_equal(host(z.C), expect)
                assert z.F.shape == (expect.shape[0], 16)


def test_epilogue_rejects_bad_operands():
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(5, 500, 8, 3, 32, 32, "fp32")
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    args = dict(sources=dev(feats).float(), weights=dev(weights).float(), source_masks=dev(esm),
                target_masks=dev(etm), kernel_map_order=dev(eorder), kernel_map_sizes=dev(esizes),
                gather_tile_size=0, scatter_tile_size=0)
    with pytest.raises(RuntimeError, match="epilogue scale"):
        F.sparse_convolution_forward(epilogue=F.Epilogue(scale=torch.ones(31, device="cuda")), **args)
    with pytest.raises(RuntimeError, match="epilogue residual"):
        F.sparse_convolution_forward(
            epilogue=F.Epilogue(residual=torch.ones(tgt.shape[0], 32, device="cuda").half()), **args)
    with pytest.raises(ValueError, match="unknown activation"):
        F.Epilogue(activation="gelu")


def test_fused_sequential_matches_modules():
    """Sequential(conv, BatchNorm, LeakyReLU) folded into one pass: equal to the
    module-by-module result within fp16 rounding in evaluation mode, and
    exactly the module-by-module path in training mode."""
    torch.manual_seed(3)
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(21, 5000, 20, 3, 16, 32, "fp16")
    plain = torch.nn.Sequential(
        minuet.nn.SparseConv3d(16, 32, 3, bias=True, dtype=torch.float16, device="cuda"),
        minuet.nn.BatchNorm(32, dtype=torch.float16, device="cuda"),
        minuet.nn.LeakyReLU(0.1))
    plain[1].running_mean.uniform_(-0.2, 0.2)
    plain[1].running_var.uniform_(0.5, 1.5)
    plain[0].bias.data.uniform_(-0.3, 0.3)
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    minuet.set_kernel_map_cache(plain, cache)
    fused = minuet.nn.fuse_conv_norm_act(plain)
    assert isinstance(fused, minuet.nn.FusedSequential)
    assert list(fused.state_dict().keys()) == list(plain.state_dict().keys())
    x = minuet.SparseTensor(dev(feats).half(), dev(src))
    with torch.no_grad():
        plain.eval(), fused.eval()
        a, b = plain(x), fused(x)
        assert torch.equal(a.C, b.C)
        rms = a.F.float().pow(2).mean().sqrt().item()
        assert (a.F.float() - b.F.float()).abs().max().item() <= 2e-2 * rms
        # float64 replay of the three modules
        w = host(plain[0].kernel.double())
        esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
        ref = orc.sparse_convolution_forward(feats, w, esm, etm, eorder, esizes) + host(plain[0].bias.double())
        bn = plain[1]
        ref = (ref - host(bn.running_mean.double())) / np.sqrt(host(bn.running_var.double()) + bn.eps)
        ref = ref * host(bn.weight.double()) + host(bn.bias.double())
        ref = np.where(ref > 0, ref, 0.1 * ref)
        assert_features_close(b.F, ref, "fp16")
    plain.train(), fused.train()
    torch.manual_seed(1)
    a = plain(x)
    assert torch.equal(fused(x).F, a.F)       # batch statistics: nothing is folded


@pytest.mark.parametrize("tile", [1, 2, 4, 8, 16, 32])
def test_forward_tile_sizes(tile):
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(5, 5000, 20, 3, 32, 64, "fp16")
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    out = F.sparse_convolution_forward(
        sources=dev(feats).half(), weights=dev(weights).half(), source_masks=dev(esm),
        target_masks=dev(etm), kernel_map_order=dev(eorder), kernel_map_sizes=dev(esizes),
        gather_tile_size=tile, scatter_tile_size=tile, allow_shortcut_matmul=True, threshold=-1)
    assert_features_close(out, ref, "fp16")


def test_forward_rejects_bad_tile():
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(5, 500, 8, 3, 32, 32, "fp32")
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    with pytest.raises(RuntimeError, match="Unsupported num_source_features"):
        F.sparse_convolution_forward(
            sources=dev(feats).float(), weights=dev(weights).float(), source_masks=dev(esm),
            target_masks=dev(etm), kernel_map_order=dev(eorder), kernel_map_sizes=dev(esizes),
            gather_tile_size=5, scatter_tile_size=1)


def test_forward_no_reorder_int64_index():
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(8, 4000, 18, 3, 32, 32, "fp32")
    esm, etm, _, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=False,
                                                  index_dtype=np.int64)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, None, esizes)
    out = F.sparse_convolution_forward(
        sources=dev(feats).float(), weights=dev(weights).float(), source_masks=dev(esm),
        target_masks=dev(etm), kernel_map_order=None, kernel_map_sizes=dev(esizes),
        gather_tile_size=4, scatter_tile_size=4, threshold=0)
    assert_features_close(out, ref, "fp32")


def _as_sparse(coords, bd, feats, dtype):
    return minuet.SparseTensor(dev(feats).to(dtype), dev(coords), batch_dims=dev(bd))


def test_kernel_map_invert_matches_brute_force():
    src, sbd = sorted_unique(random_cloud(4000, 20, seed=9, lo=-10))
    tgt, tbd = orc.target_coordinates(src, sbd, 2)
    off = orc.generate_kernel_offsets(3, 2, 1, 1)
    kmap = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd)
    expect = np.full((off.shape[0], src.shape[0]), -1, dtype=np.int32)
    for o in range(kmap.shape[0]):
        for t in range(kmap.shape[1]):
            if kmap[o, t] >= 0:
                assert expect[o, kmap[o, t]] == -1
                expect[o, kmap[o, t]] = t
    got = _C.kernel_map_invert(dev(kmap), src.shape[0])
    np.testing.assert_array_equal(host(got), expect)
    assert _C.kernel_map_invert(dev(kmap[:, :0]), 5).eq(-1).all()


@pytest.mark.parametrize("dataflow", ["gather_gemm_scatter", "implicit"])
@pytest.mark.parametrize("kind", ["fp32", "fp16"])
@pytest.mark.parametrize("batched", [False, True])
def test_module_down_sub_up(kind, batched, dataflow):
    """stride-2 conv -> submanifold conv -> transposed conv sharing one cache,
    through either dataflow."""
    dtype = TORCH[kind]
    rng = np.random.default_rng(2)
    bd = np.array([0, 7000, 15000], dtype=np.int32) if batched else None
    c, bd = sorted_unique(random_cloud(15000, 40, seed=4, lo=-20), bd)
    feats = quantise(rng.normal(size=(c.shape[0], 16)), kind)
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    down = minuet.nn.SparseConv3d(16, 32, 2, stride=2, bias=True, dtype=dtype, device="cuda")
    sub = minuet.nn.SparseConv3d(32, 32, 3, dtype=dtype, device="cuda")
    up = minuet.nn.SparseConv(3, 32, 16, 2, stride=2, transposed=True, dtype=dtype, device="cuda")
    net = torch.nn.Sequential(down, sub, up)
    minuet.set_kernel_map_cache(net, cache)
    for conv in net:
        conv.tunable_config["dataflow"] = dataflow
    x = _as_sparse(c, bd, feats, dtype)
    with torch.no_grad():
        y1 = down(x)
        y2 = sub(y1)
        y3 = up(y2)
    assert cache.num_map_builds == 2 and cache.num_coordinate_builds == 1
    w = lambda conv: host(conv.kernel.detach().float()).astype(np.float64)
    r1, c1, bd1, s1 = orc.conv_layer(c, bd, feats, w(down), 2, stride=2,
                                     bias=host(down.bias.detach().float()).astype(np.float64))
    np.testing.assert_array_equal(host(y1.C), c1)
    assert y1.stride == (2, 2, 2) and s1 == (2, 2, 2)
    if batched:
        np.testing.assert_array_equal(host(y1.batch_dims), bd1)
    assert_features_close(y1.F, r1, kind)
    r1q = quantise(host(y1.F.float()).astype(np.float64), kind)
    r2, c2, bd2, s2 = orc.conv_layer(c1, bd1, r1q, w(sub), 3, source_stride=2)
    np.testing.assert_array_equal(host(y2.C), c2)
    assert_features_close(y2.F, r2, kind)
    r2q = quantise(host(y2.F.float()).astype(np.float64), kind)
    r3, c3, bd3, s3 = orc.conv_layer(c2, bd2, r2q, w(up), 2, stride=2, source_stride=2,
                                     transposed_from=(c, bd, 1))
    np.testing.assert_array_equal(host(y3.C), c)
    assert y3.stride == (1, 1, 1)
    assert_features_close(y3.F, r3, kind)


@pytest.mark.parametrize("dataflow", ["gather_gemm_scatter", "implicit", "list_driven"])
@pytest.mark.parametrize("kernel_size,dilation,stride,source_stride", [
    (3, 2, 1, 1), ((3, 1, 2), (2, 1, 3), 1, 1), ((1, 3, 3), 1, (1, 2, 2), 1), (3, (1, 2, 1), 1, (2, 2, 1)),
    ((2, 3, 1), 1, (2, 1, 1), (1, 2, 2)),
])
def test_module_dilated_and_anisotropic_kernels(kernel_size, dilation, stride, source_stride, dataflow):
    """Dilation, per-dimension kernel sizes and strides, and inputs that already
    carry a tensor stride (the offsets scale with it, helpers.py:165-212),
    through every dataflow against the oracle's layer."""
    rng = np.random.default_rng(6)
    ss = np.asarray(orc.as_tuple(source_stride, 3))
    c, _ = sorted_unique(random_cloud(6000, 14, seed=9, lo=-7) * ss)
    feats = quantise(rng.normal(size=(c.shape[0], 16)), "fp16")
    conv = minuet.nn.SparseConv3d(16, 24, kernel_size, stride=stride, dilation=dilation, dtype=torch.float16,
                                  device="cuda")
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    conv.set_kernel_map_cache(cache)
    conv.tunable_config["dataflow"] = dataflow
    x = minuet.SparseTensor(dev(feats).half(), dev(c), stride=orc.as_tuple(source_stride, 3))
    with torch.no_grad():
        y = conv(x)
    ref, rc, _, rs = orc.conv_layer(c, None, feats, host(conv.kernel.detach().float()).astype(np.float64),
                                    kernel_size, stride=stride, dilation=dilation, source_stride=source_stride)
    np.testing.assert_array_equal(host(y.C), rc)
    assert tuple(y.stride) == tuple(rs)
    assert_features_close(y.F, ref, "fp16")


@pytest.mark.parametrize("dataflow", ["gather_gemm_scatter", "implicit"])
@pytest.mark.parametrize("ndim,kernel_size,extent", [(1, 5, 3000), (2, 3, 90), (4, 3, 9), (4, 2, 9)])
def test_module_other_dimensionalities(ndim, kernel_size, extent, dataflow):
    """1-D, 2-D and 4-D layers (csrc/minuet/enabled_arguments.h:3-22 enables
    ndim 1..4): a submanifold layer, a strided one and its transposed twin
    against the oracle's layers."""
    rng = np.random.default_rng(10 + ndim)
    cloud = rng.integers(-extent // 2, extent // 2, size=(4000, ndim)).astype(np.int32)
    c, _ = sorted_unique(cloud)
    feats = quantise(rng.normal(size=(c.shape[0], 8)), "fp16")
    factory = dict(dtype=torch.float16, device="cuda")
    sub = minuet.nn.SparseConv(ndim, 8, 16, kernel_size, **factory)
    down = minuet.nn.SparseConv(ndim, 16, 16, 2, stride=2, **factory)
    up = minuet.nn.SparseConv(ndim, 16, 8, 2, stride=2, transposed=True, **factory)
    cache = minuet.nn.KernelMapCache(ndim=ndim, dtype=torch.int32, device="cuda")
    for conv in (sub, down, up):
        conv.set_kernel_map_cache(cache)
        conv.tunable_config["dataflow"] = dataflow
    with torch.no_grad():
        y1 = sub(minuet.SparseTensor(dev(feats).half(), dev(c)))
        y2 = down(y1)
        y3 = up(y2)
    w = lambda conv: host(conv.kernel.detach().float()).astype(np.float64)
    r1, c1, _, s1 = orc.conv_layer(c, None, feats, w(sub), kernel_size)
    np.testing.assert_array_equal(host(y1.C), c1)
    assert_features_close(y1.F, r1, "fp16")
    q1 = quantise(host(y1.F.float()).astype(np.float64), "fp16")
    r2, c2, _, s2 = orc.conv_layer(c1, None, q1, w(down), 2, stride=2)
    np.testing.assert_array_equal(host(y2.C), c2)
    assert tuple(y2.stride) == (2,) * ndim == tuple(s2)
    assert_features_close(y2.F, r2, "fp16")
    q2 = quantise(host(y2.F.float()).astype(np.float64), "fp16")
    r3, c3, _, _ = orc.conv_layer(c2, None, q2, w(up), 2, stride=2, source_stride=2, transposed_from=(c, None, 1))
    np.testing.assert_array_equal(host(y3.C), c)
    assert_features_close(y3.F, r3, "fp16")


def test_module_errors_and_trivial():
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    c, _ = sorted_unique(random_cloud(500, 8, seed=1))
    x = minuet.SparseTensor(torch.randn(c.shape[0], 8, device="cuda"), dev(c))
    conv = minuet.nn.SparseConv3d(8, 8, 3, device="cuda")
    with pytest.raises(ValueError, match="Kernel map cache must be specified"):
        conv(x)
    up = minuet.nn.SparseConv(3, 8, 8, 2, stride=2, transposed=True, device="cuda")
    up.set_kernel_map_cache(cache)
    x2 = minuet.SparseTensor(x.F, x.C, stride=2)
    with pytest.raises(RuntimeError, match="non-transposed layer"):
        up(x2)
    one = minuet.nn.SparseConv3d(8, 4, 1, device="cuda")
    with torch.no_grad():
        y = one(x)
    torch.testing.assert_close(y.F, x.F @ one.kernel.view(8, 4))
    with pytest.raises(NotImplementedError):
        F.arg_sort_coordinates(torch.zeros((3, 3), dtype=torch.int32))


def test_autotune_and_timers(tmp_path):
    c, _ = sorted_unique(random_cloud(6000, 24, seed=6))
    x = minuet.SparseTensor(torch.randn(c.shape[0], 32, device="cuda").half(), dev(c))
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    net = torch.nn.Sequential(minuet.nn.SparseConv3d(32, 64, 3, dtype=torch.float16, device="cuda"),
                              minuet.nn.ReLU(),
                              minuet.nn.SparseConv3d(64, 32, 3, dtype=torch.float16, device="cuda"))
    minuet.set_kernel_map_cache(net, cache)
    minuet.nn.SparseConv.__NUM_TUNING_ROUNDS__ = 1
    minuet.nn.SparseConv.__AVAILABLE_THRESHOLD__ = [-1, 0.5, None]
    minuet.nn.SparseConv.__TUNE_THRESHOLD__ = True          # the reference's sweep, off by default here
    path = str(tmp_path / "tuned" / "config.json")
    with torch.no_grad():
        before = net(x).F.clone()
        minuet.autotune(net, cache, [x], cache_path=path)
        cache.reset()
        after = net(x).F
    cfg = minuet.dump_tunable_config(net)
    assert set(cfg["0"].keys()) == {"threshold", "gather_tile_size", "scatter_tile_size", "dataflow"}
    assert cfg["0"]["dataflow"] in ("gather_gemm_scatter", "implicit", "list_driven")
    assert 32 % cfg["0"]["gather_tile_size"] == 0 and 64 % cfg["0"]["scatter_tile_size"] == 0
    # the tuned layer may run the other dataflow: equal to rounding, not bit for bit
    rms = before.float().pow(2).mean().sqrt().item()
    assert (before.float() - after.float()).abs().max().item() <= 2e-2 * rms
    import json, os
    assert os.path.exists(path)
    with open(path) as fh:
        saved = json.load(fh)
    assert saved["0"]["gather_tile_size"] == cfg["0"]["gather_tile_size"]
    # without the sweep the tuner leaves the threshold that pads nothing
    minuet.nn.SparseConv.__TUNE_THRESHOLD__ = False
    net[0].tunable_config["threshold"] = 0.5
    with torch.no_grad():
        minuet.autotune(net, cache, [x])
    assert net[0].tunable_config["threshold"] == -1
    assert F.cuda_buffer_used_size() == 0


def test_cached_weights_are_dropped_on_request_and_by_the_module_hooks():
    """Packed kernels and folded BatchNorm constants follow in-place updates of
    the parameters by themselves; writes through ``.data`` (which bump no
    version counter) need ``invalidate_cached_weights``; ``reset_parameters``
    and ``load_state_dict`` drop the copies themselves."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(21, 3000, 16, 3, 32, 32, "fp16")
    conv = minuet.nn.SparseConv3d(32, 32, 3, dtype=torch.float16, device="cuda")
    norm = minuet.nn.BatchNorm(32, device="cuda").eval()
    net = minuet.nn.FusedSequential(conv, norm, minuet.nn.ReLU()).eval()
    minuet.set_kernel_map_cache(net, minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda"))
    x = minuet.SparseTensor(dev(feats).half(), dev(src))
    rms = lambda t: t.float().pow(2).mean().sqrt().item()
    close = lambda a, b: (a.float() - b.float()).abs().max().item() <= 2e-2 * max(rms(b), 1e-6)
    with torch.no_grad():
        for flow in ("gather_gemm_scatter", "implicit"):
            conv.tunable_config["dataflow"] = flow
            a = conv(x).F.clone()
            conv.kernel.data.mul_(2.0)                 # no version bump: the packed copy is stale
            conv.invalidate_cached_weights()
            assert close(conv(x).F, 2 * a.float())
            conv.kernel.data.mul_(0.5)
            minuet.invalidate_cached_weights(net)      # the model-wide form
            assert close(conv(x).F, a)
        # reset_parameters after a forward: the output follows the new weights
        before = conv(x).F.clone()
        conv.reset_parameters()
        after = conv(x).F
        conv.invalidate_cached_weights()
        assert torch.equal(conv(x).F, after) and not torch.equal(after, before)
        # load_state_dict
        state = {k: v.clone() for k, v in net.state_dict().items()}
        y0 = net(x).F.clone()
        conv.kernel.mul_(3.0)
        norm.weight.data.fill_(0.25)
        minuet.invalidate_cached_weights(net)
        assert not close(net(x).F, y0)
        net.load_state_dict(state)
        assert close(net(x).F, y0)
        # the folded BatchNorm: a .data write shows after invalidation
        norm.bias.data.add_(1.0)
        minuet.invalidate_cached_weights(net)
        y1 = net(x).F
        ref = torch.relu(norm(conv(x)).F.float())
        assert close(y1, ref)


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("cin,cout", [(32, 64), (64, 64), (48, 64), (16, 40)])
def test_forward_implicit_two_target_blocks_per_wavefront(kind, cin, cout):
    """Clouds of more than 2^19 targets with 33..64 output channels run the
    single-kernel forward with two target blocks per wavefront (256 targets per
    workgroup, a ragged last tile): against the three-kernel dataflow on every
    row, and against float64 sums written out here on a sample of rows."""
    dtype = TORCH[kind]
    n = (1 << 19) + 77
    rng = np.random.default_rng(77)
    extent = 300
    flat = rng.choice(extent ** 3, size=n, replace=False)
    flat.sort()                                          # lexicographic order of (x, y, z)
    coords = np.stack([flat // (extent * extent), (flat // extent) % extent, flat % extent], 1).astype(np.int32)
    off = orc.generate_kernel_offsets(3, 3, 1, 1)
    c_dev = dev(coords)
    built = _C.kernel_map_build(c_dev, c_dev, off.astype(np.int64), None, None, reorder=True,
                                want_masks=True, want_lists=True, want_dense=True)
    kmap = built["kernel_map"]
    feats = torch.from_numpy(rng.normal(size=(n, cin))).to(dtype).cuda()
    weights = torch.from_numpy(rng.normal(size=(27, cin, cout)) / np.sqrt(27 * cin)).to(dtype).cuda()
    scale = dev(rng.uniform(0.5, 1.5, size=cout).astype(np.float32))
    shift = dev(rng.uniform(-0.5, 0.5, size=cout).astype(np.float32))
    residual = torch.from_numpy(rng.normal(size=(n, cout))).to(dtype).cuda()
    kernel_map = minuet.nn.KernelMap(built["source_masks"], built["target_masks"], built["order"],
                                     built["sizes"], sizes_host=built["sizes_host"],
                                     order_host=built["order_host"], in_idx=built["in_idx"])
    sample = rng.choice(n, size=1500, replace=False)
    sample[:3] = (0, n - 1, n - 2)                       # the ragged last tile is in the sample
    # the sampled rows of the kernel map, checked against a search over packed keys
    keys = flat.astype(np.int64)
    for o in range(27):
        q = coords[sample].astype(np.int64) + off[o]
        inside = ((q >= 0) & (q < extent)).all(1)
        qk = (q[:, 0] * extent + q[:, 1]) * extent + q[:, 2]
        pos = np.searchsorted(keys, qk)
        pos_c = np.minimum(pos, n - 1)
        hit = inside & (keys[pos_c] == qk)
        np.testing.assert_array_equal(host(kmap[o, sample]), np.where(hit, pos_c, -1))
    km = host(kmap[:, sample])
    f64, w64 = host(feats.double()), host(weights.double())
    plain = np.zeros((sample.shape[0], cout))
    for o in range(27):
        rows = np.nonzero(km[o] >= 0)[0]
        plain[rows] += f64[km[o, rows]] @ w64[o]
    fused = np.maximum(plain * host(scale).astype(np.float64) + host(shift).astype(np.float64)
                       + host(residual.double())[sample], 0.0)
    for epilogue, ref in ((None, plain), (F.Epilogue(scale, shift, residual, "relu"), fused)):
        out = _C.sparse_convolution_forward_implicit(feats, weights, kmap, epilogue=epilogue)
        assert out.shape == (n, cout) and torch.isfinite(out).all()
        assert_features_close(out[sample], ref, kind)
        three = F.sparse_convolution_forward(
            sources=feats, weights=weights, kernel_map=kernel_map, gather_tile_size=0, scatter_tile_size=0,
            allow_shortcut_matmul=True, threshold=-1, epilogue=epilogue, dataflow="gather_gemm_scatter")
        # two roundings of the same sums: 2e-2 of the RMS, or one unit in the
        # last place of the largest value where that is more (bf16 keeps 8 bits)
        diff = (out.float() - three.float()).abs().max().item()
        ulp = three.float().abs().max().item() * 2.0 ** (-7 if kind == "bf16" else -10)
        assert diff <= max(2e-2 * three.float().pow(2).mean().sqrt().item(), ulp), diff


def test_kernel_map_object_is_the_fast_path(monkeypatch):
    """KernelMapCache returns a KernelMap that unpacks like the reference's
    4-tuple; handing it to F.sparse_convolution_forward keeps the pass free of
    read-backs and separate gathers whatever happened to the tables themselves
    (clones, casts), while the four bare tensors run the reference's way."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(5, 4000, 18, 3, 32, 32, "fp32")
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    c = dev(src)
    kernel_map = cache.get_kernel_map(c, 1, None, c, 1, None, 3, 1)
    assert isinstance(kernel_map, minuet.nn.KernelMap) and len(kernel_map) == 4
    source_masks, target_masks, order, sizes = kernel_map                  # the reference's tuple
    assert kernel_map.nnz == int(host(sizes).sum()) and kernel_map.num_offsets == 27
    assert kernel_map.in_idx.numel() == kernel_map.nnz and kernel_map.dense.shape == (27, src.shape[0])
    seen = []
    real, real_map = _C.cuda_sparse_convolution_forward, _C.sparse_convolution_forward_map

    def spy(*args, **kwargs):
        seen.append((kwargs.get("kernel_map_sizes_host") is not None, kwargs.get("gather_index") is not None))
        return real(*args, **kwargs)

    def spy_map(sources, weights, kernel_map, *args, **kwargs):
        # the KernelMap's own entry: host sizes and pair lists come with the map
        seen.append((kernel_map.sizes_host is not None, kernel_map.in_idx is not None))
        return real_map(sources, weights, kernel_map, *args, **kwargs)

    monkeypatch.setattr(_C, "cuda_sparse_convolution_forward", spy)
    monkeypatch.setattr(_C, "sparse_convolution_forward_map", spy_map)
    f, w = dev(feats).float(), dev(weights).float()
    common = dict(gather_tile_size=0, scatter_tile_size=0, allow_shortcut_matmul=True, threshold=-1,
                  dataflow="gather_gemm_scatter")
    a = F.sparse_convolution_forward(f, w, kernel_map=kernel_map, **common)
    cloned = kernel_map.with_tables(source_masks.clone(), target_masks.clone().contiguous())
    b = F.sparse_convolution_forward(f, w, kernel_map=cloned, **common)
    bare = F.sparse_convolution_forward(f, w, source_masks.clone(), target_masks.clone(), order, sizes, 0, 0,
                                        allow_shortcut_matmul=True, threshold=-1, dataflow="gather_gemm_scatter")
    positional = F.sparse_convolution_forward(f, w, *kernel_map, 0, 0, allow_shortcut_matmul=True, threshold=-1,
                                              dataflow="gather_gemm_scatter")
    assert seen == [(True, True), (True, True), (False, False), (False, False)]
    assert torch.equal(a, b) and torch.equal(a, bare) and torch.equal(a, positional)
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    assert_features_close(a, orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes), "fp32")
    with pytest.raises(ValueError, match="dense"):
        F.sparse_convolution_forward(f, w, source_masks, target_masks, order, sizes, 0, 0, dataflow="implicit")


@pytest.mark.parametrize("kind", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("kernel,stride,cin,cout,n,extent,batched", [
    (3, 1, 32, 32, 20000, 60, False), (3, 1, 128, 128, 5000, 22, True), (2, 2, 64, 128, 20000, 50, False),
    (5, 1, 16, 16, 3000, 16, False), (3, 1, 256, 256, 3000, 16, False), (3, 1, 24, 40, 2000, 12, True),
    (3, 1, 3, 5, 2000, 12, False), (7, 1, 16, 8, 1500, 10, False),
])
def test_forward_list_driven(kind, kernel, stride, cin, cout, n, extent, batched):
    """Gather-GEMM-Scatter driven by lists (pair lists + target-major row lists,
    no rank table read): the row lists against a plain construction from the
    oracle's dense map, the output against the float64 oracle and, to rounding,
    against the table-driven form; with and without an epilogue."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(8, n, extent, kernel, cin, cout, kind, stride, batched)
    esm, etm, eorder, esizes, em = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    dtype = TORCH[kind]
    built = _C.kernel_map_build(dev(src), dev(tgt), off.astype(np.int64), dev(sbd), dev(tbd), reorder=True,
                                want_masks=True, want_lists=True, want_dense=True)
    row_ptr, out_pos = _C.kernel_map_row_lists(built["kernel_map"], built["sizes_host"], built["order_host"])
    # expected lists: hits by target, then by list row; p numbers them by list row, then by target
    hits_t, hits_j = [], []
    dense = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd, dtype=np.int32)
    by_row = dense[eorder]                                  # [list row, target]
    jj, tt = np.nonzero(by_row >= 0)                        # row-major: by list row, then target = list numbering
    p_of = {}
    for p, (j, t) in enumerate(zip(jj, tt)):
        p_of[(j, t)] = p
    tt2, jj2 = np.nonzero(by_row.T >= 0)                    # by target, then list row = buffer numbering
    expect_pos = np.empty(len(jj), dtype=np.int32)
    for pos, (t, j) in enumerate(zip(tt2, jj2)):
        expect_pos[p_of[(j, t)]] = pos
    counts = (by_row >= 0).sum(axis=0)
    np.testing.assert_array_equal(host(row_ptr), np.concatenate([[0], np.cumsum(counts)]))
    np.testing.assert_array_equal(host(out_pos), expect_pos)
    kernel_map = minuet.nn.KernelMap(built["source_masks"], built["target_masks"], built["order"], built["sizes"],
                                     sizes_host=built["sizes_host"], order_host=built["order_host"],
                                     in_idx=built["in_idx"], out_idx=built["out_idx"], dense=built["kernel_map"])
    f, w = dev(feats).to(dtype), dev(weights).to(dtype)
    tables = F.sparse_convolution_forward(f, w, kernel_map=kernel_map, allow_shortcut_matmul=stride == 1,
                                          threshold=-1, dataflow="gather_gemm_scatter")
    assert kernel_map.row_ptr is None
    lists = F.sparse_convolution_forward(f, w, kernel_map=kernel_map, dataflow="list_driven")
    assert kernel_map.row_ptr is not None                   # built on first use
    assert lists.dtype == dtype and lists.shape == (tgt.shape[0], cout)
    assert_features_close(lists, ref, kind)
    diff = (lists.float() - tables.float()).abs().max().item()
    scale_of = tables.float().abs().max().item()
    assert diff <= max(2e-2 * tables.float().pow(2).mean().sqrt().item() if kind != "fp32" else 0.0,
                       scale_of * 2.0 ** {"fp32": -20, "fp16": -10, "bf16": -7}[kind]), diff
    packed = F.sparse_convolution_forward(f, w, kernel_map=kernel_map, dataflow="list_driven",
                                          packed_weights=F.pack_weights(w))
    assert torch.equal(packed, lists)
    rng = np.random.default_rng(5)
    scale = rng.uniform(0.5, 1.5, size=cout).astype(np.float32)
    shift = rng.uniform(-0.5, 0.5, size=cout).astype(np.float32)
    residual = quantise(rng.normal(size=ref.shape), kind)
    fused = np.maximum(ref * scale.astype(np.float64) + shift.astype(np.float64) + residual, 0.0)
    out = F.sparse_convolution_forward(f, w, kernel_map=kernel_map, dataflow="list_driven",
                                       epilogue=F.Epilogue(dev(scale), dev(shift), dev(residual).to(dtype), "relu"))
    assert_features_close(out, fused, kind)


def test_list_driven_layers_in_a_module_chain():
    """down (stride 2) -> submanifold -> transposed up through the modules with
    the list-driven dataflow chosen: every layer, the transposed one included,
    runs without rank tables and agrees with the float64 oracle."""
    rng = np.random.default_rng(4)
    c, _ = sorted_unique(random_cloud(12000, 40, seed=9, lo=-11))
    feats = rng.normal(size=(c.shape[0], 16))
    down = minuet.nn.SparseConv3d(16, 32, 2, stride=2, dtype=torch.float32, device="cuda")
    sub = minuet.nn.SparseConv3d(32, 32, 3, dtype=torch.float32, device="cuda")
    up = minuet.nn.SparseConv(3, 32, 16, 2, stride=2, transposed=True, dtype=torch.float32, device="cuda")
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    for m in (down, sub, up):
        m.set_kernel_map_cache(cache)
        m.tunable_config["dataflow"] = "list_driven"
    with torch.no_grad():
        a = down(minuet.SparseTensor(dev(feats).float(), dev(c)))
        b = sub(a)
        y = up(b)
    assert all(km.row_ptr is not None for km in cache._kernel_maps_cache.values())
    assert all(km.row_ptr is not None for km in cache._swapped_maps_cache.values())
    r1, c1, _, _ = orc.conv_layer(c, None, feats.astype(np.float32).astype(np.float64),
                                  host(down.kernel.detach().double()), 2, stride=2)
    r2, _, _, _ = orc.conv_layer(c1, None, r1, host(sub.kernel.detach().double()), 3, source_stride=2)
    r3, c3, _, _ = orc.conv_layer(c1, None, r2, host(up.kernel.detach().double()), 2, stride=2,
                                  source_stride=2, transposed_from=(c, None, 1))
    np.testing.assert_array_equal(host(y.C), c3)
    for got, ref in ((a.F, r1), (b.F, r2), (y.F, r3)):
        err = np.abs(host(got.double()) - ref).max()
        assert err <= 1e-5 * np.abs(ref).max(), err


@pytest.mark.parametrize("feature_scale,weight_scale", [(2.0 ** 100, 2.0 ** -30), (2.0 ** -100, 1.0),
                                                        (2.0 ** 20, 2.0 ** 20), (1.0, 1.0)])
@pytest.mark.parametrize("shortcut", [False, True])
def test_bf16_product_rows_keep_their_range(feature_scale, weight_scale, shortcut):
    """bfloat16 layers hand their product rows from the GEMM to Scatter as 16-bit
    words under a power-of-two scale taken from max|x| and the weights' column
    sums: features and weights far outside half precision's own range must give
    the same accuracy as ordinary ones (bound: 2e-2 of the reference's RMS), in
    every form of the three-kernel dataflow."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(11, 5000, 22, 3, 64, 48, "bf16")
    feats = feats * feature_scale
    weights = weights * weight_scale
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    assert np.isfinite(ref).all() and np.abs(ref).max() > 0
    f_dev, w_dev = dev(feats).to(torch.bfloat16), dev(weights).to(torch.bfloat16)
    assert np.array_equal(host(f_dev.double()), feats)       # powers of two: still exact in bf16
    plain = F.sparse_convolution_forward(
        sources=f_dev, weights=w_dev, source_masks=dev(esm), target_masks=dev(etm), kernel_map_order=dev(eorder),
        kernel_map_sizes=dev(esizes), gather_tile_size=0, scatter_tile_size=0, allow_shortcut_matmul=shortcut,
        threshold=-1)
    assert_features_close(plain, ref, "bf16")
    kernel_map = kernel_map_of(esm, etm, eorder, esizes)
    folded = F.sparse_convolution_forward(
        sources=f_dev, weights=w_dev, kernel_map=kernel_map, gather_tile_size=0, scatter_tile_size=0,
        allow_shortcut_matmul=shortcut, threshold=-1, packed_weights=F.pack_weights(w_dev))
    assert torch.equal(folded, plain)
    # the scale is a power of two, so a layer whose inputs are scaled by one gives
    # exactly the scaled output
    unit = F.sparse_convolution_forward(
        sources=dev(feats / feature_scale).to(torch.bfloat16), weights=dev(weights / weight_scale).to(torch.bfloat16),
        kernel_map=kernel_map, gather_tile_size=0, scatter_tile_size=0, allow_shortcut_matmul=shortcut, threshold=-1)
    assert torch.equal((unit.double() * (feature_scale * weight_scale)).to(torch.bfloat16), plain)


def test_bf16_non_finite_features_stay_in_their_rows():
    """An infinite or NaN feature does not take part in the scale of the product
    rows: targets that do not read it keep their accuracy, targets that do are
    not finite (as with any buffer)."""
    src, sbd, tgt, tbd, off, feats, weights = make_layer_case(12, 4000, 22, 3, 32, 32, "bf16")
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=True)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    bad = feats.copy()
    bad[17, 3] = np.inf
    bad[2900, 5] = np.nan
    touched = np.zeros(tgt.shape[0], dtype=bool)
    for j in range(esm.shape[0]):
        for row in (17, 2900):
            rank = esm[j, row]
            if rank >= 0:
                touched[np.nonzero(etm[j] == rank)[0]] = True
    assert touched.sum() >= 2 and not touched.all()
    out = F.sparse_convolution_forward(
        sources=dev(bad).to(torch.bfloat16), weights=dev(weights).to(torch.bfloat16), source_masks=dev(esm),
        target_masks=dev(etm), kernel_map_order=dev(eorder), kernel_map_sizes=dev(esizes), gather_tile_size=0,
        scatter_tile_size=0, allow_shortcut_matmul=True, threshold=-1)
    got = host(out.float())
    assert not np.isfinite(got[touched]).all(axis=1).any()
    assert np.isfinite(got[~touched]).all()
    err = np.abs(got[~touched].astype(np.float64) - ref[~touched]).max()
    assert err <= 2e-2 * np.sqrt(np.mean(ref ** 2))


def _surface_cloud(seed, n, extent):
    """Voxels near a few planes and one box: dense along some axes, thin along
    others, like the levels of a LiDAR scan."""
    rng = np.random.default_rng(seed)
    parts = []
    for axis in (2, 2, 0):
        pts = rng.integers(0, extent, size=(n // 3, 3))
        pts[:, axis] = rng.integers(0, extent) + rng.integers(0, 2, size=n // 3)
        parts.append(pts)
    parts.append(rng.integers(0, extent // 6, size=(n // 6, 3)) + extent // 3)
    return np.concatenate(parts).astype(np.int32)


@pytest.mark.parametrize("dilation", [1, 2])
@pytest.mark.parametrize("layout", ["minuet", "torchsparse"])
def test_offset_group_tables_match_brute_force(dilation, layout):
    """mnt_kernel_map_offset_groups against plain NumPy on the dense map: the
    axis with the fewest rows (lowest on a tie), the rows per group, every
    target's rank inside its groups and every row's three source rows."""
    from minuet_amd.utils.helpers import generate_kernel_offsets
    for seed, n, extent in ((1, 9000, 60), (2, 700, 12), (3, 30000, 90)):
        src, _ = sorted_unique(_surface_cloud(seed, n, extent), None)
        off = np.ascontiguousarray(generate_kernel_offsets(3, 3, 1, dilation, layout=layout), dtype=np.int64)
        dense, _ = _C.kernel_map_dense(dev(src), dev(src), off, None, None)
        groups = _C.kernel_map_offset_groups(dense, off)
        assert groups is not None
        table = _C.offset_group_table(off)
        for axis in range(3):
            assert sorted(table[axis].reshape(-1).tolist()) == list(range(27))
            for j in range(9):
                members = off[table[axis, j]]
                others = [a for a in range(3) if a != axis]
                assert (members[:, others] == members[0, others]).all()
                assert (np.diff(members[:, axis]) > 0).all()
        m = host(dense)
        T = m.shape[1]
        reach = np.stack([[(m[table[a, j]] >= 0).any(0) for j in range(9)] for a in range(3)])   # [3, 9, T]
        totals = reach.sum((1, 2))
        axis = int(np.argmin(totals))
        head = host(groups.head)
        assert head[0] == axis
        np.testing.assert_array_equal(head[1:10], reach[axis].sum(1))
        rank, rows = host(groups.rank), host(groups.src)
        for j in range(9):
            hit = reach[axis, j]
            np.testing.assert_array_equal(rank[j], np.where(hit, np.cumsum(hit) - 1, -1))
            expect = m[table[axis, j]][:, hit].T                                # [rows, 3]
            np.testing.assert_array_equal(rows[j * T:j * T + expect.shape[0], :3], expect)


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("cin,cout,n,extent", [(128, 128, 9000, 60), (256, 256, 3000, 30), (64, 64, 5000, 40),
                                               (128, 256, 4000, 40), (192, 72, 2500, 30), (256, 128, 700, 12)])
def test_forward_offset_groups(kind, cin, cout, n, extent):
    """The forward pass over offset groups against the float64 oracle, with and
    without an epilogue, and against the three-kernel dataflow."""
    rng = np.random.default_rng(5)
    src, _ = sorted_unique(_surface_cloud(7, n, extent), None)
    off = orc.generate_kernel_offsets(3, 3, 1, 1)
    feats = quantise(rng.normal(size=(src.shape[0], cin)), kind)
    weights = quantise(rng.normal(size=(27, cin, cout)) / np.sqrt(27 * cin), kind)
    esm, etm, eorder, esizes, _ = orc.build_kernel_map(src, None, src, None, off, reorder=True)
    ref = orc.sparse_convolution_forward(feats, weights, esm, etm, eorder, esizes)
    dtype = TORCH[kind]
    f_dev, w_dev = dev(feats).to(dtype), dev(weights).to(dtype)
    dense, _ = _C.kernel_map_dense(dev(src), dev(src), off.astype(np.int64), None, None)
    groups = _C.kernel_map_offset_groups(dense, off.astype(np.int64))
    out = _C.sparse_convolution_forward_groups(f_dev, w_dev, groups)
    assert out.dtype == dtype and out.shape == ref.shape
    assert_features_close(out, ref, kind)
    again = _C.sparse_convolution_forward_groups(f_dev, w_dev, groups, packed_weights=F.pack_weights(w_dev))
    assert torch.equal(again, out)                                   # no atomics: reruns are bit-equal
    scale = rng.uniform(0.5, 1.5, size=cout).astype(np.float32)
    shift = rng.uniform(-0.5, 0.5, size=cout).astype(np.float32)
    residual = quantise(rng.normal(size=ref.shape), kind)
    fused_ref = np.maximum(ref * scale.astype(np.float64) + shift.astype(np.float64) + residual, 0.0)
    fused = _C.sparse_convolution_forward_groups(
        f_dev, w_dev, groups, epilogue=F.Epilogue(dev(scale), dev(shift), dev(residual).to(dtype), "relu"))
    got = host(fused.float()).astype(np.float64)
    # the bound is taken from the sums before the ReLU, whose rounding it covers
    pre = ref * scale.astype(np.float64) + shift.astype(np.float64) + residual
    assert np.abs(got - fused_ref).max() <= 2e-2 * np.sqrt(np.mean(pre ** 2))


@pytest.mark.parametrize("kind", ["fp16", "bf16"])
@pytest.mark.parametrize("stride,n,extent", [(1, 8000, 50), (2, 6000, 40), (1, 40, 6), (1, 1, 6)])
def test_module_takes_offset_groups_for_wide_layers(kind, stride, n, extent):
    """A 128 -> 128 3x3x3 layer under ``dataflow="auto"`` runs over offset groups
    (the cache then builds the dense map and the group tables only) and agrees
    with the same layer forced through Gather-GEMM-Scatter; also strided (fewer
    targets than sources) and on clouds smaller than a tile."""
    dtype = TORCH[kind]
    src, _ = sorted_unique(_surface_cloud(9, max(n, 6), extent)[:n], None)
    conv = minuet.nn.SparseConv3d(128, 128, 3, stride=stride, dtype=dtype, device="cuda")
    x = minuet.SparseTensor(torch.randn(src.shape[0], 128, device="cuda").to(dtype), dev(src))
    with torch.no_grad():
        cache = minuet.nn.KernelMapCache(3, torch.int32, "cuda")
        conv.set_kernel_map_cache(cache)
        auto = conv(x).F
        assert len(cache._offset_groups_cache) == 1 and not cache._kernel_maps_cache
        conv.tunable_config["dataflow"] = "gather_gemm_scatter"
        conv._routes.clear()
        three = conv(x).F
        assert len(cache._kernel_maps_cache) == 1
    # two roundings of the same sums: 2e-2 of the RMS, or one unit in the last
    # place of the largest value where that is more (bf16 keeps 8 bits)
    diff = (auto.float() - three.float()).abs().max().item()
    ulp = three.float().abs().max().item() * 2.0 ** (-7 if kind == "bf16" else -10)
    assert diff <= max(2e-2 * three.float().pow(2).mean().sqrt().item(), ulp), diff
