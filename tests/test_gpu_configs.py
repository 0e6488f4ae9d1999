"""Full-size BASELINE configurations: oracle parity where the CPU oracle is
fast enough (plain-C oracle), size-independent properties elsewhere."""
import numpy as np
import pytest
import torch

import c_oracle
import minuet_oracle as orc
import minuet_amd as minuet
from helpers import dev, host
from minuet_amd.nn.functional import _C
from minuet_amd.synthetic import make_cloud

pytestmark = pytest.mark.gpu


def sort_on_gpu(coords):
    index, sorted_dev, bounds = _C.sort_coordinates(dev(coords), return_bounds=True)
    return index, sorted_dev, bounds


def test_config2_map_step_full_size_bit_exact():
    coords = make_cloud(2)["coords"]
    offsets = orc.generate_kernel_offsets(3, 3)
    index, sorted_dev, bounds = sort_on_gpu(coords)
    ref_index, ref_sorted = c_oracle.arg_sort(coords)
    np.testing.assert_array_equal(host(index).astype(np.int64), ref_index)
    np.testing.assert_array_equal(host(sorted_dev), ref_sorted)
    np.testing.assert_array_equal(bounds[:3], coords.min(0))
    np.testing.assert_array_equal(bounds[4:7], coords.max(0))
    built = _C.kernel_map_build(sorted_dev, sorted_dev, offsets, None, None, reorder=True,
                                want_masks=True, want_lists=True, want_dense=True,
                                source_bounds=bounds, target_bounds=bounds)
    ref_map = c_oracle.query(ref_sorted, ref_sorted, offsets.astype(np.int32))
    np.testing.assert_array_equal(host(built["kernel_map"]), ref_map)
    sizes = c_oracle.sizes(ref_map)
    order = orc.stable_size_order(sizes)
    np.testing.assert_array_equal(built["order_host"], order)
    np.testing.assert_array_equal(built["sizes_host"], sizes[order])
    sm, tm = c_oracle.masks(ref_map, coords.shape[0], order)
    np.testing.assert_array_equal(host(built["source_masks"]), sm)
    np.testing.assert_array_equal(host(built["target_masks"]), tm)
    ein, eout = c_oracle.pair_lists(np.ascontiguousarray(ref_map[order]))
    np.testing.assert_array_equal(host(built["in_idx"]), ein)
    np.testing.assert_array_equal(host(built["out_idx"]), eout)


@pytest.mark.parametrize("reorder", [True, False])
def test_config2_map_step_one_call_full_size_bit_exact(reorder):
    """The entry point bench.py times (mnt_sorted_kernel_map_lists: unsorted
    voxels -> sorted voxels -> per-offset pair lists in one call) at the full
    200 000 voxels of configuration 2, rows in size order and in offset order
    (reference flow: minuet/nn/convolutions.py:147-170)."""
    coords = make_cloud(2)["coords"]
    offsets = orc.generate_kernel_offsets(3, 3)
    built = _C.sorted_kernel_map_lists(dev(coords), offsets, reorder=reorder, result_only=True)
    ref_index, ref_sorted = c_oracle.arg_sort(coords)
    np.testing.assert_array_equal(host(built["indices"]).astype(np.int64), ref_index)
    np.testing.assert_array_equal(host(built["coordinates"]), ref_sorted)
    np.testing.assert_array_equal(built["bounds"][:3], coords.min(0))
    np.testing.assert_array_equal(built["bounds"][4:7], coords.max(0))
    ref_map = c_oracle.query(ref_sorted, ref_sorted, offsets.astype(np.int32))
    sizes = c_oracle.sizes(ref_map)
    order = orc.stable_size_order(sizes) if reorder else np.arange(offsets.shape[0])
    np.testing.assert_array_equal(built["order_host"], order)
    np.testing.assert_array_equal(built["sizes_host"], sizes[order])
    np.testing.assert_array_equal(host(built["order"]), order)
    np.testing.assert_array_equal(host(built["sizes"]), sizes[order])
    ein, eout = c_oracle.pair_lists(np.ascontiguousarray(ref_map[order]))
    np.testing.assert_array_equal(host(built["in_idx"]), ein)
    np.testing.assert_array_equal(host(built["out_idx"]), eout)
    # what the timed loop does: the same call again and again on the same stream
    again = _C.sorted_kernel_map_lists(dev(coords), offsets, reorder=reorder, result_only=True)
    assert torch.equal(again["in_idx"], built["in_idx"]) and torch.equal(again["out_idx"], built["out_idx"])


def test_config1_layer_fp32_full_size():
    coords = make_cloud(1)["coords"]
    rng = np.random.default_rng(1001)
    _, sorted_dev, _ = sort_on_gpu(coords)
    ref_sorted = host(sorted_dev)
    feats = rng.normal(size=(coords.shape[0], 32)).astype(np.float32)
    weights = (rng.normal(size=(27, 32, 32)) / np.sqrt(27 * 32)).astype(np.float32)
    conv = minuet.nn.SparseConv3d(32, 32, 3, dtype=torch.float32, device="cuda")
    conv.kernel.data.copy_(dev(weights))
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    conv.set_kernel_map_cache(cache)
    with torch.no_grad():
        y = conv(minuet.SparseTensor(dev(feats), sorted_dev))
    ref, _, _, _ = orc.conv_layer(ref_sorted, None, feats.astype(np.float64), weights.astype(np.float64), 3)
    err = np.abs(host(y.F.double()) - ref).max()
    assert err <= 1e-5 * np.abs(ref).max(), err


def test_config3_down_up_fp16_full_size():
    coords = make_cloud(3)["coords"]
    rng = np.random.default_rng(1003)
    _, sorted_dev, _ = sort_on_gpu(coords)
    ref_sorted = host(sorted_dev)
    feats = torch.from_numpy(rng.normal(size=(coords.shape[0], 64))).half()
    down = minuet.nn.SparseConv3d(64, 128, 2, stride=2, dtype=torch.float16, device="cuda")
    up = minuet.nn.SparseConv(3, 128, 64, 2, stride=2, transposed=True, dtype=torch.float16, device="cuda")
    for conv, cin in ((down, 64), (up, 128)):
        conv.kernel.data.normal_(0.0, float(np.sqrt(2.0 / (8 * cin))))
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    minuet.set_kernel_map_cache(torch.nn.Sequential(down, up), cache)
    with torch.no_grad():
        mid = down(minuet.SparseTensor(feats.cuda(), sorted_dev))
        out = up(mid)
    r1, c1, _, _ = orc.conv_layer(ref_sorted, None, feats.double().numpy(),
                                  host(down.kernel.detach().double()), 2, stride=2)
    np.testing.assert_array_equal(host(mid.C), c1)
    e1 = np.abs(host(mid.F.double()) - r1).max()
    assert e1 <= 2e-2 * np.sqrt(np.mean(r1 ** 2)), e1
    r2, c2, _, _ = orc.conv_layer(c1, None, host(mid.F.double()), host(up.kernel.detach().double()), 2,
                                  stride=2, source_stride=2, transposed_from=(ref_sorted, None, 1))
    np.testing.assert_array_equal(host(out.C), ref_sorted)
    e2 = np.abs(host(out.F.double()) - r2).max()
    assert e2 <= 2e-2 * np.sqrt(np.mean(r2 ** 2)), e2


def test_config5_large_kernel_bf16_properties():
    """5x5x5, 125 offsets, bf16, ~1M voxels: kernel-map invariants and linearity at
    full size, oracle parity on a 5 % sample of the same generator."""
    torch.manual_seed(5)
    for scale, check_oracle in ((0.05, True), (1.0, False)):
        coords = make_cloud(5, scale)["coords"]
        assert coords.min() >= 0 and coords[:, :2].max() < 2048
        offsets = orc.generate_kernel_offsets(3, 5)
        _, sorted_dev, bounds = sort_on_gpu(coords)
        built = _C.kernel_map_build(sorted_dev, sorted_dev, offsets, None, None, reorder=True,
                                    want_masks=True, want_lists=True, source_bounds=bounds,
                                    target_bounds=bounds)
        n = coords.shape[0]
        sizes, order = built["sizes_host"], built["order_host"]
        assert sizes[-1] == n and order[-1] == 62                 # centre offset is the identity
        assert (np.diff(sizes) >= 0).all()
        by_offset = np.empty(125, dtype=np.int64)
        by_offset[order] = sizes
        assert (by_offset == by_offset[::-1]).all()               # |hits(d)| == |hits(-d)|
        in_idx, out_idx = built["in_idx"], built["out_idx"]
        start = int(sizes[:-1].sum())
        assert torch.equal(in_idx[start:], out_idx[start:])       # identity rows of the centre offset
        # every listed pair satisfies source = target + offset
        cum = np.concatenate([[0], np.cumsum(sizes)])
        rows = np.repeat(order, sizes)
        delta = sorted_dev[in_idx.long()] - sorted_dev[out_idx.long()]
        assert torch.equal(delta.cpu(), torch.from_numpy(offsets[rows]).to(delta.dtype))
        # hits are ranked by target inside every offset
        for j in (0, 60, 124):
            seg = out_idx[cum[j]:cum[j + 1]].cpu().numpy()
            assert (np.diff(seg) > 0).all()
        conv = minuet.nn.SparseConv3d(64, 64, 5, dtype=torch.bfloat16, device="cuda")
        cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
        conv.set_kernel_map_cache(cache)
        feats = torch.randn(n, 64, device="cuda").bfloat16()
        outputs = {}
        # every dataflow: the single-kernel form ("auto" takes it here), the
        # reference's Gather -> grouped GEMM -> Scatter over the 125 skewed groups,
        # and its list-driven variant
        for flow in ("auto", "gather_gemm_scatter", "list_driven"):
            conv.tunable_config["dataflow"] = flow
            with torch.no_grad():
                y = conv(minuet.SparseTensor(feats, sorted_dev))
                y2 = conv(minuet.SparseTensor(feats * 2, sorted_dev))
                again = conv(minuet.SparseTensor(feats, sorted_dev))
            rms = y.F.float().pow(2).mean().sqrt().item()
            assert torch.isfinite(y.F).all()
            assert torch.equal(again.F, y.F)                        # no atomics: bit-equal reruns
            assert (y2.F.float() - 2 * y.F.float()).abs().max().item() <= 2e-2 * rms
            if check_oracle:
                ref, _, _, _ = orc.conv_layer(host(sorted_dev), None, host(feats.double()),
                                              host(conv.kernel.detach().double()), 5)
                err = np.abs(host(y.F.double()) - ref).max()
                assert err <= 2e-2 * np.sqrt(np.mean(ref ** 2)), (flow, err)
            outputs[flow] = y.F.float()
        # the two dataflows round the same fp32 sums once each: 2e-2 of the RMS, or
        # one bf16 unit in the last place of the largest value where that is more
        rms = outputs["auto"].pow(2).mean().sqrt().item()
        for flow in ("gather_gemm_scatter", "list_driven"):
            diff = (outputs["auto"] - outputs[flow]).abs().max().item()
            assert diff <= max(2e-2 * rms, outputs["auto"].abs().max().item() * 2.0 ** -7), (flow, diff)
