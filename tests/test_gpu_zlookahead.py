"""Look-ahead building of a pass's coordinate levels and kernel maps
(KernelMapCache(lookahead=True)): same results as the ordinary cache, pass
after pass, also when the network or the cloud changes between passes."""
import os

import numpy as np
import pytest
import torch

import minuet_amd as minuet
from helpers import dev
from minuet_amd.nn.functional import _C
from minuet_amd.synthetic import make_cloud
from minuet_amd.unet import SparseUNet

pytestmark = pytest.mark.gpu

# With the switch set for the whole process, caches of tests that ran before may
# still hold the one session: results must be the same then, the counts of
# builds taken from the worker are not checked.
FORCED_FOR_ALL = os.environ.get("MINUET_LOOKAHEAD", "") == "1"


@pytest.fixture(autouse=True)
def _switch_from_the_argument_only(monkeypatch):
    """The environment switch would turn the look-ahead on for the ordinary
    caches these tests compare with (one session runs at a time per process)."""
    monkeypatch.delenv("MINUET_LOOKAHEAD", raising=False)


def _cloud(scale, seed_shift):
    cloud = make_cloud(4, scale)
    coords, bd = cloud["coords"].copy(), cloud["batch_dims"]
    coords[:, 0] += seed_shift                       # another cloud of the same shape family
    idx, sorted_dev = _C.sort_coordinates(dev(coords), dev(bd))
    return sorted_dev, dev(bd)


def _run(net, cache, coords, bd, feats):
    cache.reset()
    with torch.no_grad():
        y = net(minuet.SparseTensor(feats, coords, batch_dims=bd))
    return y


def test_unet_passes_match_the_ordinary_cache():
    torch.manual_seed(0)
    net = SparseUNet(4, 16, dtype=torch.float16, device="cuda").eval()
    plain = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    ahead = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda", lookahead=True)
    hits = []
    for step, (scale, shift) in enumerate([(0.05, 0), (0.05, 3), (0.08, -5), (0.02, 11), (0.05, 3)]):
        coords, bd = _cloud(scale, shift)
        feats = torch.randn(coords.shape[0], 4, device="cuda").half()
        minuet.set_kernel_map_cache(net, plain)
        want = _run(net, plain, coords, bd, feats)
        builds = (plain.num_coordinate_builds, plain.num_map_builds)
        minuet.set_kernel_map_cache(net, ahead)
        before = ahead.num_ahead_hits
        got = _run(net, ahead, coords, bd, feats)
        torch.cuda.synchronize()
        assert torch.equal(got.C, want.C) and torch.equal(got.F, want.F), f"pass {step}"
        assert (ahead.num_coordinate_builds, ahead.num_map_builds) == builds
        hits.append(ahead.num_ahead_hits - before)
    ahead.reset()
    # the first pass has no recipe; every later one takes all of its builds from the worker
    assert FORCED_FOR_ALL or (hits[0] == 0 and all(h >= 13 for h in hits[1:])), hits


def test_config4_full_size_cold_passes_bit_equal_to_the_plain_cache():
    """The UNet of configuration 4 at its full size (2 x 100 000 voxels, widths
    32 ... 256): cold passes with the look-ahead against cold passes of the
    ordinary cache, bit for bit, coordinates and features."""
    torch.manual_seed(4)
    net = SparseUNet(4, 32, dtype=torch.float16, device="cuda").eval()
    plain = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    ahead = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda", lookahead=True)
    coords, bd = _cloud(1.0, 0)
    feats = torch.randn(coords.shape[0], 4, device="cuda").half()
    minuet.set_kernel_map_cache(net, plain)
    want = _run(net, plain, coords, bd, feats)
    minuet.set_kernel_map_cache(net, ahead)
    hits = []
    for step in range(3):
        before = ahead.num_ahead_hits
        got = _run(net, ahead, coords, bd, feats)
        torch.cuda.synchronize()
        assert torch.equal(got.C, want.C) and torch.equal(got.F, want.F), f"pass {step}"
        hits.append(ahead.num_ahead_hits - before)
    ahead.reset()
    assert FORCED_FOR_ALL or (hits[0] == 0 and all(h >= 13 for h in hits[1:])), hits


def test_changed_requests_fall_back_to_ordinary_builds():
    """A pass that asks for other maps than the recipe holds builds them itself;
    what the worker built for nobody is dropped at reset()."""
    torch.manual_seed(1)
    coords, bd = _cloud(0.03, 0)
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda", lookahead=True)
    plain = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    first = minuet.nn.SparseConv3d(8, 8, 3, dtype=torch.float16, device="cuda")
    down = minuet.nn.SparseConv3d(8, 8, 2, stride=2, dtype=torch.float16, device="cuda")
    other = minuet.nn.SparseConv3d(8, 8, 5, dtype=torch.float16, device="cuda")
    feats = torch.randn(coords.shape[0], 8, device="cuda").half()

    def net_a(c):
        for m in (first, down):
            m.set_kernel_map_cache(c)
        return down(first(minuet.SparseTensor(feats, coords, batch_dims=bd)))

    def net_b(c):
        for m in (other, down):
            m.set_kernel_map_cache(c)
        return down(other(minuet.SparseTensor(feats, coords, batch_dims=bd)))

    with torch.no_grad():
        for net in (net_a, net_a, net_b, net_b, net_a):
            cache.reset()
            plain.reset()
            got, want = net(cache), net(plain)
            assert torch.equal(got.C, want.C) and torch.equal(got.F, want.F)
    cache.reset()


def test_session_errors_are_reported_and_leave_the_library_usable():
    coords, bd = _cloud(0.02, 0)
    from minuet_amd.nn.lookahead import end_running_session
    end_running_session(coords.device)                   # whatever a cache of an earlier test still held
    with pytest.raises(RuntimeError, match=r"\[Minuet\]"):
        _C.lookahead_wait(0, coords.device)              # no session
    _C.cuda_reset_error()
    _C.lookahead_finish(coords.device)                   # a no-op without a session
    from minuet_amd.nn.lookahead import AheadSession
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        AheadSession([("tables", ((1, 1, 1), (1, 1, 1), (3, 3, 3), (1, 1, 1)), True)], cache._kernel_offsets,
                     coords, (1, 1, 1), bd)
    key = ((1, 1, 1), (1, 1, 1), (3, 3, 3), (1, 1, 1))
    session = AheadSession([("dense", key), ("invert", key)], cache._kernel_offsets, coords, (1, 1, 1), bd)
    with pytest.raises(RuntimeError, match="running"):
        AheadSession([("dense", key)], cache._kernel_offsets, coords, (1, 1, 1), bd)
    _C.cuda_reset_error()
    dense = session.take(("dense", key))
    inverse = session.take(("invert", key))
    session.finish()
    want, _ = _C.kernel_map_dense(coords, coords, cache._kernel_offsets((1, 1, 1), (3, 3, 3), (1, 1, 1)), bd, bd)
    torch.cuda.synchronize()
    assert torch.equal(dense, want)
    assert torch.equal(inverse, _C.kernel_map_invert(want, coords.shape[0]))


@pytest.mark.parametrize("coord_dtype,batched,wide", [(torch.int64, False, False), (torch.int32, False, True),
                                                       (torch.int64, True, True)])
def test_down_sub_up_chain_through_every_item_kind(coord_dtype, batched, wide):
    """Coordinates, dense maps, rank tables and inverse maps from the worker for
    int64 coordinates, single clouds and layers that run as Gather-GEMM-Scatter
    (fp32 features with 27 offsets do)."""
    torch.manual_seed(2)
    dtype = torch.float32 if wide else torch.float16
    width = 16
    first = minuet.nn.SparseConv3d(8, width, 3, dtype=dtype, device="cuda")
    down = minuet.nn.SparseConv3d(width, width, 2, stride=2, dtype=dtype, device="cuda")
    sub = minuet.nn.SparseConv3d(width, width, 3, dtype=dtype, device="cuda")
    up = minuet.nn.SparseConv(3, width, 8, 2, stride=2, transposed=True, dtype=dtype, device="cuda")
    layers = (first, down, sub, up)

    def forward(cache, coords, bd, feats):
        cache.reset()
        for layer in layers:
            layer.set_kernel_map_cache(cache)
        x = minuet.SparseTensor(feats, coords, batch_dims=bd)
        with torch.no_grad():
            for layer in layers:
                x = layer(x)
        return x

    plain = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    ahead = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda", lookahead=True)
    for step, (scale, shift) in enumerate([(0.03, 0), (0.04, 7), (0.02, -3)]):
        coords, bd = _cloud(scale, shift)
        if not batched:
            coords, bd = _C.sort_coordinates(coords)[1], None
        coords = coords.to(coord_dtype)
        feats = torch.randn(coords.shape[0], 8, device="cuda").to(dtype)
        want = forward(plain, coords, bd, feats)
        before = ahead.num_ahead_hits
        got = forward(ahead, coords, bd, feats)
        torch.cuda.synchronize()
        assert torch.equal(got.C, want.C) and torch.equal(got.F, want.F), f"pass {step}"
        if step > 0:
            assert FORCED_FOR_ALL or ahead.num_ahead_hits - before >= 4
    ahead.reset()
