"""A forward pass with cached kernel maps captured in a HIP graph: every replay
must give exactly what the eager pass gives on the same feature values, also
with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

import minuet_amd as minuet
from minuet_amd.nn.functional import _C
from minuet_amd.synthetic import make_cloud
from minuet_amd.unet import SparseUNet

pytestmark = pytest.mark.gpu


def _unet_and_input(dtype):
    device = torch.device("cuda:0")
    cloud = make_cloud(4, scale=0.05)
    coords = torch.from_numpy(cloud["coords"]).to(device)
    batch_dims = torch.from_numpy(cloud["batch_dims"]).to(device)
    _, ordered = _C.sort_coordinates(coords, batch_dims)
    torch.manual_seed(11)
    net = SparseUNet(4, 16, dtype=dtype, device=device).eval()
    minuet.set_kernel_map_cache(net, minuet.nn.KernelMapCache(3, torch.int32, device))
    features = torch.randn(ordered.shape[0], 4, device=device).to(dtype)
    return net, minuet.SparseTensor(features, ordered, batch_dims=batch_dims), features


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_graph_replays_equal_eager_passes(dtype):
    net, x, features = _unet_and_input(dtype)
    graphed = minuet.capture_forward(lambda: net(x))
    with torch.no_grad():
        for replay in range(4):
            features.copy_(torch.randn_like(features) * (1.0 + replay))     # new values, same cloud
            expected = net(x).F.clone()                                     # eager work in between
            torch.cuda.synchronize()
            out = graphed.replay()
            torch.cuda.synchronize()
            assert out.F.shape == expected.shape
            assert torch.equal(out.F, expected), f"replay {replay} differs from the eager pass"
        # two replays back to back without the host looking in between
        features.copy_(torch.randn_like(features))
        graphed.replay()
        second = graphed.replay().F.clone()
        torch.cuda.synchronize()
        assert torch.equal(second, net(x).F)


def test_capture_after_cache_reset_warms_up_first():
    # the warm-up passes inside capture_forward fill the cache; the captured
    # pass itself must not have to build anything
    net, x, _ = _unet_and_input(torch.float16)
    cache = next(m for m in net.modules() if isinstance(m, minuet.nn.SparseConv))._kernel_map_cache
    cache.reset()
    graphed = minuet.capture_forward(lambda: net(x), warmup=1)
    with torch.no_grad():
        assert torch.equal(graphed.replay().F, net(x).F)


def test_replay_is_refused_after_a_device_reset():
    """cuda_device_reset() frees the capture stream's scratch arena, whose
    addresses the captured kernels hold: the captured pass must not run again."""
    net, x, _ = _unet_and_input(torch.float16)
    graphed = minuet.capture_forward(lambda: net(x), warmup=1)
    with torch.no_grad():
        assert torch.equal(graphed.replay().F, net(x).F)
    torch.cuda.synchronize()
    _C.cuda_device_reset()
    with pytest.raises(RuntimeError, match="no longer valid"):
        graphed.replay()
    # the library itself goes on working, and a new capture is fine
    again = minuet.capture_forward(lambda: net(x), warmup=1)
    with torch.no_grad():
        assert torch.equal(again.replay().F, net(x).F)
