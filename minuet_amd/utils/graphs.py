"""Replaying a forward pass whose kernel maps are cached as one HIP graph.

Once a network has seen a cloud, every layer's kernel map sits in the
``KernelMapCache`` and a forward pass is a fixed sequence of kernel launches
with no wait on the device: the library's scratch memory comes from a
per-stream arena that is reused, the host-side tables travel in kernel
arguments, and nothing is read back.  Such a pass can be captured in a HIP
graph and replayed with new feature values, which removes the per-layer
launch cost on the host.  (Not in the reference, whose layers synchronise to
read the kernel-map sizes back on every call:
minuet/nn/functional/convolution.py:32-60.)"""
from typing import Callable

import torch

__all__ = ["GraphedForward", "capture_forward"]


class GraphedForward:
    """A captured forward pass.  ``replay()`` runs it again on the tensors it was
    captured with: write new values into the input features in place (the
    coordinates must not change), replay, and read ``output``."""

    def __init__(self, graph: "torch.cuda.CUDAGraph", output, stream: "torch.cuda.Stream"):
        from minuet_amd.nn.functional import _C
        self.graph = graph
        self.output = output
        self.stream = stream
        self._reset_count = _C.device_reset_count()

    def replay(self):
        """Raises after ``cuda_device_reset()``: the reset gave back the scratch
        memory whose addresses the captured kernels hold."""
        from minuet_amd.nn.functional import _C
        if _C.device_reset_count() != self._reset_count:
            raise RuntimeError("[Minuet] this captured pass is no longer valid: cuda_device_reset() freed the "
                               "scratch memory its kernels point into; capture the pass again")
        self.graph.replay()
        return self.output


def capture_forward(forward: Callable[[], object], warmup: int = 3) -> GraphedForward:
    """Captures ``forward()`` (a callable without arguments that runs the network
    on fixed input tensors and returns its output) in a HIP graph.

    The warm-up runs happen on the capture stream first, so that the kernel maps
    are cached, weights are packed and the stream's scratch arena has its final
    size before anything is recorded; a pass that still has to build a kernel
    map waits on the device and cannot be captured.

    The capture stream is a fresh one that only the returned object knows: the
    graph's kernels use scratch pointers of that stream's arena, which
    therefore must not be freed (``cuda_free_buffers`` acts on the arena of
    the stream that is current, never this one) nor used by other work.  Replays
    of one ``GraphedForward`` must not overlap (they share that scratch).
    ``cuda_device_reset()`` does free that arena: a ``GraphedForward`` captured
    before it refuses to replay afterwards.

    A look-ahead session of a ``KernelMapCache(lookahead=True)`` that is still
    running is ended before the capture starts: its worker thread allocates and
    launches on its own, which would invalidate a capture under way on this
    thread."""
    if not torch.cuda.is_available():
        raise RuntimeError("[Minuet] graph capture needs a GPU")
    from minuet_amd.nn.lookahead import end_running_session
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.no_grad(), torch.cuda.stream(side):
        for _ in range(max(1, warmup)):
            forward()
    torch.cuda.current_stream().wait_stream(side)
    end_running_session(torch.device("cuda", torch.cuda.current_device()))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(graph, stream=side):
        output = forward()
    return GraphedForward(graph, output, side)
