"""ResNet-style sparse classifier, the second network family of the
reference's end-to-end benchmarks (its README names ResNet and UNet; the model
definitions live outside the reference tree, README.md:6): a 3x3x3 stem,
stride-2 stages of two residual blocks each, global average pooling over every
point cloud and a linear head.  Assembled from the public modules of this
package; in evaluation mode the BatchNorm / ReLU / residual-sum layers ride the
convolutions' output pass."""
import torch
from torch import nn

from minuet_amd.nn import BatchNorm, GlobalAvgPool, ReLU, SparseConv3d
from minuet_amd.nn.fused import FusedSequential
from minuet_amd.tensors import SparseTensor
from minuet_amd.unet import ResidualBlock

__all__ = ["SparseResNet"]


class SparseResNet(nn.Module):
    """``in_channels`` features per voxel -> ``num_classes`` logits per point cloud."""

    def __init__(self, in_channels: int = 4, num_classes: int = 10, stem: int = 32,
                 stages=(64, 128, 256), dtype=None, device=None):
        super().__init__()
        factory = {"dtype": dtype, "device": device}
        self.stem = FusedSequential(SparseConv3d(in_channels, stem, 3, **factory),
                                    BatchNorm(stem, **factory), ReLU(inplace=True))
        self.down = nn.ModuleList()
        self.stages = nn.ModuleList()
        width = stem
        for out in stages:
            self.down.append(FusedSequential(SparseConv3d(width, out, 2, stride=2, **factory),
                                             BatchNorm(out, **factory), ReLU(inplace=True)))
            self.stages.append(nn.Sequential(ResidualBlock(out, out, **factory),
                                             ResidualBlock(out, out, **factory)))
            width = out
        self.pool = GlobalAvgPool()
        self.head = nn.Linear(width, num_classes, **factory)

    def forward(self, x: SparseTensor) -> torch.Tensor:
        x = self.stem(x)
        for down, stage in zip(self.down, self.stages):
            x = stage(down(x))
        pooled = self.pool(x)
        if pooled.dim() == 1:                      # a single cloud without batch_dims
            pooled = pooled.unsqueeze(0)
        return self.head(pooled)
