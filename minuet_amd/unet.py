"""Sparse UNet used by the end-to-end benchmark configuration: four stride-2
encoder stages (32/64/128/256 channels), four transposed-convolution decoder
stages with skip concatenation, two residual 3x3x3 submanifold blocks per
stage.  Everything is assembled from the public modules of this package, the
way a user of the reference would write it; in evaluation mode the
BatchNorm / ReLU / residual-sum layers ride the convolutions' output pass."""
import torch
from torch import nn

from minuet_amd.nn import BatchNorm, ReLU, SparseConv, SparseConv3d
from minuet_amd.nn.fused import FusedSequential, conv_norm_act
from minuet_amd.nn import functional as F
from minuet_amd.tensors import SparseTensor

__all__ = ["ResidualBlock", "SparseUNet"]


def _with_features(x: SparseTensor, features: torch.Tensor) -> SparseTensor:
    return SparseTensor.like(x, features)


class ResidualBlock(nn.Module):
    """conv3-BN-ReLU-conv3-BN plus the input (through a 1x1x1 projection when the
    widths differ), then ReLU."""

    def __init__(self, in_channels: int, out_channels: int, **factory):
        super().__init__()
        self.conv1 = SparseConv3d(in_channels, out_channels, 3, **factory)
        self.norm1 = BatchNorm(out_channels, **factory)
        self.conv2 = SparseConv3d(out_channels, out_channels, 3, **factory)
        self.norm2 = BatchNorm(out_channels, **factory)
        self.relu = ReLU(inplace=True)
        self.project = None
        if in_channels != out_channels:
            self.project = FusedSequential(SparseConv3d(in_channels, out_channels, 1, **factory),
                                           BatchNorm(out_channels, **factory))

    def forward(self, x: SparseTensor) -> SparseTensor:
        skip = x if self.project is None else self.project(x)
        y = conv_norm_act(self.conv1, self.norm1, self.relu, x)
        return conv_norm_act(self.conv2, self.norm2, self.relu, y, residual=skip.F)


class SparseUNet(nn.Module):
    """``in_channels`` -> ``out_channels`` segmentation-style network on a
    SparseTensor of stride 1."""

    def __init__(self, in_channels: int = 4, out_channels: int = 32,
                 encoder=(32, 64, 128, 256), decoder=(128, 64, 32, 32), stem: int = 32,
                 dtype=None, device=None):
        super().__init__()
        factory = {"dtype": dtype, "device": device}
        self.stem = FusedSequential(SparseConv3d(in_channels, stem, 3, **factory),
                                  BatchNorm(stem, **factory), ReLU(inplace=True))
        self.down = nn.ModuleList()
        self.encode = nn.ModuleList()
        widths = [stem]
        for width in encoder:
            self.down.append(FusedSequential(SparseConv3d(widths[-1], width, 2, stride=2, **factory),
                                           BatchNorm(width, **factory), ReLU(inplace=True)))
            self.encode.append(nn.Sequential(ResidualBlock(width, width, **factory),
                                             ResidualBlock(width, width, **factory)))
            widths.append(width)
        self.up = nn.ModuleList()
        self.decode = nn.ModuleList()
        current = widths[-1]
        for level, width in enumerate(decoder):
            skip = widths[len(encoder) - 1 - level]
            self.up.append(FusedSequential(
                SparseConv(3, current, width, 2, stride=2, transposed=True, **factory),
                BatchNorm(width, **factory), ReLU(inplace=True)))
            self.decode.append(nn.Sequential(ResidualBlock(width + skip, width, **factory),
                                             ResidualBlock(width, width, **factory)))
            current = width
        self.head = SparseConv3d(current, out_channels, 1, **factory)

    def forward(self, x: SparseTensor) -> SparseTensor:
        x = self.stem(x)
        skips = [x]
        for down, encode in zip(self.down, self.encode):
            x = encode(down(x))
            skips.append(x)
        skips.pop()
        for up, decode in zip(self.up, self.decode):
            x = decode(F.cat([up(x), skips.pop()]))
        return self.head(x)
