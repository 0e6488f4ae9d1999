"""Inference-time folding of the layers that follow a convolution into the
convolution's own output pass.

The reference's networks are chains of ``SparseConv -> BatchNorm -> ReLU``
modules (minuet/nn/convolutions.py, normalizations.py, activations.py), each
a full read and write of the feature tensor.  In evaluation mode a BatchNorm
is a per-channel affine map, so it, the activation and a residual sum can be
applied while Scatter still holds the output row in registers.  Nothing here
changes parameters or ``state_dict`` keys, and in training mode every module
runs as written."""
from collections import OrderedDict
from typing import Optional

import torch
from torch import nn

from minuet_amd.nn import functional as F
from minuet_amd.nn.activations import LeakyReLU, ReLU, ReLU6
from minuet_amd.nn.convolutions import SparseConv
from minuet_amd.nn.normalizations import BatchNorm
from minuet_amd.tensors import SparseTensor

__all__ = ["batch_norm_affine", "conv_norm_act", "FusedSequential", "fuse_conv_norm_act"]


def batch_norm_affine(norm: torch.nn.BatchNorm1d):
    """``(scale, shift)`` in fp32 with ``norm(x) == x * scale + shift`` in
    evaluation mode.  Cached on the module until one of its tensors changes."""
    # straight from the module's dictionaries: nn.Module.__getattr__ is the slow way in
    buffers, parameters = norm._buffers, norm._parameters
    mean, var = buffers["running_mean"], buffers["running_var"]
    weight, bias = parameters["weight"], parameters["bias"]
    key = (mean.data_ptr(), mean._version, var.data_ptr(), var._version,
           None if weight is None else (weight.data_ptr(), weight._version),
           None if bias is None else (bias.data_ptr(), bias._version))
    cached = norm.__dict__.get("_minuet_affine")
    if cached is not None and cached[0] == key:
        return cached[1], cached[2]
    with torch.no_grad():
        scale = torch.rsqrt(norm.running_var.float() + norm.eps)
        if norm.weight is not None:
            scale = scale * norm.weight.float()
        shift = -norm.running_mean.float() * scale
        if norm.bias is not None:
            shift = shift + norm.bias.float()
    norm.__dict__["_minuet_affine"] = (key, scale, shift)
    return scale, shift


def _activation_of(module):
    if isinstance(module, (ReLU, nn.ReLU)):
        return "relu", 0.0
    if isinstance(module, (LeakyReLU, nn.LeakyReLU)):
        return "leaky_relu", module.negative_slope
    if isinstance(module, (ReLU6, nn.ReLU6)):
        return "relu6", 0.0
    return None


def _foldable(norm) -> bool:
    return (isinstance(norm, torch.nn.BatchNorm1d) and not norm.training
            and norm._buffers.get("running_mean") is not None)


def conv_norm_act(conv: SparseConv, norm: Optional[torch.nn.BatchNorm1d], act: Optional[nn.Module],
                  x: SparseTensor, residual: Optional[torch.Tensor] = None) -> SparseTensor:
    """``act(norm(conv(x)) + residual)``.  One pass when ``norm`` is in
    evaluation mode (or absent) and ``act`` is a ReLU / LeakyReLU / ReLU6 (or
    absent); otherwise the modules run one after another."""
    kind = _activation_of(act) if act is not None else ("none", 0.0)
    if (norm is None or _foldable(norm)) and kind is not None and x.F.is_cuda:
        scale, shift = batch_norm_affine(norm) if norm is not None else (None, None)
        epilogue = F.Epilogue(scale, shift, residual, None if kind[0] == "none" else kind[0], kind[1])
        return conv(x, epilogue=epilogue)
    y = conv(x)
    if norm is not None:
        y = norm(y) if isinstance(norm, BatchNorm) else _like(y, norm(y.F))
    if residual is not None:
        y = _like(y, y.F + residual)
    if act is not None:
        y = act(y) if isinstance(act, (ReLU, LeakyReLU, ReLU6)) else _like(y, act(y.F))
    return y


def _like(x: SparseTensor, features: torch.Tensor) -> SparseTensor:
    return SparseTensor.like(x, features)


class FusedSequential(nn.Sequential):
    """``nn.Sequential`` that runs every ``SparseConv [-> BatchNorm] [-> ReLU]``
    run of its children through :func:`conv_norm_act`.  Children, their names
    and therefore the ``state_dict`` are those of the plain container."""

    def forward(self, x):
        children = list(self)
        i = 0
        while i < len(children):
            module = children[i]
            if isinstance(module, SparseConv) and not self.training:
                norm = act = None
                j = i + 1
                if j < len(children) and _foldable(children[j]):
                    norm = children[j]
                    j += 1
                if j < len(children) and _activation_of(children[j]) is not None:
                    act = children[j]
                    j += 1
                x = conv_norm_act(module, norm, act, x)
                i = j
            else:
                x = module(x)
                i += 1
        return x


def fuse_conv_norm_act(model: nn.Module) -> nn.Module:
    """Replaces every plain ``nn.Sequential`` below (and including) ``model``
    by a :class:`FusedSequential` over the same children.  Returns the
    (possibly new) root."""
    for name, child in list(model.named_children()):
        setattr(model, name, fuse_conv_norm_act(child))
    if type(model) is nn.Sequential:
        return FusedSequential(OrderedDict(model.named_children()))
    return model
