"""Resample (scatter input pixels to real-valued output locations) and Unresample
(gather real-valued locations into an output grid).  API of the reference's
layers/nn/resample_layer.py:14-140."""
import torch
import torch.nn as nn

from .. import _C
from .layer_utils import check_args, check_input_map_shape, interpolation_code


def _to_map(x, sample_map, interp_weights, oh, ow, interp):
    if interp_weights is not None:
        return _C.weighted_resample_to_map(x, sample_map, interp_weights, oh, ow, interp)
    return _C.resample_to_map(x, sample_map, oh, ow, interp)


def _from_map(x, sample_map, interp_weights, interp):
    if interp_weights is not None:
        return _C.weighted_resample_from_map(x, sample_map, interp_weights, interp)
    return _C.resample_from_map(x, sample_map, interp)


class ResampleFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, sample_map, output_shape, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.interp = int(interp)
        return _to_map(input, sample_map, interp_weights, int(output_shape[0]),
                       int(output_shape[1]), interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        grad_input = _from_map(grad_output.contiguous(), sample_map, interp_weights, ctx.interp)
        return grad_input, None, None, None, None


class Resample(nn.Module):
    """Maps integer input locations to real-valued output locations."""

    def __init__(self, interpolation='bilinear'):
        super().__init__()
        self.interp = interpolation_code(interpolation)

    def forward(self, x, sample_map, output_shape, interp_weights=None):
        """x [B, C, IH, IW]; sample_map [IH, IW, (P,) 2]; output_shape (OH, OW)."""
        check_args(x, sample_map, interp_weights, None, None)
        check_input_map_shape(x, sample_map)
        return ResampleFunction.apply(x, sample_map, output_shape, self.interp, interp_weights)


class UnresampleFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, sample_map, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.interp = int(interp)
        ctx.input_hw = (int(input.shape[2]), int(input.shape[3]))
        return _from_map(input, sample_map, interp_weights, interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        ih, iw = ctx.input_hw
        grad_input = _to_map(grad_output.contiguous(), sample_map, interp_weights, ih, iw,
                             ctx.interp)
        return grad_input, None, None, None


class Unresample(nn.Module):
    """Maps real-valued input locations to an integer output grid: a mapped
    convolution with unit weights, no bias and kernel size 1."""

    def __init__(self, interpolation='bilinear'):
        super().__init__()
        self.interp = interpolation_code(interpolation)

    def forward(self, x, sample_map, interp_weights=None):
        """x [B, C, IH, IW]; sample_map [OH, OW, (P,) 2]."""
        check_args(x, sample_map, interp_weights, None, None)
        return UnresampleFunction.apply(x, sample_map, self.interp, interp_weights)
