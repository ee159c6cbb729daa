"""MappedAvgPool / MappedAvgUnpool.  API of the reference's
layers/nn/mapped_avg_pooling_layer.py:12-154.  The weighted unpool call passes
its arguments in the op's declared order (the reference's wrapper at :93-94
swaps them and cannot run)."""
import torch
import torch.nn as nn

from .. import _C
from .layer_utils import check_args, check_input_map_shape, interpolation_code


def _avg_pool(x, sample_map, interp_weights, kernel_size, interp):
    if interp_weights is not None:
        return _C.weighted_mapped_avg_pool(x, sample_map, interp_weights, kernel_size, interp)
    return _C.mapped_avg_pool(x, sample_map, kernel_size, interp)


def _avg_unpool(g, sample_map, interp_weights, h, w, kernel_size, interp):
    if interp_weights is not None:
        return _C.weighted_mapped_avg_unpool(g, sample_map, interp_weights, h, w, kernel_size,
                                             interp)
    return _C.mapped_avg_unpool(g, sample_map, h, w, kernel_size, interp)


class MappedAvgPoolFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, sample_map, kernel_size, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.input_hw = (int(input.shape[2]), int(input.shape[3]))
        ctx.kernel_size, ctx.interp = int(kernel_size), int(interp)
        return _avg_pool(input, sample_map, interp_weights, kernel_size, interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        ih, iw = ctx.input_hw
        grad_input = _avg_unpool(grad_output.contiguous(), sample_map, interp_weights, ih, iw,
                                 ctx.kernel_size, ctx.interp)
        return grad_input, None, None, None, None


class MappedAvgPool(nn.Module):

    def __init__(self, kernel_size, interpolation='bilinear'):
        super().__init__()
        self.kernel_size = kernel_size
        self.interp = interpolation_code(interpolation)

    def forward(self, x, sample_map, interp_weights=None):
        check_args(x, sample_map, interp_weights, None, self.kernel_size)
        return MappedAvgPoolFunction.apply(x, sample_map, self.kernel_size, self.interp,
                                           interp_weights)


class MappedAvgUnpoolFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, oh, ow, sample_map, kernel_size, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.kernel_size, ctx.interp = int(kernel_size), int(interp)
        return _avg_unpool(input, sample_map, interp_weights, oh, ow, kernel_size, interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        grad_input = _avg_pool(grad_output.contiguous(), sample_map, interp_weights,
                               ctx.kernel_size, ctx.interp)
        return (grad_input,) + (None,) * 6


class MappedAvgUnpool(nn.Module):

    def __init__(self, kernel_size, interpolation='bilinear'):
        super().__init__()
        self.kernel_size = kernel_size
        self.interp = interpolation_code(interpolation)

    def forward(self, x, oh, ow, sample_map, interp_weights=None):
        """x [B, C, IH, IW]; sample_map [IH, IW, K, (P,) 2] pointing into the oh x ow output."""
        check_args(x, sample_map, interp_weights, None, self.kernel_size)
        check_input_map_shape(x, sample_map)
        return MappedAvgUnpoolFunction.apply(x, oh, ow, sample_map, self.kernel_size, self.interp,
                                             interp_weights)
