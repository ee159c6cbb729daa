"""MappedTransposedConvolution: the adjoint arrangement of a mapped convolution.
The sample_map has the INPUT's spatial size and points into the OUTPUT.  API of
the reference's layers/nn/mapped_transposed_convolution_layer.py:15-121."""
import math

import torch
import torch.nn as nn

from .. import _C
from .layer_utils import OwnedPlan, check_args, check_input_map_shape, interpolation_code


class MappedTransposedConvolutionFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, weight, bias, sample_map, output_height, output_width, kernel_size,
                interp, interp_weights=None, plan=None):
        ctx.save_for_backward(input, sample_map, weight, bias, interp_weights)
        ctx.kernel_size, ctx.interp, ctx.plan = int(kernel_size), int(interp), plan
        if interp_weights is not None:
            return _C.weighted_mapped_transposed_conv_forward(
                input, sample_map, interp_weights, weight, bias, output_height, output_width,
                kernel_size, interp, plan=plan)
        return _C.mapped_transposed_conv_forward(input, sample_map, weight, bias, output_height,
                                                 output_width, kernel_size, interp, plan=plan)

    @staticmethod
    def backward(ctx, grad_output):
        input, sample_map, weight, bias, interp_weights = ctx.saved_tensors
        needs = tuple(ctx.needs_input_grad[:3])  # only the gradients autograd asks for
        if interp_weights is not None:
            grads = _C.weighted_mapped_transposed_conv_backward(
                grad_output, sample_map, interp_weights, input, weight, bias, ctx.kernel_size,
                ctx.interp, plan=ctx.plan, needs=needs)
        else:
            grads = _C.mapped_transposed_conv_backward(grad_output, sample_map, input, weight,
                                                       bias, ctx.kernel_size, ctx.interp,
                                                       plan=ctx.plan, needs=needs)
        grad_input, grad_weight, grad_bias = grads
        return (grad_input, grad_weight, grad_bias) + (None,) * 7


class MappedTransposedConvolution(nn.Module):
    """weight [in_channels, out_channels, kernel_size], bias [out_channels].  `cache_plan`: see
    MappedConvolution."""

    def __init__(self, in_channels, out_channels, kernel_size=1, interpolation='bilinear',
                 bias=True, cache_plan=False):
        super().__init__()
        self._plan = OwnedPlan() if cache_plan else None
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.interp = interpolation_code(interpolation)
        self.weight = nn.Parameter(torch.empty(in_channels, out_channels, kernel_size))
        self.bias = nn.Parameter(torch.empty(out_channels))
        self.reset_parameters()
        if not bias:
            self.bias = nn.Parameter(torch.zeros(out_channels))

    def reset_parameters(self):
        stdv = 1. / math.sqrt(self.in_channels * self.kernel_size)
        self.weight.data.uniform_(-stdv, stdv)
        self.bias.data.uniform_(-stdv, stdv)

    def forward(self, x, oh, ow, sample_map, interp_weights=None):
        """x [B, C, IH, IW]; oh, ow: output size; sample_map [IH, IW, K, (P,) 2]."""
        check_args(x, sample_map, interp_weights, self.in_channels, self.kernel_size)
        check_input_map_shape(x, sample_map)
        plan = None
        if self._plan is not None:  # the map samples the OUTPUT
            plan = self._plan.get(
                lambda: _C.conv_map_plan(sample_map, interp_weights, oh, ow, self.interp, x.dtype),
                sample_map, interp_weights, int(oh), int(ow), x.dtype)
        return MappedTransposedConvolutionFunction.apply(x, self.weight, self.bias, sample_map, oh,
                                                         ow, self.kernel_size, self.interp,
                                                         interp_weights, plan)
