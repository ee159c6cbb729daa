"""MappedConvolution: convolution whose K taps per output pixel come from a
real-valued sample_map.  API of the reference's
layers/nn/mapped_convolution_layer.py:15-121; the work is done by the fused HIP
kernels behind `_C.mapped_conv_forward/backward`."""
import math

import torch
import torch.nn as nn

from .. import _C
from .layer_utils import OwnedPlan, check_args, interpolation_code


class MappedConvolutionFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, weight, bias, sample_map, kernel_size, interp, interp_weights=None,
                plan=None):
        ctx.save_for_backward(input, weight, bias, sample_map, interp_weights)
        ctx.kernel_size, ctx.interp, ctx.plan = int(kernel_size), int(interp), plan
        if interp_weights is not None:
            return _C.weighted_mapped_conv_forward(input, sample_map, interp_weights, weight, bias,
                                                   kernel_size, interp, plan=plan)
        return _C.mapped_conv_forward(input, sample_map, weight, bias, kernel_size, interp,
                                      plan=plan)

    @staticmethod
    def backward(ctx, grad_output):
        input, weight, bias, sample_map, interp_weights = ctx.saved_tensors
        # only the gradients autograd asks for: a first layer (input without gradient) skips
        # the input gradient and its transposed map, a frozen layer its weight gradient
        needs = tuple(ctx.needs_input_grad[:3])
        if interp_weights is not None:
            grads = _C.weighted_mapped_conv_backward(grad_output, sample_map, interp_weights, input,
                                                     weight, bias, ctx.kernel_size, ctx.interp,
                                                     plan=ctx.plan, needs=needs)
        else:
            grads = _C.mapped_conv_backward(grad_output, sample_map, input, weight, bias,
                                            ctx.kernel_size, ctx.interp, plan=ctx.plan,
                                            needs=needs)
        grad_input, grad_weight, grad_bias = grads
        return grad_input, grad_weight, grad_bias, None, None, None, None, None


class MappedConvolution(nn.Module):
    """weight [out_channels, in_channels, kernel_size] (a 1-D kernel: the map
    gives every tap its 2-D location), bias [out_channels].  `bias=False` keeps a
    zero-valued bias parameter, as the reference does.  `cache_plan=True` (not in the
    reference): the layer keeps the map plan of the sample map it is called with (see
    _C.conv_map_plan) for as long as it is called with that same map."""

    def __init__(self, in_channels, out_channels, kernel_size=1, interpolation='bilinear',
                 bias=True, cache_plan=False):
        super().__init__()
        self._plan = OwnedPlan() if cache_plan else None
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.interp = interpolation_code(interpolation)
        self.weight = nn.Parameter(torch.empty(out_channels, in_channels, kernel_size))
        self.bias = nn.Parameter(torch.empty(out_channels))
        self.reset_parameters()
        if not bias:
            self.bias = nn.Parameter(torch.zeros(out_channels))

    def reset_parameters(self):
        """U(-s, s) with s = 1/sqrt(in_channels * kernel_size) for weight and bias."""
        stdv = 1. / math.sqrt(self.in_channels * self.kernel_size)
        self.weight.data.uniform_(-stdv, stdv)
        self.bias.data.uniform_(-stdv, stdv)

    def forward(self, x, sample_map, interp_weights=None):
        """x [B, C, IH, IW]; sample_map [OH, OW, K, 2] as (x, y), or
        [OH, OW, K, P, 2] with interp_weights [OH, OW, K, P]."""
        check_args(x, sample_map, interp_weights, self.in_channels, self.kernel_size)
        plan = None
        if self._plan is not None:
            H, W = x.shape[2], x.shape[3]
            plan = self._plan.get(
                lambda: _C.conv_map_plan(sample_map, interp_weights, H, W, self.interp, x.dtype),
                sample_map, interp_weights, H, W, x.dtype)
        return MappedConvolutionFunction.apply(x, self.weight, self.bias, sample_map,
                                               self.kernel_size, self.interp, interp_weights, plan)
