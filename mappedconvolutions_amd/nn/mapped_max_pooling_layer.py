"""MappedMaxPool.  API of the reference's layers/nn/mapped_max_pooling_layer.py:12-90.
(The reference's MappedMaxUnpool module references undefined names and is not
exported by its package; it has no counterpart here.)"""
import torch
import torch.nn as nn

from .. import _C
from .layer_utils import check_args, interpolation_code


class MappedMaxPoolFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, input, sample_map, kernel_size, interp, interp_weights=None):
        if interp_weights is not None:
            pooled, idx_mask = _C.weighted_mapped_max_pool(input, sample_map, interp_weights,
                                                           kernel_size, interp)
        else:
            pooled, idx_mask = _C.mapped_max_pool(input, sample_map, kernel_size, interp)
        ctx.mark_non_differentiable(idx_mask)
        ctx.save_for_backward(idx_mask, sample_map, interp_weights)
        ctx.input_hw = (int(input.shape[2]), int(input.shape[3]))
        ctx.kernel_size, ctx.interp = int(kernel_size), int(interp)
        return pooled, idx_mask

    @staticmethod
    def backward(ctx, grad_output, idx_mask_grad=None):
        idx_mask, sample_map, interp_weights = ctx.saved_tensors
        ih, iw = ctx.input_hw
        grad_output = grad_output.contiguous()
        if interp_weights is not None:
            grad_input = _C.weighted_mapped_max_unpool(grad_output, idx_mask, sample_map,
                                                       interp_weights, ih, iw, ctx.kernel_size,
                                                       ctx.interp)
        else:
            grad_input = _C.mapped_max_unpool(grad_output, idx_mask, sample_map, ih, iw,
                                              ctx.kernel_size, ctx.interp)
        return grad_input, None, None, None, None


class MappedMaxPool(nn.Module):

    def __init__(self, kernel_size, interpolation='bilinear', return_indices=False):
        super().__init__()
        self.kernel_size = kernel_size
        self.return_indices = return_indices
        self.interp = interpolation_code(interpolation)

    def forward(self, x, sample_map, interp_weights=None):
        check_args(x, sample_map, interp_weights, None, self.kernel_size)
        pooled, idx_mask = MappedMaxPoolFunction.apply(x, sample_map, self.kernel_size,
                                                       self.interp, interp_weights)
        return (pooled, idx_mask) if self.return_indices else pooled
