"""Argument checks shared by the mapped layers.

Same rules and AssertionError behaviour as the reference's
layers/nn/layer_utils.py:21-148, with one documented relaxation: bfloat16 data
takes float32 sample maps / interpolation weights.
"""
from collections.abc import Iterable

import torch

INTERPOLATIONS = {'nearest': 0, 'bilinear': 1, 'bispherical': 2}


def interpolation_code(name):
    """'nearest' -> 0, 'bilinear' -> 1, 'bispherical' -> 2; anything else asserts."""
    assert name in INTERPOLATIONS, 'Unsupported interpolation type'
    return INTERPOLATIONS[name]


def _ntuple(n):
    def parse(x):
        return x if isinstance(x, Iterable) else tuple(x for _ in range(n))
    return parse


_pair = _ntuple(2)


def _map_dtype_for(input):
    return torch.float32 if input.dtype == torch.bfloat16 else input.dtype


def check_type(input, sample_map, interp_weights=None):
    want = _map_dtype_for(input)
    assert sample_map.dtype == want, \
        'Input and sample map must be the same dtype ({} != {})'.format(
            input.dtype, sample_map.dtype)
    if interp_weights is not None:
        assert interp_weights.dtype == want, \
            'Input and interpolation weights must be the same dtype ' \
            '({} != {})'.format(input.dtype, interp_weights.dtype)


def check_input_dim(input):
    assert input.dim() == 4, \
        'Input must have 4 dimensions ({} != 4)'.format(input.dim())


def check_sample_map_dim(sample_map, interp_weights=None, kernel=True):
    """[OH, OW, (K,) (P,) 2]: K present for kernel ops, P present when weighted."""
    want = 3 + int(kernel) + int(interp_weights is not None)
    assert sample_map.dim() == want, \
        'Sample map must have {} dimensions ({} != {})'.format(want, sample_map.dim(), want)
    assert sample_map.shape[-1] == 2, \
        'Last dimension of sample map must have size 2 ({} != 2)'.format(sample_map.shape[-1])


def check_interp_weights_dim(interp_weights, kernel=True):
    want = 3 + int(kernel)
    assert interp_weights.dim() == want, \
        'Interpolation  weights must have {} dimensions ({} != {})'.format(
            want, interp_weights.dim(), want)


def check_input_shape(input, in_channels):
    assert input.shape[1] == in_channels, \
        'Number of input channels must match weight parameter ' \
        '({} != {})'.format(input.shape[1], in_channels)


def check_sample_map_shape(sample_map, kernel_size):
    assert sample_map.shape[2] == kernel_size, \
        'Kernel size of sample map must match weight parameter ' \
        '({} != {})'.format(sample_map.shape[2], kernel_size)


def check_interp_weights_shape(sample_map, interp_weights):
    assert sample_map.shape[-2] == interp_weights.shape[-1], \
        'Sample map and interpolation weights should have the same number' \
        'of interpolation points ({} != {})'.format(
            sample_map.shape[-2], interp_weights.shape[-1])


def check_input_map_shape(input, sample_map):
    assert tuple(input.shape[2:4]) == tuple(sample_map.shape[0:2]), \
        'Input dimensions 2 and 3 must match sample map dimensions 0 ' \
        'and 1 ({},{}) != ({},{}))'.format(input.shape[2], input.shape[3],
                                           sample_map.shape[0], sample_map.shape[1])


def check_args(input, sample_map, interp_weights, in_channels, kernel_size):
    kernel = kernel_size is not None
    check_input_dim(input)
    check_sample_map_dim(sample_map, interp_weights, kernel)
    if interp_weights is not None:
        check_interp_weights_dim(interp_weights, kernel)
    check_type(input, sample_map, interp_weights)
    if in_channels is not None:
        check_input_shape(input, in_channels)
    if kernel:
        check_sample_map_shape(sample_map, kernel_size)
    if interp_weights is not None:
        check_interp_weights_shape(sample_map, interp_weights)


class OwnedPlan:
    """The map plan of a layer whose sample map stays the same from call to call (a layer
    built with cache_plan=True): one plan, rebuilt when the layer is handed another map
    tensor, a map that was modified in place (torch's version counter; writes through
    `.data` are not seen), or another sampled size or data type."""

    def __init__(self):
        self.key, self.plan = None, None

    def get(self, build, sample_map, interp_weights, *rest):
        def ident(t):
            return None if t is None else (t.data_ptr(), t._version, tuple(t.shape), t.device)
        key = (ident(sample_map), ident(interp_weights)) + tuple(rest)
        if key != self.key:
            self.plan = build()
            self.key = key
        return self.plan
