"""Sample-map builders with the reference's names and arguments
(package/layers/util/spherical_projections.py), computed on the GPU.

The reference evaluates these maps with torch expressions on the host and the
caller moves them to the device; here a kernel writes the map straight into
device memory (`device` defaults to the current GPU), in float32 like the
reference's.  Every entry is the formula's value evaluated in double and rounded
once, so it can differ from the reference's step-by-step float evaluation by that
evaluation's own rounding error (largest next to the poles, where asin amplifies
it).  A longitude that lands on the +/-pi seam maps to x = 0 or x = W depending
on rounding, in the reference as here; both name the same sample under
'bispherical' interpolation.
"""
import torch

from .. import _C


def _device(device):
    return torch.device("cuda", torch.cuda.current_device()) if device is None else device


def get_projection_map(shape, kernel_size, proj='grid', stride=1, dilation=1, device=None):
    """spherical_projections.py:12-24: 'gnomonic' and 'equirectangular' give pixel
    coordinates, any other value the lon/lat grid in radians."""
    if proj not in ('gnomonic', 'equirectangular'):
        proj = 'grid'
    return _C.projection_map(shape, kernel_size, proj, stride, dilation, _device(device))


def get_perspective_projection_map(shape, kernel_size, stride=1, dilation=1, device=None):
    """spherical_projections.py:33-35: the regular grid of a planar convolution."""
    return _C.projection_map(shape, kernel_size, 'perspective', stride, dilation,
                             _device(device))


def get_reverse_cube_projection_map(cube_dim, kernel_size, stride=1, device=None):
    """spherical_projections.py:26-30: map into the dim x 6*dim cube-map image."""
    return _C.cube_projection_map(cube_dim, kernel_size, stride, _device(device))


def cube_to_rect(cubemap, rect_height, rect_width, interpolation='nearest'):
    """spherical_projections.py:196-213: cubemap [C, dim, 6*dim], faces laid out as
    [-z, -x, +z, +x, +y, -y], to an equirectangular image [C, rect_height, rect_width]."""
    assert len(cubemap.shape) == 3, 'Cubemape must have 3 dimensions'
    if interpolation == 'nearest':
        interp = 0
    elif interpolation == 'bilinear':
        interp = 1
    else:
        assert False, 'Invalid interpolation option'
    return _C.cube2rect(cubemap, rect_height, rect_width, interp)
