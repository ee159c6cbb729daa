"""Kernel maps over triangle meshes of the sphere: the host-side helpers of the reference's
package/layers/util/icosphere_functions.py:132-262 with the mesh handed over as tensors
(vertices [V, 3], faces [F, 3]) instead of a `Sphere` object, and the face search on the GPU.

    spherical = convert_3d_to_spherical(vertices)                  # [V, 2] (lon, lat)
    samples = gnomonic_kernel(spherical, kh, kw, res, res)         # [1, V, kh*kw, 2]
    idx, w = kernel_map_from_samples(samples, vertices, faces)     # [1, V, K, 3, 2], [1, V, K, 3]
    y = MappedConvolution(C, C2, kh*kw, 'nearest')(x, idx, w)      # x: [B, C, 1, V]
"""
import torch

from .. import _C


def convert_3d_to_spherical(xyz):
    """[.., 3] points -> [.., 2] (longitude, latitude), the convention of
    package/layers/util/conversions.py:19-29: lon = atan2(x, z), lat = atan2(-y, sqrt(x^2+z^2))."""
    x, y, z = xyz[..., 0], xyz[..., 1], xyz[..., 2]
    return torch.stack((torch.atan2(x, z), torch.atan2(-y, (x * x + z * z).sqrt())), -1)


def gnomonic_kernel(spherical_coords, kh, kw, res_lat, res_lon):
    """icosphere_functions.py:135-183: a kh x kw grid of spacing (res_lon, res_lat) on the
    tangent plane at every (lon, lat) of `spherical_coords` [V, 2], carried back onto the
    sphere by a device kernel.  Returns [1, V, kh*kw, 2] (lon, lat) on the input's device."""
    centres = spherical_coords.reshape(-1, 2).float().contiguous()
    return _C.gnomonic_samples(centres, kh, kw, res_lat, res_lon)


def kernel_map_from_samples(samples, vertices, faces, nearest=False):
    """The maps a weighted MappedConvolution over mesh vertices takes, from spherical sample
    locations [OH, OW, K, 2]: vertex indices [OH, OW, K, 3, 2] (float; x = index, y = 0, as
    icosphere_functions.py:256-260 stacks them) and barycentric weights [OH, OW, K, 3]."""
    _, vidx, w = _C.planar_conv_operator_from_samples(samples.contiguous().float(), vertices,
                                                      faces, True, nearest)
    vidx = torch.stack((vidx, torch.zeros_like(vidx)), -1)
    return vidx.float(), w


def vertex_resolution(vertices, faces):
    """Sphere::getVertexResolution, package/ext_modules/src/util/cpp/sphere.cpp:610-628: the
    mean over vertices of the mean distance to the adjacent vertices.  (On a closed mesh the
    directed edges of the faces leave every vertex once per neighbour.)"""
    e = torch.cat((faces[:, [0, 1]], faces[:, [1, 2]], faces[:, [2, 0]]), 0)
    length = (vertices[e[:, 1]] - vertices[e[:, 0]]).norm(dim=1)
    total = torch.zeros(vertices.shape[0], device=vertices.device).index_add_(0, e[:, 0], length)
    count = torch.zeros(vertices.shape[0], device=vertices.device).index_add_(
        0, e[:, 0], torch.ones_like(length))
    return (total / count).mean().item()


def vertex_to_vertex_kernel_map(vertices, faces, kh, kw, target_vertices=None, target_faces=None,
                                resolution=None, nearest=False):
    """icosphere_functions.py:226-262: a kh x kw gnomonic kernel centred at every vertex of
    (vertices, faces), sampled from the mesh (target_vertices, target_faces) - the same mesh
    by default, a finer or coarser one for a down- or up-sampling map.  `resolution` is the
    kernel's spacing; default: vertex_resolution(vertices, faces).
    Returns (indices [1, V, kh*kw, 3, 2], weights [1, V, kh*kw, 3])."""
    if target_vertices is None:
        target_vertices, target_faces = vertices, faces
    if resolution is None:
        resolution = vertex_resolution(vertices, faces)
    samples = gnomonic_kernel(convert_3d_to_spherical(vertices), kh, kw, resolution, resolution)
    return kernel_map_from_samples(samples, target_vertices, target_faces, nearest)
