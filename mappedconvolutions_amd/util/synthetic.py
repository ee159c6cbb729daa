"""Synthetic sample maps and point sets used by the tests and the benchmark.

Everything is generated on the CPU with numpy in float64 from a fixed rule or a
seeded generator and returned as torch tensors, so CPU checkers and GPU kernels
see identical bits.
"""
import math

import numpy as np
import torch


def latitude_map(height, width, radius=1, dtype=torch.float32):
    """Latitude-distorted square kernel on an equirectangular grid.

    For output pixel (i, j): lat = ((i + 0.5) / H) * pi - pi/2; taps are ordered
    dy-major over offsets {-r..r}^2; x = (j + dx / max(cos lat, 0.05)) mod W,
    y = clamp(i + dy, 0, H - 1).  Returns [H, W, (2r+1)^2, 2] with (x, y) last.
    """
    i = np.arange(height, dtype=np.float64)[:, None, None]
    j = np.arange(width, dtype=np.float64)[None, :, None]
    offs = np.arange(-radius, radius + 1, dtype=np.float64)
    dy, dx = np.meshgrid(offs, offs, indexing='ij')
    dy, dx = dy.reshape(1, 1, -1), dx.reshape(1, 1, -1)
    lat = ((i + 0.5) / height) * math.pi - math.pi / 2
    stretch = 1.0 / np.maximum(np.cos(lat), 0.05)
    x = np.mod(j + dx * stretch, width)
    y = np.clip(i + dy, 0, height - 1) + 0 * j
    out = np.stack([np.broadcast_to(x, y.shape), y], axis=-1)
    return torch.from_numpy(np.ascontiguousarray(out)).to(dtype)


def identity_grid_map(height, width, radius=1, dtype=torch.float32):
    """Regular grid taps x = j + dx, y = i + dy (dy-major): with this map a mapped
    convolution equals a zero-padded (2r+1)x(2r+1) convolution."""
    i = np.arange(height, dtype=np.float64)[:, None, None]
    j = np.arange(width, dtype=np.float64)[None, :, None]
    offs = np.arange(-radius, radius + 1, dtype=np.float64)
    dy, dx = np.meshgrid(offs, offs, indexing='ij')
    x = j + dx.reshape(1, 1, -1) + 0 * i
    y = i + dy.reshape(1, 1, -1) + 0 * j
    return torch.from_numpy(np.ascontiguousarray(np.stack([x, y], axis=-1))).to(dtype)


def cube_to_equirect_map(face_dim, height, width, dtype=torch.float32):
    """Equirectangular (x, y) of every pixel centre of a horizontally tiled
    cube map [face_dim, 6 * face_dim], faces ordered -z, -x, +z, +x, +y, -y.

    Exact gnomonic projection: pixel (u, v) of a face -> point on the cube
    (face/axis convention of the reference's layers/util/conversions.py:123-180)
    -> lon = atan2(x, z), lat = atan2(-y, sqrt(x^2 + z^2)) (:19-29) ->
    x = (W/2)(lon/pi + 1), y = ((H-1)/2)(1 - 2 lat/pi) (:6-16).
    Returns [face_dim, 6 * face_dim, 2].
    """
    v, u = np.meshgrid(np.arange(face_dim, dtype=np.float64),
                       np.arange(face_dim, dtype=np.float64), indexing='ij')
    u = 2 * (u + 0.5) / face_dim - 1
    v = 2 * (v + 0.5) / face_dim - 1
    one = np.ones_like(u)
    faces = [(-u, -v, -one), (-one, -v, u), (u, -v, one), (one, -v, -u), (u, one, v),
             (u, -one, -v)]
    cols = []
    for (x, y, z) in faces:
        lon = np.arctan2(x, z)
        lat = np.arctan2(-y, np.sqrt(x * x + z * z))
        px = (width / 2) * (lon / math.pi + 1)
        py = ((height - 1) / 2) * (1 - 2 * lat / math.pi)
        cols.append(np.stack([px, py], axis=-1))
    out = np.concatenate(cols, axis=1)
    return torch.from_numpy(np.ascontiguousarray(out)).to(dtype)


def pixel_shuffle_map(height, width, seed=0, dtype=torch.float32):
    """The map of the reference's timing sweep (profile/profile_mapped_convolution.py:16-37,
    78-81): the pixels of an H x W image are shuffled by a random permutation; tap (a, b) of
    output pixel (i, j) points at the shuffled position of grid cell (i + a - 1, j + b - 1)
    (cells outside the grid at (-1, -1)), plus 0.5 in x and y so that a bilinear tap blends four
    unrelated pixels.  Returns [H, W, 9, 2]."""
    rng = np.random.default_rng(seed)
    perm = rng.permutation(height * width)
    x = np.full((height + 2, width + 2), -1.0)
    y = np.full((height + 2, width + 2), -1.0)
    x[1:-1, 1:-1] = (perm % width).reshape(height, width)
    y[1:-1, 1:-1] = (perm // width).reshape(height, width)
    taps = [np.stack([x[a:a + height, b:b + width], y[a:a + height, b:b + width]], -1)
            for a in range(3) for b in range(3)]
    out = np.stack(taps, axis=2) + 0.5
    return torch.from_numpy(np.ascontiguousarray(out)).to(dtype)


def mesh_weighted_map(num_vertices, kernel_size, num_points, seed=0, dtype=torch.float32):
    """Weighted map of a mesh signal stored as a [1, V] image: every tap blends
    `num_points` vertices.  x = integer vertex index ~ U{0..V-1} (stored as a
    float), y = 0; weights ~ Dirichlet(1,..,1).  Returns
    (sample_map [1, V, K, P, 2], interp_weights [1, V, K, P])."""
    rng = np.random.default_rng(seed)
    idx = rng.integers(0, num_vertices, size=(1, num_vertices, kernel_size, num_points))
    smap = np.stack([idx.astype(np.float64), np.zeros(idx.shape)], axis=-1)
    w = rng.dirichlet(np.ones(num_points), size=(1, num_vertices, kernel_size))
    return (torch.from_numpy(smap).to(dtype), torch.from_numpy(w).to(dtype))


def sphere_points(n, seed=0, dtype=torch.float32):
    """n points uniform on the unit sphere (normalised N(0, I3)), shape [1, 3, n]."""
    rng = np.random.default_rng(seed)
    p = rng.standard_normal((3, n))
    p /= np.linalg.norm(p, axis=0, keepdims=True)
    return torch.from_numpy(p[None]).to(dtype).contiguous()


def upsampling_map(src_height, src_width, factor, radius=1, latitude=False, aligned=False,
                   dtype=torch.float32):
    """Square kernel of an output grid `factor` times finer than the source image it samples:
    [factor*H, factor*W, (2r+1)^2, 2].  Output pixel (i, j) sits at source position
    ((j + 0.5) / f - 0.5, (i + 0.5) / f - 0.5), or (j / f, i / f) with `aligned` (coordinates
    are then multiples of 1/f: integral, .5, ...).  Taps are dy-major at unit source spacing;
    with `latitude` the x offsets are stretched by 1 / max(cos lat, 0.05) and wrap around.
    About factor^2 output pixels share every source pixel: the strongly many-to-one case of a
    scatter through the map."""
    oh, ow = src_height * factor, src_width * factor
    i = np.arange(oh, dtype=np.float64)[:, None, None]
    j = np.arange(ow, dtype=np.float64)[None, :, None]
    cy = i / factor if aligned else (i + 0.5) / factor - 0.5
    cx = j / factor if aligned else (j + 0.5) / factor - 0.5
    offs = np.arange(-radius, radius + 1, dtype=np.float64)
    dy, dx = np.meshgrid(offs, offs, indexing='ij')
    dy, dx = dy.reshape(1, 1, -1), dx.reshape(1, 1, -1)
    if latitude:
        lat = ((i + 0.5) / oh) * math.pi - math.pi / 2
        x = np.mod(cx + dx / np.maximum(np.cos(lat), 0.05), src_width)
        y = np.clip(cy + dy, 0, src_height - 1) + 0 * j
    else:
        x = cx + dx + 0 * i
        y = cy + dy + 0 * j
    out = np.stack([np.broadcast_to(x, y.shape), y], axis=-1)
    return torch.from_numpy(np.ascontiguousarray(out)).to(dtype)


def subdivided_icosahedron(order):
    """Triangle mesh of the unit sphere: midpoint subdivision of the icosahedron, every new
    vertex pushed onto the sphere (10 * 4^order + 2 vertices, 20 * 4^order faces).  Not the
    reference's Loop-subdivided icosphere, whose vertex order differs.  Returns
    (vertices [V, 3] float32, faces [F, 3] int64)."""
    r = (1.0 + 5 ** 0.5) / 2
    v = [(-1, r, 0), (1, r, 0), (-1, -r, 0), (1, -r, 0), (0, -1, r), (0, 1, r), (0, -1, -r),
         (0, 1, -r), (r, 0, -1), (r, 0, 1), (-r, 0, -1), (-r, 0, 1)]
    f = [(0, 11, 5), (0, 5, 1), (0, 1, 7), (0, 7, 10), (0, 10, 11), (1, 5, 9), (5, 11, 4),
         (11, 10, 2), (10, 7, 6), (7, 1, 8), (3, 9, 4), (3, 4, 2), (3, 2, 6), (3, 6, 8),
         (3, 8, 9), (4, 9, 5), (2, 4, 11), (6, 2, 10), (8, 6, 7), (9, 8, 1)]
    v = [np.array(p, np.float64) / np.linalg.norm(p) for p in v]
    for _ in range(order):
        cache, nf = {}, []

        def mid(a, b):
            key = (min(a, b), max(a, b))
            if key not in cache:
                m = v[a] + v[b]
                v.append(m / np.linalg.norm(m))
                cache[key] = len(v) - 1
            return cache[key]
        for a, b, c in f:
            ab, bc, ca = mid(a, b), mid(b, c), mid(c, a)
            nf += [(a, ab, ca), (b, bc, ab), (c, ca, bc), (ab, bc, ca)]
        f = nf
    return (torch.from_numpy(np.array(v, np.float32)), torch.from_numpy(np.array(f, np.int64)))
