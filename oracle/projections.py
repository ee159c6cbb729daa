"""TEST INFRASTRUCTURE: numpy restatement of the reference's sample-map builders and of
its cube-map -> equirectangular kernel.

Each function follows the cited reference lines operation by operation, in the numpy
dtype given: float32 reproduces the reference's own arithmetic (torch's default dtype),
float64 gives the value of the same formulas with negligible rounding.  The reference
holds no test or fixture for these functions, so the restatement is pinned by what the
mathematics fixes (tests/test_projections.py): the forward gnomonic projection inverts
the gnomonic map, the equirectangular map has the closed form (j + cj / cos(lat'),
i - ci), cube conversion round-trips, known directions land on known faces, and
cube2rect of a cube map that holds a linear function of the face coordinates returns
that function.
"""
import math

import numpy as np


# ------------------------------------------------------------------ helpers
def _linspace(start, end, steps, dt):
    """torch.linspace for a floating dtype: step = (end - start) / (steps - 1); the first
    half counts up from `start`, the second half down from `end`."""
    start, end = dt(start), dt(end)
    if steps == 1:
        return np.array([start], dtype=dt)
    step = dt((end - start) / dt(steps - 1))
    idx = np.arange(steps)
    lo = (start + step * idx.astype(dt)).astype(dt)
    hi = (end - step * (steps - 1 - idx).astype(dt)).astype(dt)
    return np.where(idx < steps // 2, lo, hi).astype(dt)


def _remainder(a, b):
    """torch's `%` on tensors: the result takes the sign of the divisor."""
    return np.mod(a, b)


def _kernel_offsets(kernel_size):
    kh, kw = kernel_size
    ci = np.repeat(np.arange(kh) - kh // 2, kw)
    cj = np.tile(np.arange(kw) - kw // 2, kh)
    return ci, cj


def equirectangular_meshgrid(shape, dt=np.float32):
    """spherical_projections.py:106-114 (the definition in that file, which shadows the one
    imported from grids.py: latitude runs from +pi/2 down to -pi/2)."""
    H, W = shape
    lat = _linspace(math.pi / 2, -math.pi / 2, H, dt).reshape(H, 1, 1)
    lon = _linspace(-math.pi, math.pi, W + 1, dt)[:-1].reshape(1, W, 1)
    return lat, lon, math.pi / (H - 1), 2 * math.pi / W


def convert_spherical_to_image(rad, shape):
    """conversions.py:6-17."""
    H, W = shape
    dt = rad.dtype.type
    xy = rad.copy()
    xy[..., 0] = dt(W / 2) * (xy[..., 0] / dt(math.pi) + dt(1))
    xy[..., 1] = dt((H - 1) / 2) * (dt(-2) * xy[..., 1] / dt(math.pi) + dt(1))
    return xy


# ------------------------------------------------------------------ map builders
def grid_projection_map(shape, kernel_size, dilation=1, dt=np.float32):
    """spherical_projections.py:39-70."""
    lat, lon, res_lat, res_lon = equirectangular_meshgrid(shape, dt)
    ci, cj = _kernel_offsets(kernel_size)
    y = (ci * dilation * res_lat).astype(dt).reshape(1, 1, -1)
    x = (cj * dilation * res_lon).astype(dt).reshape(1, 1, -1)
    out_lat = y + lat + np.zeros_like(lon)
    out_lon = x + lon + np.zeros_like(lat)
    return np.stack((out_lon, out_lat), -1).astype(dt)


def perspective_projection_map(shape, kernel_size, dilation=1, dt=np.float32):
    """spherical_projections.py:73-103."""
    H, W = shape
    ci, cj = _kernel_offsets(kernel_size)
    r = np.arange(H, dtype=dt).reshape(H, 1, 1)
    c = np.arange(W, dtype=dt).reshape(1, W, 1)
    y = (ci * dilation).astype(dt).reshape(1, 1, -1)
    x = (cj * dilation).astype(dt).reshape(1, 1, -1)
    return np.stack((x + c + 0 * r, y + r + 0 * c), -1).astype(dt)


def reverse_equirectangular_projection_map(shape, kernel_size, dt=np.float32):
    """spherical_projections.py:117-150."""
    lat, lon, res_lat, res_lon = equirectangular_meshgrid(shape, dt)
    ci, cj = _kernel_offsets(kernel_size)
    x = (cj * res_lon).astype(dt).reshape(1, 1, -1)
    y = (ci * res_lat).astype(dt).reshape(1, 1, -1)
    out_lat = y + lat
    out_lon = x / np.cos(out_lat) + lon
    out_lon = _remainder(out_lon + dt(math.pi), dt(2 * math.pi)) - dt(math.pi)
    out_lat = out_lat + np.zeros_like(out_lon)
    return np.stack((out_lon, out_lat), -1).astype(dt)


def reverse_gnomonic_projection_map(shape, kernel_size, dt=np.float32):
    """spherical_projections.py:153-193."""
    kh, kw = kernel_size
    lat, lon, res_lat, res_lon = equirectangular_meshgrid(shape, dt)
    ci, cj = _kernel_offsets(kernel_size)
    x = (cj * res_lon).astype(dt).reshape(1, 1, -1)
    y = (ci * res_lat).astype(dt).reshape(1, 1, -1)
    with np.errstate(invalid="ignore", divide="ignore"):
        rho = np.sqrt(x ** 2 + y ** 2)
        nu = np.arctan(rho)
        out_lat = np.arcsin(np.cos(nu) * np.sin(lat) + y * np.sin(nu) * np.cos(lat) / rho)
        out_lon = lon + np.arctan2(x * np.sin(nu),
                                   rho * np.cos(lat) * np.cos(nu) - y * np.sin(lat) * np.sin(nu))
    out_lat = out_lat + np.zeros_like(out_lon)
    centre = kh * kw // 2
    out_lat[..., centre] = (lat + np.zeros_like(lon))[..., 0]
    out_lon[..., centre] = (lon + np.zeros_like(lat))[..., 0]
    out_lon = _remainder(out_lon + dt(math.pi), dt(2 * math.pi)) - dt(math.pi)
    return np.stack((out_lon, out_lat), -1).astype(dt)


def get_projection_map(shape, kernel_size, proj="grid", stride=1, dilation=1, dt=np.float32):
    """spherical_projections.py:12-24."""
    if proj == "gnomonic":
        m = reverse_gnomonic_projection_map(shape, kernel_size, dt)
        m = convert_spherical_to_image(m, m.shape[:2])
    elif proj == "equirectangular":
        m = reverse_equirectangular_projection_map(shape, kernel_size, dt)
        m = convert_spherical_to_image(m, m.shape[:2])
    else:
        m = grid_projection_map(shape, kernel_size, dilation, dt)
    return m[::stride, ::stride]


def get_perspective_projection_map(shape, kernel_size, stride=1, dilation=1, dt=np.float32):
    """spherical_projections.py:33-35."""
    return perspective_projection_map(shape, kernel_size, dilation, dt)[::stride, ::stride]


# ------------------------------------------------------------------ cube maps
def convert_3d_to_spherical(xyz):
    """conversions.py:20-31."""
    x, y, z = xyz[..., 0], xyz[..., 1], xyz[..., 2]
    lat = np.arctan2(-y, np.sqrt(x ** 2 + z ** 2))
    lon = np.arctan2(x, z)
    return np.stack((lon, lat), -1)


def convert_spherical_to_3d(lonlat):
    """conversions.py:34-42."""
    x = np.cos(lonlat[..., 1]) * np.sin(lonlat[..., 0])
    y = -np.sin(lonlat[..., 1])
    z = np.cos(lonlat[..., 1]) * np.cos(lonlat[..., 0])
    return np.stack((x, y, z), -1)


def convert_3d_to_cube(xyz, cube_dim):
    """conversions.py:45-116 (same case order as include/core/conversions.h:69-141; a later
    case overrides an earlier one where both hold).  Returns uv in [0, cube_dim], index."""
    dt = xyz.dtype.type
    x, y, z = xyz[..., 0], xyz[..., 1], xyz[..., 2]
    ax, ay, az = np.abs(x), np.abs(y), np.abs(z)
    xp, yp, zp = x > 0, y > 0, z > 0
    u = np.zeros(x.shape, dt)
    v = np.zeros(x.shape, dt)
    index = np.zeros(x.shape, np.int64)
    cases = [
        (xp & (ax >= ay) & (ax >= az), -z, -y, ax, 3),
        (~xp & (ax >= ay) & (ax >= az), z, -y, ax, 1),
        (yp & (ay >= ax) & (ay >= az), x, z, ay, 4),
        (~yp & (ay >= ax) & (ay >= az), x, -z, ay, 5),
        (zp & (az >= ax) & (az >= ay), x, -y, az, 2),
        (~zp & (az >= ax) & (az >= ay), -x, -y, az, 0),
    ]
    with np.errstate(invalid="ignore", divide="ignore"):
        for mask, uc, vc, m, face in cases:
            u = np.where(mask, dt(0.5) * (uc / m + dt(1)), u)
            v = np.where(mask, dt(0.5) * (vc / m + dt(1)), v)
            index = np.where(mask, face, index)
    return np.stack((u, v), -1).astype(dt) * dt(cube_dim), index


def convert_cube_to_3d(uv, index, cube_dim, dt=np.float32):
    """conversions.py:126-181: pixel (u, v) of face `index`, centres at +0.5."""
    uv = (uv.astype(dt) + dt(0.5)) / dt(cube_dim)
    uv = dt(2) * uv - dt(1)
    u, v = uv[..., 0], uv[..., 1]
    one = np.ones_like(u)
    table = {3: (one, -v, -u), 1: (-one, -v, u), 4: (u, one, v), 5: (u, -one, -v),
             2: (u, -v, one), 0: (-u, -v, -one)}
    xyz = np.zeros(u.shape + (3,), dt)
    for face, comps in table.items():
        for a in range(3):
            xyz[..., a] = np.where(index == face, comps[a], xyz[..., a])
    return xyz


def get_reverse_cube_projection_map(cube_dim, kernel_size, stride=1, dt=np.float32):
    """spherical_projections.py:26-30 with :261-311 and grids.py:23-45."""
    H, W = cube_dim, 6 * cube_dim
    v = np.broadcast_to(np.arange(cube_dim).reshape(-1, 1), (H, W))
    u = np.tile(np.broadcast_to(np.arange(cube_dim).reshape(1, -1), (H, cube_dim)), (1, 6))
    idx = np.repeat(np.arange(6), cube_dim).reshape(1, W) + np.zeros((H, 1), np.int64)
    res = math.pi / (2 * cube_dim)
    uv = np.stack((u, v), -1).astype(dt)
    lonlat = convert_3d_to_spherical(convert_cube_to_3d(uv, idx, cube_dim, dt)).astype(dt)
    ci, cj = _kernel_offsets(kernel_size)
    dx = (cj * res).astype(dt).reshape(1, 1, -1)
    dy = (ci * res).astype(dt).reshape(1, 1, -1)
    out_lat = lonlat[..., 1].reshape(H, W, 1) + dy
    out_lon = lonlat[..., 0].reshape(H, W, 1) + dx
    spherical = np.stack((out_lon, out_lat), -1).astype(dt)
    uv2, idx2 = convert_3d_to_cube(convert_spherical_to_3d(spherical).astype(dt), cube_dim)
    x = idx2.astype(dt) * dt(cube_dim) + uv2[..., 0]
    y = uv2[..., 1]
    return np.stack((x, y), -1).astype(dt)[::stride, ::stride]


# ------------------------------------------------------------------ cube2rect
def cube2rect_coordinates(cube_dim, rect_height, rect_width, dt=np.float32):
    """Face index and face coordinates (u, v) in [0, cube_dim - 1] of every pixel of the
    equirectangular image: include/util/cuda/cube2rect.cuh:27-45 with
    include/core/conversions.h:20-38 (differences in the data type, products and quotients
    in double, result rounded to the data type)."""
    xr = np.arange(rect_width).astype(dt)
    yr = np.arange(rect_height).astype(dt)
    with np.errstate(invalid="ignore", divide="ignore"):
        lon = (2 * math.pi * (xr - dt(rect_width) / dt(2)).astype(np.float64)
               / np.float64(dt(rect_width))).astype(dt).reshape(1, -1)
        lat = (math.pi * (yr - (dt(rect_height) - dt(1)) / dt(2)).astype(np.float64)
               / np.float64(dt(rect_height) - dt(1))).astype(dt).reshape(-1, 1)
    x = (np.cos(lat) * np.sin(lon)).astype(dt)
    y = (-np.sin(lat) + 0 * lon).astype(dt)
    z = (np.cos(lat) * np.cos(lon)).astype(dt)
    uv, face = convert_3d_to_cube(np.stack((x, y, z), -1), 1)
    uv = (uv * dt(cube_dim - 1)).astype(dt)
    return face, uv[..., 0], uv[..., 1]


def cube2rect(cubemap, rect_height, rect_width, interpolation):
    """include/util/cuda/cube2rect.cuh:16-64: the face is sampled inside the
    dim x 6*dim image from the face's first column on, with the nearest / bilinear
    interpolators of include/core/interpolation.h:85-160 (height dim, width 6*dim); a
    neighbour past the end of the buffer counts as zero (its weight is zero)."""
    dt = cubemap.dtype.type
    C, dim, width = cubemap.shape
    face, u, v = cube2rect_coordinates(dim, rect_height, rect_width, dt)
    flat = cubemap.reshape(C, -1)
    total = C * dim * width
    start = face * dim

    def fetch(xi, yi):
        ok = (xi >= 0) & (xi <= width - 1) & (yi >= 0) & (yi <= dim - 1)
        off = np.where(ok, start + yi * width + xi, 0)
        out = np.zeros((C,) + off.shape, dt)
        for c in range(C):
            inside = ok & (c * dim * width + off < total)
            idx = np.where(inside, off, 0)
            src = np.concatenate((flat[c], flat[c + 1][:1] if c + 1 < C else np.zeros(1, dt)))
            out[c] = np.where(inside, src[np.minimum(idx, dim * width)], dt(0))
        return out

    if interpolation == 1:
        x1f, y1f = np.floor(u), np.floor(v)
        x1, y1 = x1f.astype(np.int64), y1f.astype(np.int64)
        x2, y2 = x1 + 1, y1 + 1
        A = (y2.astype(dt) - v).astype(dt)
        B = (x2.astype(dt) - u).astype(dt)
        Cw = (u - x1f).astype(dt)
        D = (v - y1f).astype(dt)
        return ((A * B) * fetch(x1, y1) + (A * Cw) * fetch(x2, y1) + (D * B) * fetch(x1, y2)
                + (D * Cw) * fetch(x2, y2)).astype(dt)
    # llround(double(.)): halves away from zero
    rnd = lambda t: (np.sign(t) * np.floor(np.abs(t.astype(np.float64)) + 0.5)).astype(np.int64)
    return fetch(rnd(u), rnd(v))
