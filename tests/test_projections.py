"""Sample-map builders and cube2rect.

CPU part: the numpy restatement (oracle/projections.py) against what the mathematics
fixes -- the reference has no test or fixture for these functions.  GPU part: the HIP
builders against the restatement.

Bars.  Maps: the device evaluates each entry in double and rounds once, so it matches the
float64 restatement within 2 float32 ulps; against the float32 restatement (the reference's
own arithmetic) it stays within that arithmetic's rounding error: 2e-3 pixel away from the
two rows next to each pole, 0.1 pixel anywhere.  x is compared on the circle (x = 0 and
x = W are the same longitude).  cube2rect: 1e-5 relative (float32 bilinear), 1e-12
(float64); nearest is exact except where an ulp of difference in sin/cos moves a sample
across a pixel boundary (fewer than 0.5 % of the pixels in float32).
"""
import math

import numpy as np
import pytest
import torch

from oracle import projections as P


def _circ(a, b, period):
    d = np.abs(a - b) % period
    return np.minimum(d, period - d)


# ------------------------------------------------------------------ CPU: the restatement
@pytest.mark.parametrize("shape,ks", [((33, 64), (3, 3)), ((16, 40), (5, 3))])
def test_gnomonic_is_inverted_by_the_forward_projection(shape, ks):
    """Forward gnomonic projection about (lon0, lat0) (Snyder 22-3..22-5) of every mapped
    point returns the tap's tangent-plane offset (cj * res_lon, ci * res_lat)."""
    H, W = shape
    m = P.reverse_gnomonic_projection_map(shape, ks, np.float64)
    lat0, lon0, res_lat, res_lon = P.equirectangular_meshgrid(shape, np.float64)
    ci, cj = P._kernel_offsets(ks)
    lon, lat = m[..., 0], m[..., 1]
    cosc = np.sin(lat0) * np.sin(lat) + np.cos(lat0) * np.cos(lat) * np.cos(lon - lon0)
    X = np.cos(lat) * np.sin(lon - lon0) / cosc
    Y = (np.cos(lat0) * np.sin(lat) - np.sin(lat0) * np.cos(lat) * np.cos(lon - lon0)) / cosc
    rows = slice(1, H - 1)  # at the poles themselves longitude is degenerate
    assert np.abs(X - cj * res_lon)[rows].max() < 1e-9
    assert np.abs(Y - ci * res_lat)[rows].max() < 1e-9
    centre = ks[0] * ks[1] // 2
    assert np.array_equal(lat[..., centre], np.broadcast_to(lat0[..., 0], (H, W)))
    assert np.abs(lon).max() <= math.pi


def test_equirectangular_map_closed_form():
    """Pixel coordinates of tap (ci, cj) at pixel (i, j): row i - ci (latitude decreases
    with the row), column j + cj / cos(latitude of that row), modulo the width."""
    shape, ks = (21, 48), (3, 5)
    H, W = shape
    m = P.get_projection_map(shape, ks, "equirectangular", dt=np.float64)
    ci, cj = P._kernel_offsets(ks)
    i = np.arange(H).reshape(H, 1, 1)
    j = np.arange(W).reshape(1, W, 1)
    row = i - ci + 0 * j
    lat = math.pi / 2 - row * math.pi / (H - 1)
    assert np.abs(m[..., 1] - row).max() < 1e-9
    ok = np.abs(np.cos(lat)) > 1e-6  # the formula divides by cos at the poles
    col = (j + cj / np.cos(np.where(ok, lat, 0.3))) % W
    assert _circ(m[..., 0], col, W)[ok].max() < 1e-7


def test_grid_and_perspective_closed_forms():
    shape, ks = (9, 12), (3, 3)
    H, W = shape
    ci, cj = P._kernel_offsets(ks)
    g = P.get_projection_map(shape, ks, "grid", dilation=2, dt=np.float64)
    lat = math.pi / 2 - np.arange(H).reshape(H, 1, 1) * math.pi / (H - 1)
    lon = -math.pi + np.arange(W).reshape(1, W, 1) * 2 * math.pi / W
    assert np.abs(g[..., 0] - (lon + 2 * cj * 2 * math.pi / W)).max() < 1e-12
    assert np.abs(g[..., 1] - (lat + 2 * ci * math.pi / (H - 1))).max() < 1e-12
    p = P.get_perspective_projection_map(shape, ks, stride=2, dilation=3)
    assert p.shape == (5, 6, 9, 2) and p.dtype == np.float32
    assert np.array_equal(p[1, 2, :, 0], 4 + 3 * cj) and np.array_equal(p[1, 2, :, 1], 2 + 3 * ci)
    assert P.get_projection_map(shape, ks, "gnomonic", stride=4).shape == (3, 3, 9, 2)


@pytest.mark.parametrize("proj", ["gnomonic", "equirectangular"])
def test_float32_chain_stays_close_to_float64(proj):
    shape, ks = (64, 128), (3, 3)
    a = P.get_projection_map(shape, ks, proj, dt=np.float32).astype(np.float64)
    b = P.get_projection_map(shape, ks, proj, dt=np.float64)
    dx, dy = _circ(a[..., 0], b[..., 0], shape[1]), np.abs(a[..., 1] - b[..., 1])
    assert max(dx[2:-2].max(), dy[2:-2].max()) < 2e-3


def test_cube_conversions_are_consistent():
    """conversions.py's two independent functions invert each other, and known directions
    land where the face order [-z, -x, +z, +x, +y, -y] says."""
    dim = 7
    v, u = np.meshgrid(np.arange(dim), np.arange(dim), indexing="ij")
    for face in range(6):
        uv = np.stack((u, v), -1).astype(np.float64)
        idx = np.full(u.shape, face)
        uv2, idx2 = P.convert_3d_to_cube(P.convert_cube_to_3d(uv, idx, dim, np.float64), dim)
        assert np.array_equal(idx2, idx)
        assert np.abs(uv2 - (uv + 0.5)).max() < 1e-12
    dirs = {(0, 0, 1): 2, (1, 0, 0): 3, (-1, 0, 0): 1, (0, 0, -1): 0, (0, 1, 0): 4, (0, -1, 0): 5}
    for d, face in dirs.items():
        uv, idx = P.convert_3d_to_cube(np.array([d], np.float64), 1)
        assert idx[0] == face and np.allclose(uv[0], 0.5)
    # orientation inside the +z face: u grows with x, v grows with -y
    uv, _ = P.convert_3d_to_cube(np.array([[0.5, 0, 1], [0, -0.5, 1]], np.float64), 1)
    assert np.allclose(uv, [[0.75, 0.5], [0.5, 0.75]])
    # spherical conventions: lon from +z towards +x, lat towards -y
    ll = P.convert_3d_to_spherical(np.array([[0, 0, 1], [1, 0, 0], [0, -1, 0]], np.float64))
    assert np.allclose(ll, [[0, 0], [math.pi / 2, 0], [0, math.pi / 2]])
    rng = np.random.default_rng(0)
    ll = np.stack((rng.uniform(-3, 3, 100), rng.uniform(-1.5, 1.5, 100)), -1)
    assert np.allclose(P.convert_3d_to_spherical(P.convert_spherical_to_3d(ll)), ll)


def _cube_direction(xy, dim):
    """Unit direction of cube-map image coordinates (x = face * dim + u, y = v, with u, v in
    face units [0, dim]), through conversions.py:126-181 (pixel centres at +0.5)."""
    face = np.clip(np.floor(xy[..., 0] / dim), 0, 5).astype(np.int64)
    uv = np.stack((xy[..., 0] - face * dim, xy[..., 1]), -1) - 0.5
    d = P.convert_cube_to_3d(uv, face, dim, np.float64)
    return d / np.linalg.norm(d, axis=-1, keepdims=True)


def test_cube_projection_map_moves_by_the_tap_offset_on_the_sphere():
    dim, ks = 6, (3, 3)
    m = P.get_reverse_cube_projection_map(dim, ks, dt=np.float64)
    ci, cj = P._kernel_offsets(ks)
    centre = ks[0] * ks[1] // 2
    jj, ii = np.meshgrid(np.arange(6 * dim), np.arange(dim))
    assert np.abs(m[..., centre, 0] - (jj + 0.5)).max() < 1e-9
    assert np.abs(m[..., centre, 1] - (ii + 0.5)).max() < 1e-9
    ll0 = P.convert_3d_to_spherical(_cube_direction(m[..., centre, :], dim))
    res = math.pi / (2 * dim)
    want = np.stack((ll0[..., None, 0] + cj * res, ll0[..., None, 1] + ci * res), -1)
    got = _cube_direction(m, dim)
    # x = face * dim + u cannot tell the right edge of a face (u = dim) from the left edge
    # of the next: leave out the entries that sit exactly on one
    inner = (m[..., 0] % dim != 0)[..., None]
    assert np.abs(np.where(inner, got - P.convert_spherical_to_3d(want), 0)).max() < 1e-9
    assert inner.mean() > 0.99


def _linear_cubemap(C, dim, dt):
    """cubemap[c, y, x] = a_c * x + b_c * y + c_c over the dim x 6*dim image."""
    y, x = np.meshgrid(np.arange(dim), np.arange(6 * dim), indexing="ij")
    coef = np.array([[1.0, 0.0, 0.0], [0.0, 1.0, 0.0], [0.25, -0.5, 3.0]])[:C]
    return np.stack([a * x + b * y + c for a, b, c in coef]).astype(dt), coef


def test_cube2rect_reproduces_linear_functions_and_faces():
    dim, RH, RW = 9, 17, 32
    cube, coef = _linear_cubemap(3, dim, np.float64)
    face, u, v = P.cube2rect_coordinates(dim, RH, RW, np.float64)
    out = P.cube2rect(cube, RH, RW, 1)
    for c, (a, b, c0) in enumerate(coef):
        assert np.abs(out[c] - (a * (face * dim + u) + b * v + c0)).max() < 1e-9
    near = P.cube2rect(cube, RH, RW, 0)
    rnd = lambda t: np.floor(t + 0.5)
    assert np.array_equal(near[0], face * dim + rnd(u)) and np.array_equal(near[1], rnd(v))
    # geometry: image centre looks at +z, its left edge at -z, quarter points at -x / +x,
    # first row (lat = -pi/2, y = +1) at the +y face, last row at the -y face
    mid = RH // 2
    assert face[mid, RW // 2] == 2 and face[mid, 0] == 0
    assert face[mid, RW // 4] == 1 and face[mid, 3 * RW // 4] == 3
    assert (face[0] == 4).all() and (face[-1] == 5).all()
    assert abs(u[mid, RW // 2] - (dim - 1) / 2) < 1e-9 and abs(v[mid, RW // 2] - (dim - 1) / 2) < 1e-9
    # the face coordinates point back at the pixel's direction
    lon = 2 * math.pi * (np.arange(RW) - RW / 2) / RW
    lat = math.pi * (np.arange(RH) - (RH - 1) / 2) / (RH - 1)
    want = P.convert_spherical_to_3d(np.stack(np.broadcast_arrays(lon[None], lat[:, None]), -1))
    uv = np.stack((u, v), -1) / (dim - 1) * dim - 0.5  # to conversions.py's pixel-centre units
    got = P.convert_cube_to_3d(uv, face, dim, np.float64)
    got /= np.linalg.norm(got, axis=-1, keepdims=True)
    assert np.abs(got - want).max() < 1e-9


def test_abi_exports_projection_symbols():
    from mappedconvolutions_amd import _lib
    lib = _lib.load()
    for name in ("mcx_projection_map", "mcx_cube_projection_map", "mcx_cube2rect"):
        assert hasattr(lib, name)


# ------------------------------------------------------------------ GPU: parity
def _ulps32(ref64):
    return 2 * np.spacing(np.maximum(np.abs(ref64), 1e-3).astype(np.float32)).astype(np.float64)


@pytest.mark.gpu
@pytest.mark.parametrize("proj", ["gnomonic", "equirectangular", "grid"])
@pytest.mark.parametrize("shape,ks,stride,dilation", [
    ((64, 128), (3, 3), 1, 1), ((33, 50), (5, 3), 2, 2), ((16, 24), (2, 2), 3, 1),
    ((40, 64), (1, 1), 1, 1)])
def test_projection_map_matches_restatement(proj, shape, ks, stride, dilation, device):
    from mappedconvolutions_amd.util import get_projection_map
    got = get_projection_map(shape, ks, proj, stride, dilation, device=device)
    assert got.dtype == torch.float32 and got.is_cuda
    got = got.cpu().numpy().astype(np.float64)
    ref = P.get_projection_map(shape, ks, proj, stride, dilation, dt=np.float64)
    assert got.shape == ref.shape
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)  # even kernels: 0/0 taps, as in the reference
    # (such a tap's longitude is atan2(0, +-0): 0 or pi by the sign of a zero)
    nan = nan | nan.any(-1, keepdims=True)
    if proj == "equirectangular":
        # taps that land on a pole divide by cos(+-pi/2) ~ 6e-17: their longitude is noise
        # of the order 1e16 folded back onto the circle, in the reference as here
        ci, cj = P._kernel_offsets(ks)
        rows = np.arange(0, shape[0], stride).reshape(-1, 1, 1) - ci
        lat = math.pi / 2 - rows * math.pi / (shape[0] - 1)
        nan = nan | ((np.abs(np.cos(lat)) < 1e-9) & (cj != 0))[..., None]
    got, ref = np.where(nan, 0, got), np.where(nan, 0, ref)
    period = shape[1] if proj != "grid" else 1e30
    tol = _ulps32(ref)
    assert (_circ(got[..., 0], ref[..., 0], period) <= tol[..., 0]).all()
    assert (np.abs(got[..., 1] - ref[..., 1]) <= tol[..., 1]).all()
    # the reference's own float32 arithmetic
    r32 = np.where(nan, 0, P.get_projection_map(shape, ks, proj, stride, dilation, dt=np.float32))
    d = np.maximum(_circ(got[..., 0], r32[..., 0], period), np.abs(got[..., 1] - r32[..., 1]))
    assert d.max() < 0.1
    if stride == 1:
        assert d[2:-2].max() < 2e-3


@pytest.mark.gpu
def test_perspective_map_is_exact(device):
    from mappedconvolutions_amd.util import get_perspective_projection_map
    got = get_perspective_projection_map((37, 53), (3, 5), stride=2, dilation=3, device=device)
    ref = P.get_perspective_projection_map((37, 53), (3, 5), stride=2, dilation=3)
    assert np.array_equal(got.cpu().numpy(), ref)


@pytest.mark.gpu
@pytest.mark.parametrize("dim,ks,stride", [(8, (3, 3), 1), (13, (3, 5), 2)])
def test_cube_projection_map_matches_restatement(dim, ks, stride, device):
    from mappedconvolutions_amd.util import get_reverse_cube_projection_map
    got = get_reverse_cube_projection_map(dim, ks, stride, device=device).cpu().numpy()
    ref = P.get_reverse_cube_projection_map(dim, ks, stride, dt=np.float64)
    assert got.shape == ref.shape and got.dtype == np.float32
    got = got.astype(np.float64)
    close = (np.abs(got - ref) <= _ulps32(ref)).all(-1)
    assert close.mean() > 0.999
    # a direction on a cube edge may be put on either face: same point of the sphere
    rest = ~close & (ref[..., 0] % dim != 0) & (got[..., 0] % dim != 0)
    assert np.abs(_cube_direction(got, dim) - _cube_direction(ref, dim))[rest].max(initial=0) < 1e-5


def _smooth_cubemap(C, dim, dt):
    """Values of smooth functions of the direction, sampled where cube2rect places the pixels
    (pixel 0 and pixel dim-1 on the face edges), so that neighbouring faces agree on edges."""
    v, u = np.meshgrid(np.arange(dim), np.arange(dim), indexing="ij")
    planes = []
    for face in range(6):
        uv = np.stack((u, v), -1) / max(dim - 1, 1) * dim - 0.5
        d = P.convert_cube_to_3d(uv, np.full(u.shape, face), dim, np.float64)
        d /= np.linalg.norm(d, axis=-1, keepdims=True)
        planes.append(np.stack([d[..., 0] + 2 * d[..., 1] * d[..., 2], np.sin(3 * d[..., 1]) - d[..., 2],
                                d[..., 0] * d[..., 0] + 0.5][:C]))
    return np.ascontiguousarray(np.concatenate(planes, -1).astype(dt))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("interpolation", ["nearest", "bilinear"])
def test_cube2rect_matches_restatement(dt, interpolation, device):
    from mappedconvolutions_amd.util import cube_to_rect
    dim, RH, RW = 24, 61, 128
    cube = _smooth_cubemap(3, dim, dt)
    got = cube_to_rect(torch.from_numpy(cube).to(device), RH, RW, interpolation).cpu().numpy()
    ref = P.cube2rect(cube, RH, RW, 1 if interpolation == "bilinear" else 0)
    assert got.shape == ref.shape and got.dtype == ref.dtype
    scale = np.abs(ref).max()
    if interpolation == "bilinear":
        assert np.abs(got - ref).max() <= (1e-5 if dt == np.float32 else 1e-12) * scale
    else:
        assert (got != ref).mean() < (5e-3 if dt == np.float32 else 1e-4)
        assert np.abs(got - ref).max() < 0.3 * scale  # a moved sample is a neighbouring pixel


@pytest.mark.gpu
def test_cube2rect_linear_cubemap_and_last_face_corner(device):
    """Exact-arithmetic case: a cube map linear in the image coordinates comes back as that
    function of the face coordinates; the last pixel of the last face of the last channel
    (whose right-hand neighbour lies past the buffer) is handled."""
    from mappedconvolutions_amd.util import cube_to_rect
    dim, RH, RW = 9, 17, 32
    cube, coef = _linear_cubemap(3, dim, np.float64)
    got = cube_to_rect(torch.from_numpy(cube).to(device), RH, RW, "bilinear").cpu().numpy()
    face, u, v = P.cube2rect_coordinates(dim, RH, RW, np.float64)
    for c, (a, b, c0) in enumerate(coef):
        assert np.abs(got[c] - (a * (face * dim + u) + b * v + c0)).max() < 1e-9
    assert np.abs(got - P.cube2rect(cube, RH, RW, 1)).max() < 1e-12


@pytest.mark.gpu
def test_device_built_map_feeds_the_convolution(device):
    """A gnomonic map built on the device drives the mapped convolution (bispherical) and
    gives what the CPU oracle gives with the same map."""
    from mappedconvolutions_amd import _C
    from mappedconvolutions_amd.util import get_projection_map
    from oracle import ops as O
    g = torch.Generator().manual_seed(11)
    H, W, C = 24, 48, 8
    smap = get_projection_map((H, W), (3, 3), "gnomonic", device=device)
    x = torch.randn(2, C, H, W, generator=g)
    w, b = torch.randn(C, C, 9, generator=g) / 8, torch.randn(C, generator=g)
    y = _C.mapped_conv_forward(x.to(device), smap, w.to(device), b.to(device), 9, 2)
    y_o = O.mapped_conv_forward(x, smap.cpu(), w, b, 9, 2)
    assert ((y.cpu() - y_o).abs().max() / y_o.abs().max()).item() < 1e-5


@pytest.mark.gpu
def test_projection_argument_errors(device):
    from mappedconvolutions_amd.util import get_projection_map, cube_to_rect
    with pytest.raises(RuntimeError):
        get_projection_map((1, 16), (3, 3), "gnomonic", device=device)  # divides by H - 1
    with pytest.raises(RuntimeError):
        cube_to_rect(torch.zeros(2, 4, 20, device=device), 8, 16)
    with pytest.raises(RuntimeError):
        cube_to_rect(torch.zeros(2, 4, 24), 8, 16)  # CPU tensor
