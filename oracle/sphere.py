"""TEST INFRASTRUCTURE: numpy restatement of the reference's planar-convolution operator on a
triangle mesh of the sphere (package/ext_modules/src/util/cpp/sphere.cpp): the per-face test
Sphere::_isPointInFace (:1055-1105), the face normal (:466-484), SphericalToXYZ
(include/core/conversions.h:21-26), maxOfThreeValues (:1108-1113) and the output order of
getPlanarConvolutionOperatorFromSamples (:1117-1270).  float32 arithmetic in the reference's
order of operations.  The mesh is passed in (vertices [V, 3], faces [F, 3]); the reference
builds its own icosphere and narrows the search by a breadth-first walk, which decides only
WHICH of several passing faces is returned for a sample within the test's tolerance of an
edge - `planar_conv_operator` returns the one the sample lies deepest inside (lowest index on
ties) and also the full table of passing faces, so a checker can accept any of them.

Pinned by tests/test_sphere.py: against the reference's own build (oracle/_ref/_sphere.so) on
its own icospheres of order 0-3, against the fixture written from that build, and by
mathematics (weights sum to 1, reconstruct the pierced point, a vertex gets weight 1)."""
import numpy as np

F32 = np.float32


def _dot(a, b):
    return a[..., 0] * b[..., 0] + a[..., 1] * b[..., 1] + a[..., 2] * b[..., 2]


def _cross(a, b):
    return np.stack([a[..., 1] * b[..., 2] - a[..., 2] * b[..., 1],
                     a[..., 2] * b[..., 0] - a[..., 0] * b[..., 2],
                     a[..., 0] * b[..., 1] - a[..., 1] * b[..., 0]], -1)


def _normalized(a):
    return a / np.sqrt(_dot(a, a))[..., None]


def spherical_to_xyz(lon, lat):
    lon, lat = lon.astype(F32), lat.astype(F32)
    return np.stack([np.cos(lat) * np.sin(lon), -np.sin(lat), np.cos(lat) * np.cos(lon)], -1)


def barycentric_table(points, vertices, faces):
    """(s, t, u, inside) [N, F] of every point against every face, as _isPointInFace."""
    pt = points.astype(F32)[:, None, :]
    A = vertices.astype(F32)[faces[:, 0]][None]
    B = vertices.astype(F32)[faces[:, 1]][None]
    C = vertices.astype(F32)[faces[:, 2]][None]
    with np.errstate(divide="ignore", invalid="ignore"):
        normal = _normalized(_cross(C - B, A - B))
        d = -_dot(normal, A)
        ray = _normalized(pt)
        denom = _dot(normal, ray)
        dist_o = _dot(normal, pt) + d
        proj_o = pt - normal * dist_o[..., None]
        dist_r = _dot(A, normal) / denom
        proj_r = ray * dist_r[..., None]
        proj = np.where((denom < F32(1e-12))[..., None], proj_o, proj_r)
        BA, CA = B - A, C - A
        N = _cross(BA, CA)
        W = proj - A
        nn = _dot(N, N)
        s = _dot(_cross(BA, W), N) / nn
        t = _dot(_cross(W, CA), N) / nn
        u = F32(1) - s - t
        tol = F32(-1e-3)
        inside = (denom >= 0) & (s >= tol) & (t >= tol) & (u >= tol)
    return s, t, u, inside


def planar_conv_operator(samples, vertices, faces, nearest=False, chunk=512):
    """samples [N, 2] (lon, lat) -> face [N] int64, vertex indices [N, 3] int64 (the face's
    vertices in reverse order), weights [N, 3] float32 (s, t, u), passing [N, F] bool."""
    samples = np.asarray(samples, F32).reshape(-1, 2)
    vertices = np.asarray(vertices, F32)
    faces = np.asarray(faces, np.int64)
    n = samples.shape[0]
    face = np.full(n, -1, np.int64)
    vidx = np.full((n, 3), -1, np.int64)
    w = np.zeros((n, 3), F32)
    passing = np.zeros((n, faces.shape[0]), bool)
    for i0 in range(0, n, chunk):
        sl = slice(i0, min(n, i0 + chunk))
        pts = spherical_to_xyz(samples[sl, 0], samples[sl, 1])
        s, t, u, inside = barycentric_table(pts, vertices, faces)
        depth = np.where(inside, np.minimum(s, np.minimum(t, u)), F32(-np.inf))
        best = depth.argmax(1)  # first maximum: the lower index on ties
        found = inside.any(1)
        rows = np.arange(best.shape[0])
        face[sl] = np.where(found, best, -1)
        vidx[sl] = np.where(found[:, None], faces[best][:, ::-1], -1)
        stu = np.stack([s[rows, best], t[rows, best], u[rows, best]], -1)
        if nearest:
            m = np.zeros(best.shape[0], np.int64)
            m[(stu[:, 1] > stu[:, 0]) & (stu[:, 1] > stu[:, 2])] = 1
            m[(stu[:, 2] > stu[:, 0]) & (stu[:, 2] > stu[:, 1])] = 2
            stu = np.eye(3, dtype=F32)[m]
        w[sl] = np.where(found[:, None], stu, F32(0))
        passing[sl] = inside
    return face, vidx, w, passing


def gnomonic_kernel(spherical_coords, kh, kw, res_lat, res_lon, dt=np.float32):
    """package/layers/util/icosphere_functions.py:135-183: a kh x kw grid of spacing (res_lon,
    res_lat) on the plane tangent at every (lon, lat) of spherical_coords [V, 2], carried back
    onto the sphere; [1, V, kh*kw, 2] (lon in [-pi, pi), lat).  dt=float32 follows the
    reference's arithmetic, dt=float64 gives the formulas' value.  Pinned by mathematics in
    tests/test_sphere.py (the textbook forward gnomonic projection about the centre returns the
    grid; the reference holds no test or fixture for it): parity otherwise unpinned."""
    sc = np.asarray(spherical_coords, dtype=dt)
    lon = sc[..., 0].reshape(1, -1, 1)
    lat = sc[..., 1].reshape(1, -1, 1)
    x = np.zeros(kh * kw, dtype=dt)
    y = np.zeros(kh * kw, dtype=dt)
    for i in range(kh):
        for j in range(kw):
            x[i * kw + j] = dt(j - kw // 2) * dt(res_lon)
            y[i * kw + j] = dt(i - kh // 2) * dt(res_lat)
    x, y = x.reshape(1, 1, -1), y.reshape(1, 1, -1)
    with np.errstate(invalid="ignore", divide="ignore"):
        rho = np.sqrt(x ** 2 + y ** 2)
        nu = np.arctan(rho)
        out_lat = np.arcsin(np.cos(nu) * np.sin(lat) + y * np.sin(nu) * np.cos(lat) / rho)
        out_lon = lon + np.arctan2(x * np.sin(nu),
                                   rho * np.cos(lat) * np.cos(nu) - y * np.sin(lat) * np.sin(nu))
    centre = (kh // 2) * kw + kw // 2
    out_lat[..., centre] = lat[..., 0]
    out_lon[..., centre] = lon[..., 0]
    pi = dt(np.pi)
    out_lon = np.mod(out_lon + pi, dt(2) * pi) - pi
    return np.stack([out_lon, out_lat], -1).astype(dt)
