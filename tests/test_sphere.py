"""The planar-convolution operator on sphere meshes (reference:
package/ext_modules/src/util/cpp/sphere.cpp:1055-1270).

CPU part: the numpy oracle (oracle/sphere.py) against the fixture written from the reference's
own build, against that build directly where it is present (oracle/_ref/_sphere.so), and by
mathematics.  GPU part: the HIP kernel through the C ABI against the oracle and the fixture.

A sample within the face test's tolerance (1e-3 in barycentric units) of an edge passes the
test of both faces; the reference returns whichever its breadth-first walk meets first.  Such
samples are compared through what is fixed: the returned face must pass the test, and the
weighted sum of its vertices must be the pierced point."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import reference, sphere as osph

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "icosphere_operator.json")) as fh:
    FIX = json.load(fh)
VERTS = np.array(FIX["vertices"], np.float32)
FACES = np.array(FIX["faces"], np.int64)
SAMPLES = np.array(FIX["samples"], np.float32)


def _decided():
    """Samples whose two largest barycentric weights differ by more than rounding: only there
    is the one-hot `nearest` output determined (edge midpoints sit exactly on the boundary)."""
    _, _, bary, _ = osph.planar_conv_operator(SAMPLES, VERTS, FACES, False)
    top2 = np.sort(bary, 1)[:, 1:]
    return (top2[:, 1] - top2[:, 0]) > 1e-4


def _check_against(face, vidx, w, want, passing, nearest, tol=2e-6):
    """`face`, `vidx`, `w`: what is being tested; `want`: the reference's answer."""
    wf = np.array(want["face"])
    wv = np.array(want["vertex_idx"])
    ww = np.array(want["weights"], np.float32)
    same = face == wf
    if nearest:
        same &= _decided()
    # the first 400 samples are random directions (well inside one face but for a few); the
    # rest sit on mesh vertices and edge midpoints, where five, six or two faces pass
    assert same[:400].mean() > 0.97, "random samples lie well inside one face"
    assert (vidx[same] == wv[same]).all()
    assert np.abs(w[same] - ww[same]).max() <= tol
    rows = np.arange(len(face))
    # where the faces differ, both must pass the reference's own face test
    assert passing[rows, wf].all(), "the reference's face passes the restated test"
    assert passing[rows, face].all()
    if not nearest:
        # and both describe the same point: sum of weights x vertices
        p_got = (w[..., None] * VERTS[vidx]).sum(1)
        p_ref = (ww[..., None] * VERTS[wv]).sum(1)
        assert np.abs(p_got - p_ref).max() < 2e-3   # within the edge tolerance
    else:
        picked = vidx[rows, w.argmax(1)]
        picked_ref = wv[rows, ww.argmax(1)]
        # away from the decision boundary the nearest vertex is the same one, whichever of the
        # passing faces was returned
        assert (picked == picked_ref)[_decided()].all()


@pytest.mark.parametrize("nearest", [False, True])
def test_oracle_matches_reference_fixture(nearest):
    face, vidx, w, passing = osph.planar_conv_operator(SAMPLES, VERTS, FACES, nearest)
    _check_against(face, vidx, w, FIX["nearest" if nearest else "barycentric"], passing, nearest)


def test_oracle_mathematics():
    face, vidx, w, passing = osph.planar_conv_operator(SAMPLES, VERTS, FACES, False)
    assert (face >= 0).all() and passing.any(1).all()
    np.testing.assert_allclose(w.sum(1), 1.0, atol=2e-6)
    assert (w >= -1e-3 - 1e-6).all()
    # the weighted vertices reconstruct the point where the ray pierces the face's plane
    pts = osph.spherical_to_xyz(SAMPLES[:, 0], SAMPLES[:, 1]).astype(np.float64)
    A, B, C = (VERTS[FACES[face, i]].astype(np.float64) for i in range(3))
    n = np.cross(B - A, C - A)
    hit = pts * ((A * n).sum(1) / (pts * n).sum(1))[:, None]
    recon = (w[..., None].astype(np.float64) * VERTS[vidx]).sum(1)
    assert np.abs(recon - hit).max() < 1e-5
    # a mesh vertex as the sample: weight 1 (within rounding) at that vertex
    nv = VERTS.shape[0]
    at_vertex = slice(400, 400 + nv)
    top = vidx[at_vertex][np.arange(nv), w[at_vertex].argmax(1)]
    assert (top == np.arange(nv)).all()
    assert w[at_vertex].max(1).min() > 1 - 1e-4
    # brute force in float64 over all faces agrees on well-inside samples
    deep = w.min(1) > 0.02
    s64 = SAMPLES[deep].astype(np.float64)
    p64 = np.stack([np.cos(s64[:, 1]) * np.sin(s64[:, 0]), -np.sin(s64[:, 1]),
                    np.cos(s64[:, 1]) * np.cos(s64[:, 0])], -1)
    V64 = VERTS.astype(np.float64)
    M = np.stack([V64[FACES[:, 0]], V64[FACES[:, 1]], V64[FACES[:, 2]]], -1)  # [F, 3, 3]
    coef = np.linalg.solve(M[None], p64[:, None, :, None])[..., 0]            # p = M @ coef
    inside = (coef > 0).all(-1)
    assert (inside.sum(1) == 1).all() and (inside.argmax(1) == face[deep]).all()
    bary = coef[np.arange(len(s64)), face[deep]]
    bary /= bary.sum(1, keepdims=True)
    np.testing.assert_allclose(w[deep][:, ::-1], bary, atol=1e-5)


@pytest.mark.skipif(not reference.available("_sphere"), reason="reference build absent")
@pytest.mark.parametrize("order", [0, 1, 3])
def test_oracle_matches_reference_build(order):
    S = reference.module("_sphere").Sphere
    mesh = S.generate_icosphere(0).loop_subdivision(order)
    verts, faces = mesh.get_vertices().numpy(), mesh.get_all_face_vertex_indices().numpy()
    rng = np.random.default_rng(order)
    n = 1500
    smp = np.stack([rng.uniform(-np.pi, np.pi, n), np.arcsin(rng.uniform(-1, 1, n))], -1)
    smp_t = torch.tensor(smp, dtype=torch.float32).view(1, n, 1, 2)
    for nearest in (False, True):
        f_r, v_r, w_r = S.get_planar_conv_operator_from_samples(smp_t, order, True, nearest)
        f_o, v_o, w_o, passing = osph.planar_conv_operator(smp_t.view(-1, 2).numpy(), verts,
                                                           faces, nearest)
        f_r, v_r, w_r = f_r.view(-1).numpy(), v_r.view(-1, 3).numpy(), w_r.view(-1, 3).numpy()
        same = f_r == f_o
        assert same.mean() > 0.98
        assert (v_r[same] == v_o[same]).all()
        assert np.abs(w_r[same] - w_o[same]).max() < 2e-6
        assert passing[np.arange(n), f_r].all()


def test_vertex_resolution_matches_the_reference_value():
    """Sphere::getVertexResolution of the fixture mesh, as the reference build reported it."""
    from mappedconvolutions_amd.util.icosphere_functions import vertex_resolution
    got = vertex_resolution(torch.tensor(VERTS), torch.tensor(FACES))
    assert abs(got - FIX["vertex_resolution"]) < 1e-5 * FIX["vertex_resolution"] + 1e-6


def test_alias_table_covers_the_reference_extension_modules():
    """Every `_mapped_convolution_ext.<module>` the reference's setup.py builds
    (package/setup.py:52-95) resolves after install_aliases(), and the ops of the hot path are
    this backend's."""
    import sys
    import mappedconvolutions_amd as mc
    mc.install_aliases(ext_only=True)
    built = ["_convolution", "_transposed_convolution", "_mapped_convolution",
             "_mapped_transposed_convolution", "_mapped_max_pooling", "_mapped_avg_pooling",
             "_resample", "_weighted_mapped_convolution",
             "_weighted_mapped_transposed_convolution", "_weighted_mapped_max_pooling",
             "_weighted_mapped_avg_pooling", "_weighted_resample", "_knn", "_cube2rect",
             "_sphere"]
    for name in built:
        assert "_mapped_convolution_ext." + name in sys.modules, name
    hot = {"_mapped_convolution": ["mapped_conv_forward", "mapped_conv_backward"],
           "_weighted_mapped_convolution": ["weighted_mapped_conv_forward",
                                            "weighted_mapped_conv_backward"],
           "_mapped_transposed_convolution": ["mapped_transposed_conv_forward",
                                              "mapped_transposed_conv_backward"],
           "_weighted_mapped_transposed_convolution": ["weighted_mapped_transposed_conv_forward",
                                                       "weighted_mapped_transposed_conv_backward"],
           "_mapped_max_pooling": ["mapped_max_pool", "mapped_max_unpool"],
           "_weighted_mapped_max_pooling": ["weighted_mapped_max_pool",
                                            "weighted_mapped_max_unpool"],
           "_mapped_avg_pooling": ["mapped_avg_pool", "mapped_avg_unpool"],
           "_weighted_mapped_avg_pooling": ["weighted_mapped_avg_pool",
                                            "weighted_mapped_avg_unpool"],
           "_resample": ["resample_to_map", "resample_from_map"],
           "_weighted_resample": ["weighted_resample_to_map", "weighted_resample_from_map"],
           "_knn": ["knn_forward"]}
    for mod, ops in hot.items():
        m = sys.modules["_mapped_convolution_ext." + mod]
        for op in ops:
            assert getattr(m, op) is getattr(mc._C, op)
    # the plain-convolution baselines are the library routine
    x, w, b = torch.randn(2, 3, 6, 7), torch.randn(4, 3, 3, 3), torch.randn(4)
    conv = sys.modules["_mapped_convolution_ext._convolution"]
    want = torch.nn.functional.conv2d(x, w, b, stride=1, padding=1)
    assert torch.allclose(conv.conv_forward(x, w, b, 3, 3, 1, 1, 1, 1, 1, 1), want)
    g = torch.randn_like(want)
    gx, gw, gb = conv.conv_backward(g, x, w, b, 3, 3, 1, 1, 1, 1, 1, 1)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = torch.autograd.grad(torch.nn.functional.conv2d(xr, wr, b, padding=1), (xr, wr), g)
    assert torch.allclose(gx, ref[0], atol=1e-5) and torch.allclose(gw, ref[1], atol=1e-4)
    assert torch.allclose(gb, g.sum((0, 2, 3)), atol=1e-5)
    with pytest.raises(RuntimeError, match="host-side"):
        sys.modules["_mapped_convolution_ext._sphere"].Sphere


# ------------------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("nearest", [False, True])
def test_gpu_operator_matches_oracle_and_fixture(nearest, device):
    from mappedconvolutions_amd import _C
    smp = torch.tensor(SAMPLES).view(1, -1, 1, 2).cuda()
    f, v, w = _C.planar_conv_operator_from_samples(smp, torch.tensor(VERTS).cuda(),
                                                   torch.tensor(FACES).cuda(), True, nearest)
    assert f.shape == (1, len(SAMPLES), 1) and v.shape == (1, len(SAMPLES), 1, 3)
    f, v, w = f.view(-1).cpu().numpy(), v.view(-1, 3).cpu().numpy(), w.view(-1, 3).cpu().numpy()
    f_o, v_o, w_o, passing = osph.planar_conv_operator(SAMPLES, VERTS, FACES, nearest)
    # same rule (deepest face, lowest index on ties), same float32 arithmetic: equal but for
    # samples whose two best faces are within rounding of each other
    same = f == f_o
    assert same[:400].mean() > 0.99 and same.mean() > 0.8
    assert (v[same] == v_o[same]).all()
    if nearest:
        # one-hot at the largest weight: compared where the two largest weights are apart by
        # more than rounding (edge midpoints sit exactly on that decision boundary)
        same &= _decided()
        assert same[:400].mean() > 0.98
    assert np.abs(w[same] - w_o[same]).max() < 2e-6
    assert passing[np.arange(len(f)), f].all()
    _check_against(f, v, w, FIX["nearest" if nearest else "barycentric"], passing, nearest)


@pytest.mark.gpu
def test_gpu_vertex_kernel_map_drives_a_mapped_convolution(device):
    """Order-5 mesh (10242 vertices, 20480 faces), 3x3 gnomonic kernel at every vertex: the
    maps are valid (weights sum to 1, indices inside, pierced point reconstructed), agree with
    the oracle on a subset, and feed the weighted mapped convolution."""
    from mappedconvolutions_amd import nn, util
    verts, faces = util.synthetic.subdivided_icosahedron(5)
    verts, faces = verts.numpy(), faces.numpy()
    vt, ft = torch.tensor(verts).cuda(), torch.tensor(faces).cuda()
    assert 0.03 < util.icosphere_functions.vertex_resolution(vt, ft) < 0.045
    idx, w = util.vertex_to_vertex_kernel_map(vt, ft, 3, 3)
    V = verts.shape[0]
    assert idx.shape == (1, V, 9, 3, 2) and w.shape == (1, V, 9, 3)
    assert (idx[..., 0] >= 0).all() and (idx[..., 0] < V).all() and (idx[..., 1] == 0).all()
    torch.testing.assert_close(w.sum(-1), torch.ones_like(w[..., 0]), atol=1e-5, rtol=0)
    assert w.min() > -1.1e-3
    # the centre tap is the vertex itself
    centre = idx[0, :, 4, :, 0].long()
    top = centre.gather(1, w[0, :, 4].argmax(1, keepdim=True))[:, 0]
    assert (top.cpu() == torch.arange(V)).all()
    # oracle on a subset of vertices
    spherical = util.convert_3d_to_spherical(vt)
    res = util.icosphere_functions.vertex_resolution(vt, ft)
    samples = util.gnomonic_kernel(spherical, 3, 3, res, res)
    pick = torch.arange(0, V, 41)
    sub = samples[0, pick.cuda()].reshape(-1, 2).cpu().numpy()
    f_o, v_o, w_o, passing = osph.planar_conv_operator(sub, verts, faces, False)
    got_v = idx[0, pick.cuda(), :, :, 0].reshape(-1, 3).long().cpu().numpy()
    got_w = w[0, pick.cuda()].reshape(-1, 3).cpu().numpy()
    same = (got_v == v_o).all(1)
    assert same.mean() > 0.8        # centre taps sit on vertices: five or six faces tie
    # (a barycentric weight is a position divided by the edge length, 0.04 here: one ulp of
    # the device's and numpy's sin / cos of the sample direction shows as up to 1e-5)
    assert np.abs(got_w[same] - w_o[same]).max() < 1e-4
    recon = (got_w[..., None] * verts[got_v]).sum(1)
    recon_o = (w_o[..., None] * verts[v_o]).sum(1)
    assert np.abs(recon - recon_o).max() < 1e-4
    # and a convolution over the mesh signal runs on them
    layer = nn.MappedConvolution(8, 16, 9, interpolation='nearest').cuda()
    x = torch.randn(2, 8, 1, V, device=device)
    y = layer(x, idx, w)
    assert y.shape == (2, 16, 1, V) and torch.isfinite(y).all()
    # constant signal, unit-sum weights: every tap samples 1, so y = sum of weights + bias
    ones = torch.ones(1, 8, 1, V, device=device)
    want = layer.weight.sum((1, 2)) + layer.bias
    torch.testing.assert_close(layer(ones, idx, w)[0, :, 0].mean(1), want, atol=1e-4, rtol=1e-4)


def _forward_gnomonic(lon, lat, lon0, lat0):
    """Textbook gnomonic projection about (lon0, lat0): plane coordinates of (lon, lat)."""
    cosc = np.sin(lat0) * np.sin(lat) + np.cos(lat0) * np.cos(lat) * np.cos(lon - lon0)
    x = np.cos(lat) * np.sin(lon - lon0) / cosc
    y = (np.cos(lat0) * np.sin(lat) - np.sin(lat0) * np.cos(lat) * np.cos(lon - lon0)) / cosc
    return x, y


def _gnomonic_case():
    g = np.random.default_rng(21)
    centres = np.stack([g.uniform(-np.pi, np.pi, 200), g.uniform(-1.45, 1.45, 200)], -1)
    centres[:4] = [[3.1, 0.2], [-3.1, -0.2], [0.0, 1.5], [1.0, -1.5]]  # seam and near the poles
    return centres.astype(np.float32), 3, 5, 0.031, 0.047


def test_oracle_gnomonic_kernel_mathematics():
    """The mesh kernels' sample locations: projected forward about their centre they are the
    regular grid (j - kw/2) * res_lon, (i - kh/2) * res_lat; the centre tap is the centre;
    longitudes lie in [-pi, pi); float32 stays within its rounding of float64."""
    centres, kh, kw, rlat, rlon = _gnomonic_case()
    s64 = osph.gnomonic_kernel(centres, kh, kw, rlat, rlon, np.float64)
    assert s64.shape == (1, 200, kh * kw, 2)
    c64 = centres.astype(np.float64)
    x, y = _forward_gnomonic(s64[0, :, :, 0], s64[0, :, :, 1], c64[:, None, 0], c64[:, None, 1])
    jj = (np.arange(kh * kw) % kw - kw // 2) * rlon
    ii = (np.arange(kh * kw) // kw - kh // 2) * rlat
    np.testing.assert_allclose(x, np.broadcast_to(jj, x.shape), atol=1e-12)
    np.testing.assert_allclose(y, np.broadcast_to(ii, y.shape), atol=1e-12)
    centre = (kh // 2) * kw + kw // 2
    np.testing.assert_array_equal(s64[0, :, centre], c64)
    assert (s64[..., 0] >= -np.pi).all() and (s64[..., 0] < np.pi).all()
    s32 = osph.gnomonic_kernel(centres, kh, kw, rlat, rlon, np.float32)
    dlon = np.abs((s32[..., 0] - s64[..., 0] + np.pi) % (2 * np.pi) - np.pi)
    # (near a pole a longitude is ill-conditioned: compare on the sphere there)
    assert (dlon * np.cos(s64[..., 1])).max() < 2e-6
    assert np.abs(s32[..., 1] - s64[..., 1]).max() < 2e-6


@pytest.mark.gpu
def test_gpu_gnomonic_kernel_matches_oracle(device):
    """The device evaluates every entry in double and rounds once: within a float32 ulp of the
    float64 restatement (longitudes on the circle), within float32 rounding of the float32 one."""
    from mappedconvolutions_amd import util
    centres, kh, kw, rlat, rlon = _gnomonic_case()
    got = util.gnomonic_kernel(torch.tensor(centres).cuda(), kh, kw, rlat, rlon).cpu().numpy()
    s64 = osph.gnomonic_kernel(centres, kh, kw, rlat, rlon, np.float64)
    assert got.shape == s64.shape and got.dtype == np.float32
    dlon = np.abs((got[..., 0].astype(np.float64) - s64[..., 0] + np.pi) % (2 * np.pi) - np.pi)
    assert dlon.max() <= 2.5e-7 and np.abs(got[..., 1] - s64[..., 1]).max() <= 1.2e-7
    s32 = osph.gnomonic_kernel(centres, kh, kw, rlat, rlon, np.float32)
    dlon = np.abs((got[..., 0] - s32[..., 0] + np.pi) % (2 * np.pi) - np.pi)
    assert (dlon * np.cos(s64[..., 1])).max() < 2e-6
    assert np.abs(got[..., 1] - s32[..., 1]).max() < 2e-6
    assert (got[..., 0] >= -np.float32(np.pi)).all() and (got[..., 0] <= np.float32(np.pi)).all()


@pytest.mark.gpu
def test_gpu_operator_with_non_finite_samples_and_invalid_faces(device):
    """A sample direction with a NaN or infinite coordinate gets face -1 (and zeros), also in
    a mesh that holds faces with vertex indices out of range: those are culled before their
    vertices are read, for every sample.  All other samples are unaffected."""
    from mappedconvolutions_amd import _C, util
    verts, faces = util.synthetic.subdivided_icosahedron(2)
    g = torch.Generator().manual_seed(9)
    lon = (torch.rand(300, generator=g) * 2 - 1) * 3.1
    lat = (torch.rand(300, generator=g) - 0.5) * 3.0
    samples = torch.stack([lon, lat], -1)
    clean = _C.planar_conv_operator_from_samples(samples.view(30, 10, 2).cuda(), verts.cuda(),
                                                 faces.cuda())
    bad = samples.clone()
    bad[7, 0] = float("nan")
    bad[11, 1] = float("inf")
    bad[13] = float("nan")
    faces_bad = torch.cat([faces, torch.tensor([[0, 1, 10 ** 9], [-5, 2, 3]])]).contiguous()
    got = _C.planar_conv_operator_from_samples(bad.view(30, 10, 2).cuda(), verts.cuda(),
                                               faces_bad.cuda())
    for a, b in zip(got, clean):
        a, b = a.cpu().reshape(300, -1), b.cpu().reshape(300, -1)
        keep = torch.ones(300, dtype=torch.bool)
        keep[[7, 11, 13]] = False
        assert torch.equal(a[keep], b[keep])
    face, vidx, wts = [t.cpu().reshape(300, -1) for t in got]
    assert (face[[7, 11, 13]] == -1).all() and (vidx[[7, 11, 13]] == -1).all()
    assert (wts[[7, 11, 13]] == 0).all()
