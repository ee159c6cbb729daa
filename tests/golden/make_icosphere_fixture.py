"""Writes tests/golden/icosphere_operator.json from the reference's own `_sphere` module as
built by oracle/build_ref.py (its sphere.cpp compiled with g++ where it lies under
/root/reference; no reference Python is imported).  Run once in the build container:

    python tests/golden/make_icosphere_fixture.py

Contents (data only): the order-2 mesh the reference's operator works on internally
(generate_icosphere(0) then two Loop subdivisions: 162 vertices, 320 faces), seeded sample
directions - random ones plus every mesh vertex and points on edges - and what
Sphere.get_planar_conv_operator_from_samples(samples, 2, True, nearest) returned for them,
for nearest = False and True; and Sphere.get_vertex_resolution() of that mesh."""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import reference  # noqa: E402


def main():
    S = reference.module("_sphere").Sphere
    order = 2
    mesh = S.generate_icosphere(0).loop_subdivision(order)
    verts = mesh.get_vertices()
    faces = mesh.get_all_face_vertex_indices()
    rng = np.random.default_rng(7)
    n = 400
    lon = rng.uniform(-np.pi, np.pi, n)
    lat = np.arcsin(rng.uniform(-1, 1, n))
    v = verts.numpy().astype(np.float64)
    mid = 0.5 * (v[faces[:40, 0].numpy()] + v[faces[:40, 1].numpy()])  # on edges
    pts = np.concatenate([v, mid], 0)
    lon = np.concatenate([lon, np.arctan2(pts[:, 0], pts[:, 2])])
    lat = np.concatenate([lat, np.arctan2(-pts[:, 1], np.hypot(pts[:, 0], pts[:, 2]))])
    samples = torch.tensor(np.stack([lon, lat], -1), dtype=torch.float32).view(1, -1, 1, 2)
    out = {"order": order, "vertices": verts.tolist(), "faces": faces.tolist(),
           "samples": samples.view(-1, 2).tolist(),
           "vertex_resolution": float(mesh.get_vertex_resolution())}
    for nearest in (False, True):
        f, vi, w = S.get_planar_conv_operator_from_samples(samples, order, True, nearest)
        out["nearest" if nearest else "barycentric"] = {
            "face": f.view(-1).tolist(), "vertex_idx": vi.view(-1, 3).tolist(),
            "weights": w.view(-1, 3).tolist()}
    with open(os.path.join(HERE, "icosphere_operator.json"), "w") as fh:
        json.dump(out, fh)
    print("wrote %d samples on a mesh of %d vertices" % (samples.numel() // 2, verts.shape[0]))


if __name__ == "__main__":
    main()
