"""KNN through the grid search (points of one to three dimensions, 512 reference points or
more): bit-exact against the CPU oracle on small cases of every kind of point set the bins
could get wrong, and against the library's own walk over all points at full size."""
import ctypes

import pytest
import torch

from mappedconvolutions_amd import _lib
from mappedconvolutions_amd.util import knn, synthetic
from oracle import ops as O

pytestmark = pytest.mark.gpu


def _points(kind, D, n, g, dtype):
    if kind == "uniform":
        p = torch.rand(1, D, n, generator=g, dtype=torch.float64) * 4 - 1
    elif kind == "gaussian":
        p = torch.randn(1, D, n, generator=g, dtype=torch.float64)
    elif kind == "shell":  # points of a sphere / circle: most cells of the box stay empty
        p = torch.randn(1, D, n, generator=g, dtype=torch.float64)
        p = p / p.norm(dim=1, keepdim=True).clamp_min(1e-9) if D > 1 else p.sign()
    elif kind == "clusters":  # a few tight clusters and a handful of far points
        centres = torch.randn(D, 7, generator=g, dtype=torch.float64) * 5
        which = torch.randint(0, 7, (n,), generator=g)
        p = (centres[:, which] + 0.01 * torch.randn(D, n, generator=g, dtype=torch.float64))[None]
        p[0, :, :5] = torch.randn(D, 5, generator=g, dtype=torch.float64) * 100
    elif kind == "lattice":  # integer coordinates: equal distances everywhere
        p = torch.randint(-6, 7, (1, D, n), generator=g).to(torch.float64)
    else:
        raise ValueError(kind)
    return p.to(dtype).contiguous()


def _check(ref, qry, k):
    io, do = O.knn_forward(ref, qry, k)
    i, d = knn(ref.cuda(), qry.cuda(), k)
    assert torch.equal(i.cpu(), io), "KNN indices must be bit-exact"
    assert torch.equal(d.cpu(), do)


def _raw_knn(ref, qry, k, with_workspace):
    lib = _lib.load()
    B, D, R = ref.shape
    Q = qry.shape[2]
    idx = torch.empty(B, k, Q, dtype=torch.int64, device=ref.device)
    dist = torch.empty(B, k, Q, dtype=ref.dtype, device=ref.device)
    n = lib.mcx_knn_workspace(B, D, R, 0) if with_workspace else 0
    ws = torch.empty(max(n, 1), dtype=torch.uint8, device=ref.device)
    rc = lib.mcx_knn(ref.data_ptr(), qry.data_ptr(), idx.data_ptr(), dist.data_ptr(),
                     ws.data_ptr() if with_workspace else None, n, B, D, R, Q, k, 0,
                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    return idx, dist


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [1, 2, 3])
@pytest.mark.parametrize("kind", ["uniform", "gaussian", "shell", "clusters", "lattice"])
def test_grid_knn_vs_oracle(kind, D, dtype, device):
    g = torch.Generator().manual_seed(sum(map(ord, kind)) * 10 + D)
    R, Q = 1500 + 37 * D, 1100
    ref = _points(kind, D, R, g, dtype)
    qry = _points(kind, D, Q, g, dtype)
    qry[:, :, :40] = ref[:, :, 100:140]          # queries on top of reference points
    qry[:, :, 40:80] = qry[:, :, 40:80] * 3 + 2   # queries outside the references' box
    ref[:, :, 700] = ref[:, :, 20]               # a duplicate reference point
    assert _lib.load().mcx_knn_workspace(1, D, R, 0 if dtype == torch.float32 else 1) > 0
    for k in (1, 8, 33):
        _check(ref, qry, k)


def test_grid_knn_non_finite_points(device):
    """A point with a non-finite coordinate is nearer to nothing.  Among reference points past
    the first k the oracle (like the reference's insertion sort) says the same; for the first k,
    which the reference keeps unseen, and for non-finite queries the grid search is held to the
    library's walk over all points, which never lets such a point in."""
    g = torch.Generator().manual_seed(11)
    ref = torch.randn(1, 3, 900, generator=g)
    qry = torch.randn(1, 3, 300, generator=g)
    ref[0, 0, 105] = float("nan")
    ref[0, 1, 206] = float("inf")
    ref[0, 2, 307] = float("-inf")
    _check(ref, qry, 8)
    ref[0, 0, 2] = float("nan")
    ref[0, 1, 3] = float("inf")
    qry[0, 0, 3] = float("nan")
    qry[0, 2, 4] = float("inf")
    gi, gd = _raw_knn(ref.cuda(), qry.cuda(), 8, True)
    wi, wd = _raw_knn(ref.cuda(), qry.cuda(), 8, False)
    assert torch.equal(gi, wi) and torch.equal(gd, wd)
    assert (gi[0, :, 3:5] == 0).all() and not (gi == 3).any() and not (gi == 4).any()
    # fewer finite reference points than k: the unfilled rows are index 0, distance 0
    ref2 = torch.full((1, 2, 600), float("nan"))
    ref2[0, :, 100:109] = torch.randn(2, 9, generator=g)
    qry2 = torch.randn(1, 2, 50, generator=g)
    gi, gd = _raw_knn(ref2.cuda(), qry2.cuda(), 16, True)
    wi, wd = _raw_knn(ref2.cuda(), qry2.cuda(), 16, False)
    assert torch.equal(gi, wi) and torch.equal(gd, wd)
    assert (gi[:, 9:] == 0).all() and (gi[:, :9] > 100).all()


def test_grid_knn_degenerate_boxes(device):
    g = torch.Generator().manual_seed(12)
    # all reference points in one plane / on one line / at one point
    ref = torch.randn(1, 3, 800, generator=g)
    qry = torch.randn(1, 3, 200, generator=g)
    for flat in ([2], [1, 2], [0, 1, 2]):
        r = ref.clone()
        for d in flat:
            r[0, d] = 0.25
        _check(r, qry, 5)
    # most points at one spot (a skewed grid: the library walks all points instead)
    r = ref.clone()
    r[0, :, 100:] = r[0, :, 100:101]
    _check(r, qry, 8)


def test_grid_knn_batches_are_independent(device):
    g = torch.Generator().manual_seed(13)
    ref = torch.cat([_points(kind, 3, 1024, g, torch.float32) * s
                     for kind, s in (("uniform", 1.0), ("shell", 50.0), ("clusters", 0.01))])
    qry = torch.cat([_points(kind, 3, 513, g, torch.float32) * s
                     for kind, s in (("uniform", 1.0), ("shell", 50.0), ("clusters", 0.01))])
    _check(ref, qry, 8)


def test_grid_knn_full_size_equals_walk_over_all_points(device):
    """Config 4's shape (40962 references on the unit sphere, k = 8), a quarter of its queries:
    the grid search and the walk over all points, both through the C ABI, agree bit for bit."""
    ref = synthetic.sphere_points(40962, seed=1).to(device)
    qry = synthetic.sphere_points(131072, seed=2).to(device)
    gi, gd = _raw_knn(ref, qry, 8, True)
    wi, wd = _raw_knn(ref, qry, 8, False)
    assert torch.equal(gi, wi) and torch.equal(gd, wd)
    # a cube filled uniformly, and a workspace that is too small
    g = torch.Generator().manual_seed(5)
    ref = torch.rand(1, 3, 30000, generator=g).to(device)
    qry = (torch.rand(1, 3, 50000, generator=g) * 1.2 - 0.1).to(device)
    gi, gd = _raw_knn(ref, qry, 16, True)
    wi, wd = _raw_knn(ref, qry, 16, False)
    assert torch.equal(gi, wi) and torch.equal(gd, wd)
    lib = _lib.load()
    need = lib.mcx_knn_workspace(1, 3, 30000, 0)
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    assert lib.mcx_knn(ref.data_ptr(), qry.data_ptr(), gi.data_ptr(), gd.data_ptr(),
                       ws.data_ptr(), need - 1, 1, 3, 30000, 50000, 16, 0, None) == -4


@pytest.mark.parametrize("offset", [0.0, 4096.0])
def test_grid_knn_long_one_dimensional_grid(offset, device):
    """65 536 cells along one axis in fp32: the cell index of a point and the position of a
    cell face are rounded by amounts that grow with the index, up to hundredths of a cell at
    the far end (more when the coordinates sit far from the origin), so the early stop has to
    allow for them.  Points on a regular lattice of half a cell put a point on or next to
    every face; queries sit next to faces too.  Oracle on a sample, the walk over all points
    for the rest."""
    g = torch.Generator().manual_seed(77)
    R, Q = 131072, 8192
    step = 1.0 / 3.0
    ref = (torch.arange(R, dtype=torch.float64) * step + offset)
    ref = ref + (torch.rand(R, generator=g, dtype=torch.float64) - 0.5) * 1e-3 * step
    ref = ref[torch.randperm(R, generator=g)].float().view(1, 1, R).contiguous()
    at = torch.randint(0, R, (Q,), generator=g).double() * step + offset
    qry = (at + (torch.rand(Q, generator=g, dtype=torch.float64) - 0.5) * 4 * step).float()
    qry = qry.view(1, 1, Q).contiguous()
    assert _lib.load().mcx_knn_workspace(1, 1, R, 0) > 0
    gi, gd = _raw_knn(ref.cuda(), qry.cuda(), 8, True)
    wi, wd = _raw_knn(ref.cuda(), qry.cuda(), 8, False)
    assert torch.equal(gi, wi) and torch.equal(gd, wd)
    io, do = O.knn_forward(ref, qry[:, :, :256].contiguous(), 8)
    assert torch.equal(gi[:, :, :256].cpu(), io) and torch.equal(gd[:, :, :256].cpu(), do)
