"""Pooling gathers through LDS windows (unweighted, at most nine taps, rows a whole number of
16-byte chunks): every way a wave's taps can or cannot fit windows, bit-exact against the CPU
oracle - outputs and argmax - like the register path the windows replace."""
import math

import numpy as np
import pytest
import torch

from mappedconvolutions_amd import _C
from mappedconvolutions_amd.util import synthetic
from oracle import ops as O

pytestmark = pytest.mark.gpu


def _same(a, b):
    """Bitwise equality of values, a NaN in the same place counting as equal."""
    return torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(
        torch.nan_to_num(a, nan=0.0), torch.nan_to_num(b, nan=0.0))


def _check(x, smap, K, interp):
    mo, mi = O.mapped_max_pool(x, smap, K, interp)
    ao = O.mapped_avg_pool(x, smap, K, interp)
    m, i = _C.mapped_max_pool(x.cuda(), smap.cuda(), K, interp)
    a = _C.mapped_avg_pool(x.cuda(), smap.cuda(), K, interp)
    assert torch.equal(i.cpu(), mi), "argmax must be bit-exact"
    assert _same(m.cpu(), mo)
    assert _same(a.cpu(), ao)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("shape", [(24, 192), (9, 200), (6, 64), (5, 1024)])
def test_latitude_kernels(shape, interp, dtype, device):
    """Distortion-aware 3x3 kernels: taps of a row segment stay in one source row; stretched
    by up to 20 pixels next to the poles, across the seam at both ends of every row.  Widths
    of one to sixteen waves, one of them not a multiple of 64."""
    H, W = shape
    g = torch.Generator().manual_seed(H * W + interp)
    x = torch.randn(2, 5, H, W, generator=g, dtype=torch.float64).to(dtype)
    _check(x, synthetic.latitude_map(H, W, 1, dtype=dtype), 9, interp)


@pytest.mark.parametrize("interp", [0, 1, 2])
def test_fewer_taps_and_more_planes_than_a_thread_takes(interp, device):
    """2x2 kernels (K = 4 of the nine tap slots), and 3 x 50 planes: with few row segments a
    thread takes 64 planes, so the last of three groups is ragged."""
    H, W = 8, 128
    g = torch.Generator().manual_seed(7 + interp)
    i = np.arange(H, dtype=np.float64)[:, None, None]
    j = np.arange(W, dtype=np.float64)[None, :, None]
    dy = np.array([0, 0, 1, 1], np.float64).reshape(1, 1, -1)
    dx = np.array([0, 1, 0, 1], np.float64).reshape(1, 1, -1)
    stretch = 1.0 / np.maximum(np.cos(((i + 0.5) / H) * math.pi - math.pi / 2), 0.05)
    smap = np.stack([np.broadcast_to(j + dx * stretch, (H, W, 4)),
                     np.broadcast_to(i + dy + 0 * j, (H, W, 4))], -1)
    smap = torch.from_numpy(np.ascontiguousarray(smap)).float()
    x = torch.randn(3, 50, H, W, generator=g)
    _check(x, smap, 4, interp)


@pytest.mark.parametrize("interp", [0, 1, 2])
def test_zero_padded_borders_and_strides(interp, device):
    """Plain 3x3 grid taps (corners beyond every border), a map of stride 2 (the pooled image is
    half as wide as the source); with nearest taps the source holds an Inf and a NaN (bilinear
    corners of weight exactly zero are not read by any of the library's pooling paths, where
    the reference multiplies them by zero: a non-finite value under one is out of contract)."""
    H, W = 10, 128
    g = torch.Generator().manual_seed(17 + interp)
    x = torch.randn(1, 3, H, W, generator=g)
    if interp == 0:
        x[0, 0, 3, 70] = float("inf")
        x[0, 1, 5, 5] = float("nan")
    _check(x, synthetic.identity_grid_map(H, W, 1), 9, interp)
    OH, OW = H // 2, W // 2
    i = np.arange(OH, dtype=np.float64)[:, None, None]
    j = np.arange(OW, dtype=np.float64)[None, :, None]
    offs = np.arange(-1, 2, dtype=np.float64)
    dy, dx = [a.reshape(1, 1, -1) for a in np.meshgrid(offs, offs, indexing="ij")]
    smap = np.stack([2 * j + dx + 0 * i, 2 * i + dy + 0 * j], -1)
    _check(x, torch.from_numpy(np.ascontiguousarray(smap)).float(), 9, interp)


@pytest.mark.parametrize("interp", [0, 1])
def test_maps_that_do_not_fit_windows(interp, device):
    """Waves whose taps cannot use windows take the register path, wave by wave: row coordinates
    that are not integral, taps scattered at random, lanes of one tap in different source rows
    (a rotated grid), spans longer than a window; and a row length that is not a whole number of
    chunks (no windows at all)."""
    H, W = 12, 256
    g = torch.Generator().manual_seed(27 + interp)
    x = torch.randn(2, 4, H, W, generator=g)
    lat = synthetic.latitude_map(H, W, 1)
    frac = lat.clone()
    frac[..., 1] += 0.25
    _check(x, frac, 9, interp)
    rnd = torch.stack([torch.rand(H, W, 9, generator=g) * (W + 4) - 2,
                       torch.rand(H, W, 9, generator=g) * (H + 4) - 2], -1)
    _check(x, rnd, 9, interp)
    mixed = lat.clone()
    mixed[:, 100:, :, :] = rnd[:, 100:, :, :]      # some waves fit, their neighbours do not
    _check(x, mixed, 9, interp)
    rot = lat.clone()
    rot[..., 1] = (rot[..., 1] + torch.arange(W).view(1, W, 1) // 40).clamp(max=H - 1)
    _check(x, rot, 9, interp)
    wide = lat.clone()
    wide[..., 0] = (torch.arange(W).view(1, W, 1) * 9.0 + wide[..., 0]) % W   # 9 columns apart
    _check(x, wide, 9, interp)
    xo = torch.randn(1, 2, 7, 202, generator=g)
    _check(xo, synthetic.latitude_map(7, 202, 1), 9, interp)


# ------------------------------------------------------------------ unpoolings
def _rel(a, b):
    return float((a.cpu().double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def _check_unpool(gy, smap, H, W, K, interp, plan=False):
    """avg and max unpooling of gy (the size of the map) onto H x W, against the oracle; the
    argmax comes from the oracle's pooling of a random image."""
    g = torch.Generator().manual_seed(99)
    x = torch.randn(gy.shape[0], gy.shape[1], H, W, generator=g, dtype=gy.dtype)
    _, mi = O.mapped_max_pool(x, smap, K, interp)
    want_avg = O.mapped_avg_unpool(gy, smap, H, W, K, interp)
    want_max = O.mapped_max_unpool(gy, mi, smap, H, W, K, interp)
    kw = {}
    if plan:
        kw_avg = {"plan": _C.scatter_map_plan(smap.cuda(), None, H, W, interp, kernel=True)}
        kw_max = {"plan": _C.scatter_map_plan(smap.cuda(), None, H, W, interp, for_max_unpool=True,
                                              kernel=True)}
    else:
        kw_avg = kw_max = kw
    got_avg = _C.mapped_avg_unpool(gy.cuda(), smap.cuda(), H, W, K, interp, **kw_avg)
    got_max = _C.mapped_max_unpool(gy.cuda(), mi.cuda(), smap.cuda(), H, W, K, interp, **kw_max)
    assert _rel(got_avg, want_avg) < 1e-5     # tolerance of the atomic-accumulated paths
    assert _rel(got_max, want_max) < 1e-5


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("shape", [(24, 192), (9, 200), (6, 64), (5, 1024), (7, 202)])
def test_unpoolings_over_latitude_kernels(shape, interp, device):
    """The unpoolings gather through per-pixel lists; where a wave's lists read a few short runs
    of the pooled image they are staged in LDS.  Widths of one to sixteen waves, one whose
    destination rows end inside a wave, one whose planes are not whole 16-byte chunks (no
    windows); with and without a plan."""
    H, W = shape
    g = torch.Generator().manual_seed(H + W + interp)
    gy = torch.randn(2, 70, H, W, generator=g)      # 140 planes: groups of 64, the last ragged
    lmap = synthetic.latitude_map(H, W, 1)
    _check_unpool(gy, lmap, H, W, 9, interp)
    _check_unpool(gy[:, :3].contiguous(), lmap, H, W, 9, interp, plan=True)


@pytest.mark.parametrize("interp", [0, 1])
def test_unpoolings_whose_lists_do_not_fit_windows(interp, device):
    """Lists longer than a lane keeps (row coordinates that are not integral: up to 36 entries),
    scattered taps, a pooled image smaller than the unpooled one (stride 2), and a mixture."""
    H, W = 12, 256
    g = torch.Generator().manual_seed(31 + interp)
    gy = torch.randn(1, 5, H, W, generator=g)
    lat = synthetic.latitude_map(H, W, 1)
    frac = lat.clone()
    frac[..., 1] += 0.25
    _check_unpool(gy, frac, H, W, 9, interp)
    rnd = torch.stack([torch.rand(H, W, 9, generator=g) * (W + 4) - 2,
                       torch.rand(H, W, 9, generator=g) * (H + 4) - 2], -1)
    _check_unpool(gy, rnd, H, W, 9, interp)
    mixed = lat.clone()
    mixed[:, 100:, :, :] = rnd[:, 100:, :, :]
    _check_unpool(gy, mixed, H, W, 9, interp)
    OH, OW = H // 2, W // 2
    i = np.arange(OH, dtype=np.float64)[:, None, None]
    j = np.arange(OW, dtype=np.float64)[None, :, None]
    offs = np.arange(-1, 2, dtype=np.float64)
    dy, dx = [a.reshape(1, 1, -1) for a in np.meshgrid(offs, offs, indexing="ij")]
    smap = torch.from_numpy(np.ascontiguousarray(
        np.stack([2 * j + dx + 0 * i, 2 * i + dy + 0 * j], -1))).float()
    _check_unpool(gy[:, :, :OH, :OW].contiguous(), smap, H, W, 9, interp)


@pytest.mark.parametrize("interp", [0, 1])
def test_weighted_unpoolings_through_windows(interp, device):
    """Weighted taps (two points per tap, the second one column to the right): lists of up to
    twelve (nearest) entries go through the windows, longer ones (bilinear) through the register
    path; the recorded winners of the weighted max pooling count points, not taps."""
    H, W, K, P = 10, 192, 3, 2
    g = torch.Generator().manual_seed(41 + interp)
    i = np.arange(H, dtype=np.float64)[:, None, None, None]
    j = np.arange(W, dtype=np.float64)[None, :, None, None]
    dx = np.array([-1.0, 0.0, 1.0]).reshape(1, 1, K, 1)
    pt = np.array([0.0, 1.0]).reshape(1, 1, 1, P)
    x = np.mod(j + dx * 1.5 + pt + 0 * i, W)
    y = i + 0 * j + 0 * dx + 0 * pt
    smap = torch.from_numpy(np.ascontiguousarray(np.stack([x, y], -1))).float()
    wts = torch.rand(H, W, K, P, generator=g) + 0.1
    gy = torch.randn(2, 6, H, W, generator=g)
    src = torch.randn(2, 6, H, W, generator=g)
    _, mi = O.weighted_mapped_max_pool(src, smap, wts, K, interp)
    want_avg = O.weighted_mapped_avg_unpool(gy, smap, wts, H, W, K, interp)
    want_max = O.weighted_mapped_max_unpool(gy, mi, smap, wts, H, W, K, interp)
    got_avg = _C.weighted_mapped_avg_unpool(gy.cuda(), smap.cuda(), wts.cuda(), H, W, K, interp)
    got_max = _C.weighted_mapped_max_unpool(gy.cuda(), mi.cuda(), smap.cuda(), wts.cuda(), H, W,
                                            K, interp)
    assert _rel(got_avg, want_avg) < 1e-5
    assert _rel(got_max, want_max) < 1e-5
