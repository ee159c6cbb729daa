"""CPU tests that pin the oracle: (1) the reference's own hand-computed known
answers, (2) the reference's CPU build (oracle/_ref) where it has been built,
(3) what the mathematics fixes: library special cases (grid_sample, conv2d,
cdist), adjointness, brute force."""
import pytest
import torch
import torch.nn.functional as F

import helpers
from helpers import CASES, rel_err
from oracle import ops as O
from oracle import reference as R

from mappedconvolutions_amd.util import synthetic

DTYPES = [torch.float32, torch.float64]


@pytest.mark.parametrize("name", sorted(CASES))
def test_known_answers(name):
    out, exp = helpers.run_case(O, CASES[name])
    torch.testing.assert_close(out, exp.expand_as(out), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("name", sorted(CASES))
def test_known_answers_float32(name):
    out, exp = helpers.run_case(O, CASES[name], dtype=torch.float32)
    torch.testing.assert_close(out, exp.expand_as(out), rtol=1e-6, atol=1e-6)


def test_nearest_rounds_half_away_from_zero():
    # 0.5 -> 1, 1.5 -> 2, 2.5 -> 3 (half-even would give 0, 2, 2); -0.5 -> -1 (outside)
    x = torch.arange(12, dtype=torch.float32).view(1, 1, 3, 4)
    smap = torch.tensor([[[0.5, 0.0], [1.5, 0.5], [2.5, 1.5], [-0.5, 0.0],
                          [0.49999997, 0.0]]], dtype=torch.float32)
    out = O.resample_from_map(x, smap, 0)
    assert out.flatten().tolist() == [1.0, 6.0, 11.0, 0.0, 0.0]


# ---------------------------------------------------------------- vs oracle/_ref
needs_ref = pytest.mark.skipif(not R.available(), reason="oracle/_ref not built")


def _problem(dtype, seed, p=0, integer=False, half=False):
    g = torch.Generator().manual_seed(seed)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 3, 5, 6, 7, 4, 5, 4
    x = torch.randn(B, Ci, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, wts = helpers.random_map(g, OH, OW, K, p, IH, IW, dtype, integer, half)
    w = torch.randn(Co, Ci, K, generator=g, dtype=torch.float64).to(dtype)
    b = torch.randn(Co, generator=g, dtype=torch.float64).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    return x, smap, wts, w, b, gy


def _tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-12, atol=1e-12)


@needs_ref
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_conv_vs_reference_build(dtype, interp, p):
    x, smap, wts, w, b, gy = _problem(dtype, 1 + interp + 10 * p, p)
    K = 4
    if p:
        ref = R.module("_weighted_mapped_convolution")
        y_r = ref.weighted_mapped_conv_forward(x, smap, wts, w, b, K, interp)
        g_r = ref.weighted_mapped_conv_backward(gy, smap, wts, x, w, b, K, interp)
        y_o = O.weighted_mapped_conv_forward(x, smap, wts, w, b, K, interp)
        g_o = O.weighted_mapped_conv_backward(gy, smap, wts, x, w, b, K, interp)
    else:
        ref = R.module("_mapped_convolution")
        y_r = ref.mapped_conv_forward(x, smap, w, b, K, interp)
        g_r = ref.mapped_conv_backward(gy, smap, x, w, b, K, interp)
        y_o = O.mapped_conv_forward(x, smap, w, b, K, interp)
        g_o = O.mapped_conv_backward(gy, smap, x, w, b, K, interp)
    torch.testing.assert_close(y_o, y_r, **_tol(dtype))
    for a, r in zip(g_o, g_r):
        torch.testing.assert_close(a, r, **_tol(dtype))


@needs_ref
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_tconv_vs_reference_build(dtype, interp, p):
    g = torch.Generator().manual_seed(7 + interp + 10 * p)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 3, 4, 4, 5, 6, 7, 4
    x = torch.randn(B, Ci, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, wts = helpers.random_map(g, IH, IW, K, p, OH, OW, dtype)
    w = torch.randn(Ci, Co, K, generator=g, dtype=torch.float64).to(dtype)
    b = torch.randn(Co, generator=g, dtype=torch.float64).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    if p:
        ref = R.module("_weighted_mapped_transposed_convolution")
        y_r = ref.weighted_mapped_transposed_conv_forward(x, smap, wts, w, b, OH, OW, K, interp)
        g_r = ref.weighted_mapped_transposed_conv_backward(gy, smap, wts, x, w, b, K, interp)
        y_o = O.weighted_mapped_transposed_conv_forward(x, smap, wts, w, b, OH, OW, K, interp)
        g_o = O.weighted_mapped_transposed_conv_backward(gy, smap, wts, x, w, b, K, interp)
    else:
        ref = R.module("_mapped_transposed_convolution")
        y_r = ref.mapped_transposed_conv_forward(x, smap, w, b, OH, OW, K, interp)
        g_r = ref.mapped_transposed_conv_backward(gy, smap, x, w, b, K, interp)
        y_o = O.mapped_transposed_conv_forward(x, smap, w, b, OH, OW, K, interp)
        g_o = O.mapped_transposed_conv_backward(gy, smap, x, w, b, K, interp)
    torch.testing.assert_close(y_o, y_r, **_tol(dtype))
    for a, r in zip(g_o, g_r):
        torch.testing.assert_close(a, r, **_tol(dtype))


@needs_ref
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_pools_vs_reference_build(dtype, interp, p):
    g = torch.Generator().manual_seed(11 + interp + 10 * p)
    B, C, IH, IW, OH, OW, K = 2, 3, 6, 7, 4, 5, 4
    # strictly positive data: the reference's CPU max-pool starts its running
    # maximum at the smallest positive normal, the CUDA build (followed here) at -FLT_MAX
    x = (torch.rand(B, C, IH, IW, generator=g, dtype=torch.float64) + 0.5).to(dtype)
    smap, wts = helpers.random_map(g, OH, OW, K, p, IH - 3, IW - 3, dtype)
    smap = smap.clamp(0, 3)  # every tap inside the image: every value positive
    gy = torch.randn(B, C, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    if p:
        rm, ra = R.module("_weighted_mapped_max_pooling"), R.module("_weighted_mapped_avg_pooling")
        mp_r = rm.weighted_mapped_max_pool(x, smap, wts, K, interp)
        mp_o = O.weighted_mapped_max_pool(x, smap, wts, K, interp)
        mu_r = rm.weighted_mapped_max_unpool(gy, mp_r[1], smap, wts, IH, IW, K, interp)
        mu_o = O.weighted_mapped_max_unpool(gy, mp_o[1], smap, wts, IH, IW, K, interp)
        ap_r = ra.weighted_mapped_avg_pool(x, smap, wts, K, interp)
        ap_o = O.weighted_mapped_avg_pool(x, smap, wts, K, interp)
        au_r = ra.weighted_mapped_avg_unpool(gy, smap, wts, IH, IW, K, interp)
        au_o = O.weighted_mapped_avg_unpool(gy, smap, wts, IH, IW, K, interp)
    else:
        rm, ra = R.module("_mapped_max_pooling"), R.module("_mapped_avg_pooling")
        mp_r = rm.mapped_max_pool(x, smap, K, interp)
        mp_o = O.mapped_max_pool(x, smap, K, interp)
        mu_r = rm.mapped_max_unpool(gy, mp_r[1], smap, IH, IW, K, interp)
        mu_o = O.mapped_max_unpool(gy, mp_o[1], smap, IH, IW, K, interp)
        ap_r = ra.mapped_avg_pool(x, smap, K, interp)
        ap_o = O.mapped_avg_pool(x, smap, K, interp)
        au_r = ra.mapped_avg_unpool(gy, smap, IH, IW, K, interp)
        au_o = O.mapped_avg_unpool(gy, smap, IH, IW, K, interp)
    assert torch.equal(mp_o[0], mp_r[0]) and torch.equal(mp_o[1], mp_r[1])
    torch.testing.assert_close(mu_o, mu_r, **_tol(dtype))
    torch.testing.assert_close(ap_o, ap_r, **_tol(dtype))
    torch.testing.assert_close(au_o, au_r, **_tol(dtype))


@needs_ref
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
@pytest.mark.parametrize("half", [False, True])
def test_resample_vs_reference_build(dtype, interp, p, half):
    g = torch.Generator().manual_seed(3 + interp + 10 * p)
    B, C, IH, IW, OH, OW = 2, 3, 5, 6, 7, 8
    x = torch.randn(B, C, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, wts = helpers.random_map(g, IH, IW, 1, p, OH, OW, dtype, half=half)
    smap = smap[:, :, 0].contiguous()
    wts = None if wts is None else wts[:, :, 0].contiguous()
    y = torch.randn(B, C, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    if p:
        ref = R.module("_weighted_resample")
        to_r = ref.weighted_resample_to_map(x, smap, wts, OH, OW, interp)
        fr_r = ref.weighted_resample_from_map(y, smap, wts, interp)
        to_o = O.weighted_resample_to_map(x, smap, wts, OH, OW, interp)
        fr_o = O.weighted_resample_from_map(y, smap, wts, interp)
    else:
        ref = R.module("_resample")
        to_r = ref.resample_to_map(x, smap, OH, OW, interp)
        fr_r = ref.resample_from_map(y, smap, interp)
        to_o = O.resample_to_map(x, smap, OH, OW, interp)
        fr_o = O.resample_from_map(y, smap, interp)
    assert torch.equal(fr_o, fr_r)  # gathers are order-free: bit-exact
    torch.testing.assert_close(to_o, to_r, **_tol(dtype))


# ------------------------------------------------------------- closed-form checks
def test_bilinear_equals_grid_sample():
    """Bilinear with zero padding == grid_sample(align_corners=True, zeros)."""
    g = torch.Generator().manual_seed(5)
    H, W = 9, 11
    src = torch.randn(2, 3, H, W, generator=g, dtype=torch.float64)
    smap, _ = helpers.random_map(g, 6, 7, 1, 0, H, W, torch.float64)
    smap = smap[:, :, 0].contiguous()
    out = O.resample_from_map(src, smap, 1)
    grid = torch.stack([2 * smap[..., 0] / (W - 1) - 1, 2 * smap[..., 1] / (H - 1) - 1], -1)
    ref = F.grid_sample(src, grid[None].expand(2, -1, -1, -1), mode='bilinear',
                        padding_mode='zeros', align_corners=True)
    torch.testing.assert_close(out, ref, rtol=1e-10, atol=1e-10)


def test_bispherical_equals_grid_sample_on_wrapped_input():
    g = torch.Generator().manual_seed(6)
    H, W = 7, 8
    src = torch.randn(1, 2, H, W, generator=g, dtype=torch.float64)
    x = torch.rand(5, 6, generator=g, dtype=torch.float64) * (W + 1) - 1  # [-1, W)
    y = torch.rand(5, 6, generator=g, dtype=torch.float64) * (H + 1) - 1
    smap = torch.stack([x, y], -1)
    out = O.resample_from_map(src, smap, 2)
    padded = torch.cat([src[..., -1:], src, src[..., :1]], -1)  # one wrapped column each side
    Wp = W + 2
    grid = torch.stack([2 * (x + 1) / (Wp - 1) - 1, 2 * y / (H - 1) - 1], -1)[None]
    ref = F.grid_sample(padded, grid, mode='bilinear', padding_mode='zeros', align_corners=True)
    torch.testing.assert_close(out, ref, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("interp", [0, 1])
@pytest.mark.parametrize("radius", [1, 2])
def test_identity_map_conv_equals_conv2d(interp, radius):
    g = torch.Generator().manual_seed(8)
    B, Ci, Co, H, W = 2, 3, 4, 7, 9
    k = 2 * radius + 1
    x = torch.randn(B, Ci, H, W, generator=g, dtype=torch.float64)
    w = torch.randn(Co, Ci, k * k, generator=g, dtype=torch.float64)
    b = torch.randn(Co, generator=g, dtype=torch.float64)
    smap = synthetic.identity_grid_map(H, W, radius, torch.float64)
    x.requires_grad_(True)
    wr = w.clone().requires_grad_(True)
    ref = F.conv2d(x, wr.view(Co, Ci, k, k), b, padding=radius)
    gy = torch.randn(ref.shape, generator=g, dtype=torch.float64)
    gx_ref, gw_ref = torch.autograd.grad(ref, (x, wr), gy)
    out = O.mapped_conv_forward(x.detach(), smap, w, b, k * k, interp)
    gx, gw, gb = O.mapped_conv_backward(gy, smap, x.detach(), w, b, k * k, interp)
    torch.testing.assert_close(out, ref.detach(), rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gx, gx_ref, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gw, gw_ref, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gb, gy.sum((0, 2, 3)), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 2])
def test_scatter_is_adjoint_of_gather(interp, p):
    """<from_map(s), g> == <s, to_map(g)>, which pins resample_to_map (the
    reference has no direct test for it) and the unpool ops."""
    g = torch.Generator().manual_seed(9)
    B, C, SH, SW, MH, MW, K = 2, 2, 5, 6, 4, 7, 3
    s = torch.randn(B, C, SH, SW, generator=g, dtype=torch.float64)
    smap, wts = helpers.random_map(g, MH, MW, K, p, SH, SW, torch.float64)
    gk = torch.randn(B, C, MH, MW, generator=g, dtype=torch.float64)
    sm1 = smap[:, :, 0].contiguous()
    w1 = None if wts is None else wts[:, :, 0].contiguous()
    lhs = (O.weighted_resample_from_map(s, sm1, w1, interp) * gk).sum()
    rhs = (s * O.weighted_resample_to_map(gk, sm1, w1, SH, SW, interp)).sum()
    torch.testing.assert_close(lhs, rhs, rtol=1e-12, atol=1e-12)
    lhs = (O.weighted_mapped_avg_pool(s, smap, wts, K, interp) * gk).sum()
    rhs = (s * O.weighted_mapped_avg_unpool(gk, smap, wts, SH, SW, K, interp)).sum()
    torch.testing.assert_close(lhs, rhs, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 2])
def test_pools_brute_force(interp, p):
    """max/avg over the K taps of resample_from_map, argmax offset formula."""
    g = torch.Generator().manual_seed(10)
    B, C, IH, IW, OH, OW, K = 2, 3, 5, 6, 3, 4, 5
    x = torch.randn(B, C, IH, IW, generator=g, dtype=torch.float64)
    smap, wts = helpers.random_map(g, OH, OW, K, p, IH, IW, torch.float64)
    taps = []
    for k in range(K):
        sm = smap[:, :, k].contiguous()
        w = None if wts is None else wts[:, :, k].contiguous()
        taps.append(O.weighted_resample_from_map(x, sm, w, interp))
    taps = torch.stack(taps, -1)  # B,C,OH,OW,K
    mx, arg = taps.max(-1)
    # first maximum wins
    first = (taps == mx[..., None]).to(torch.int64).argmax(-1)
    pm = max(p, 1)
    n = torch.arange(OH * OW).view(OH, OW)
    exp_idx = (n * K + first) * pm * 2
    out, idx = O.weighted_mapped_max_pool(x, smap, wts, K, interp)
    assert torch.equal(out, mx) and torch.equal(idx, exp_idx)
    avg = O.weighted_mapped_avg_pool(x, smap, wts, K, interp)
    seq = torch.zeros_like(mx)
    for k in range(K):
        seq = seq + taps[..., k]
    assert torch.equal(avg, seq / K)
    # unpool routes the gradient through the recorded tap only
    gy = torch.randn(B, C, OH, OW, generator=g, dtype=torch.float64)
    gin = O.weighted_mapped_max_unpool(gy, idx, smap, wts, IH, IW, K, interp)
    exp = torch.zeros_like(x)
    for k in range(K):
        sm = smap[:, :, k].contiguous()
        w = None if wts is None else wts[:, :, k].contiguous()
        exp += O.weighted_resample_to_map(gy * (first == k), sm, w, IH, IW, interp)
    torch.testing.assert_close(gin, exp, rtol=1e-12, atol=1e-12)


def test_max_pool_all_negative_follows_gpu_semantics():
    x = -torch.ones(1, 1, 3, 3, dtype=torch.float32)
    smap = torch.tensor([[[[1.0, 1.0], [0.0, 0.0]]]])
    out, idx = O.mapped_max_pool(x, smap, 2, 0)
    assert out.item() == -1.0 and idx.item() == 0


def test_tconv_forward_is_conv_backward_input():
    g = torch.Generator().manual_seed(12)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 3, 4, 4, 5, 6, 7, 3
    x = torch.randn(B, Ci, IH, IW, generator=g, dtype=torch.float64)
    smap, _ = helpers.random_map(g, IH, IW, K, 0, OH, OW, torch.float64)
    w = torch.randn(Ci, Co, K, generator=g, dtype=torch.float64)
    y = O.mapped_transposed_conv_forward(x, smap, w, torch.zeros(Co, dtype=torch.float64), OH, OW,
                                         K, 1)
    # conv with weight [Ci(out), Co(in), K]: its backward-input maps [B,Ci,IH,IW] -> [B,Co,OH,OW]
    dummy = torch.zeros(B, Co, OH, OW, dtype=torch.float64)
    gx = O.mapped_conv_backward(x, smap, dummy, w, None, K, 1)[0]
    torch.testing.assert_close(y, gx, rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------------------- knn
@pytest.mark.parametrize("dtype", DTYPES)
def test_knn_brute_force(dtype):
    """orc_knn against a stable sort of distances accumulated the same way
    (fused multiply-add per dimension, in order)."""
    g = torch.Generator().manual_seed(13)
    B, D, R, Q, k = 2, 3, 200, 150, 8
    ref = torch.randn(B, D, R, generator=g, dtype=torch.float64).to(dtype)
    qry = torch.randn(B, D, Q, generator=g, dtype=torch.float64).to(dtype)
    ref[:, :, 50] = ref[:, :, 10]  # exact duplicates: ties must keep the lower index
    qry[:, :, 0] = ref[:, :, 10]
    idx, dist = O.knn_forward(ref, qry, k)
    ssd = torch.zeros(B, R, Q, dtype=dtype)
    for d in range(D):
        t = ref[:, d, :, None] - qry[:, d, None, :]
        ssd = torch.addcmul(ssd, t, t) if dtype == torch.float64 else _fma32(t, t, ssd)
    order = torch.sort(ssd, dim=1, stable=True)
    assert torch.equal(idx, order.indices[:, :k] + 1)
    torch.testing.assert_close(dist, order.values[:, :k].sqrt(), rtol=1e-6, atol=0)
    assert (idx[:, 0, 0] == 11).all() and (idx[:, 1, 0] == 51).all()
    # against the library routine, on distances
    cd = torch.cdist(qry.transpose(1, 2).double(), ref.transpose(1, 2).double())
    torch.testing.assert_close(dist.double(), cd.sort(-1).values[..., :k].transpose(1, 2),
                               rtol=1e-5, atol=1e-6)


def _fma32(a, b, c):
    """float32 fused multiply-add emulated exactly through float64."""
    return (a.double() * b.double() + c.double()).float()


def test_latitude_map_rule():
    H, W = 64, 128
    m = synthetic.latitude_map(H, W, 1)
    assert m.shape == (H, W, 9, 2)
    import math
    i, j, k = 10, 100, 2  # dy=-1, dx=+1
    lat = ((i + 0.5) / H) * math.pi - math.pi / 2
    assert abs(m[i, j, k, 0].item() - ((j + 1 / max(math.cos(lat), 0.05)) % W)) < 1e-4
    assert m[i, j, k, 1].item() == i - 1
    assert m[0, 5, 0, 1].item() == 0 and m[H - 1, 5, 8, 1].item() == H - 1
