"""GPU parity tests of the convolution code paths that ordinary (one-to-few) maps never take,
and of the BASELINE configurations 3 and 5 at their full sizes.

* Strongly many-to-one maps: the input gradient of a convolution whose output grid is several
  times finer than its input, and the forward of a transposed convolution whose input grid is
  several times finer than its output, overflow the slotted transposed map and its overflow
  list, so the product runs through the scatter kernel (LDS windows, race check, atomics).
  Each such test asserts on the host that the map does overflow.
* fp32 with more than four interpolation points per tap (scalar kernels), a single tap.
* The reference's known answers pushed through the fp32 and bf16 matrix-core kernels.
* Full-size configurations 3 and 5: sampled output positions against the oracle evaluated on
  just those positions, and size-independent properties.

Bars as elsewhere: 1e-5 of the result's magnitude in fp32, 2e-2 with bf16 storage."""
import pytest
import torch
import torch.nn.functional as F

import helpers
from helpers import CASES, KNOWN, rel_err, assert_close_elementwise
from oracle import ops as O

from mappedconvolutions_amd import _C, nn
from mappedconvolutions_amd.util import synthetic

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


def _weighted_variant(smap, p, gen):
    """[.., K, 2] -> ([.., K, p, 2], weights [.., K, p]): every tap becomes p points jittered
    around the original location."""
    if not p:
        return smap, None
    jitter = torch.rand(smap.shape[:-1] + (p, 2), generator=gen) * 1.5 - 0.75
    iw = torch.rand(smap.shape[:-1] + (p,), generator=gen) + 0.1
    return (smap.unsqueeze(-2) + jitter).contiguous(), iw.contiguous()


MANY_TO_ONE = {
    # name: (source H, W, factor, radius, latitude, aligned)
    "grid_x4": (6, 10, 4, 1, False, False),
    "aligned_x4": (5, 9, 4, 1, False, True),       # integral and .5 coordinates, zero weights
    "latitude_x4_5x5": (8, 64, 4, 2, True, False),  # pole rows: windows beyond 160 slots
    "grid_x3": (7, 11, 3, 1, False, False),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("interp", [1, 2])
@pytest.mark.parametrize("p", [0, 3])
@pytest.mark.parametrize("case", sorted(MANY_TO_ONE))
def test_conv_input_gradient_through_scatter_kernel(case, p, interp, dtype, device):
    """Convolution whose output grid is finer than its input: grad_input collects about
    factor^2 x corners contributions per (pixel, tap).  Channels are ragged for every tile
    size in use (70 = 64 + 6 source channels, 21 = 16 + 5 destination channels)."""
    IH, IW, f, radius, latitude, aligned = MANY_TO_ONE[case]
    if p and case == "latitude_x4_5x5":
        pytest.skip("K=25 x P=3: covered unweighted")
    g = torch.Generator().manual_seed(1000 + 7 * p + interp)
    B, Ci, Co = 2, 21, 70
    K = (2 * radius + 1) ** 2
    smap = synthetic.upsampling_map(IH, IW, f, radius, latitude, aligned)
    smap, iw = _weighted_variant(smap, p, g)
    OH, OW = smap.shape[:2]
    if case != "grid_x3":  # x3: near the limit, the overflow list holds most contributions
        assert helpers.transposed_map_overflows(smap, iw, IH, IW, interp), \
            "this map is meant to overflow the transposed map"
    x = torch.randn(B, Ci, IH, IW, generator=g).to(dtype)
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dtype)
    b = torch.randn(Co, generator=g).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g).to(dtype)
    y_o = O.weighted_mapped_conv_forward(x.float(), smap, iw, w.float(), b.float(), K, interp)
    g_o = O.weighted_mapped_conv_backward(gy.float(), smap, iw, x.float(), w.float(), b.float(),
                                          K, interp)
    xd, sd, iwd, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    if p:
        y = _C.weighted_mapped_conv_forward(xd, sd, iwd, wd_, bd, K, interp)
        gr = _C.weighted_mapped_conv_backward(gyd, sd, iwd, xd, wd_, bd, K, interp)
    else:
        y = _C.mapped_conv_forward(xd, sd, wd_, bd, K, interp)
        gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, interp)
    tol = TOL[dtype]
    assert rel_err(y.float(), y_o) < tol
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm
    assert_close_elementwise(gr[0].float(), g_o[0], 4 * tol, "grad_input")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("interp", [1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_tconv_forward_through_scatter_kernel(p, interp, dtype, device):
    """Transposed convolution whose input grid is four times finer than its output: the
    forward is the many-to-one scatter.  130 source channels (three register blocks of 64),
    37 destination channels; the bias initialises the output."""
    g = torch.Generator().manual_seed(1100 + 7 * p + interp)
    B, Ci, Co, OH, OW, f = 2, 130, 37, 6, 9, 4
    smap = synthetic.upsampling_map(OH, OW, f, 1)
    smap, iw = _weighted_variant(smap, p, g)
    IH, IW, K = smap.shape[0], smap.shape[1], 9
    assert helpers.transposed_map_overflows(smap, iw, OH, OW, interp)
    x = torch.randn(B, Ci, IH, IW, generator=g).to(dtype)
    w = (torch.randn(Ci, Co, K, generator=g) / (Ci * K) ** 0.5).to(dtype)
    b = torch.randn(Co, generator=g).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g).to(dtype)
    y_o = O.weighted_mapped_transposed_conv_forward(x.float(), smap, iw, w.float(), b.float(),
                                                    OH, OW, K, interp)
    g_o = O.weighted_mapped_transposed_conv_backward(gy.float(), smap, iw, x.float(), w.float(),
                                                     b.float(), K, interp)
    xd, sd, iwd, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    if p:
        y = _C.weighted_mapped_transposed_conv_forward(xd, sd, iwd, wd_, bd, OH, OW, K, interp)
        gr = _C.weighted_mapped_transposed_conv_backward(gyd, sd, iwd, xd, wd_, bd, K, interp)
    else:
        y = _C.mapped_transposed_conv_forward(xd, sd, wd_, bd, OH, OW, K, interp)
        gr = _C.mapped_transposed_conv_backward(gyd, sd, xd, wd_, bd, K, interp)
    tol = TOL[dtype]
    assert rel_err(y.float(), y_o) < tol
    assert_close_elementwise(y.float(), y_o, 4 * tol, "tconv forward")
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm


@pytest.mark.parametrize("interp", [0, 1, 2])
def test_tconv_upsampling_decoder(interp, device):
    """The decoder use of a transposed convolution: a coarse input spread over an output grid
    three times finer (each input pixel's taps land on different output pixels)."""
    g = torch.Generator().manual_seed(1200 + interp)
    B, Ci, Co, IH, IW, f, K = 2, 24, 20, 8, 12, 3, 9
    OH, OW = IH * f, IW * f
    i = torch.arange(IH, dtype=torch.float64).view(-1, 1, 1)
    j = torch.arange(IW, dtype=torch.float64).view(1, -1, 1)
    offs = torch.arange(-1, 2, dtype=torch.float64)
    dy, dx = torch.meshgrid(offs, offs, indexing='ij')
    x_ = (j * f + 1 + dx.reshape(1, 1, -1) * 1.25 + 0 * i)
    y_ = (i * f + 1 + dy.reshape(1, 1, -1) * 1.25 + 0 * j)
    smap = torch.stack([x_, y_], -1).float().contiguous()
    x = torch.randn(B, Ci, IH, IW, generator=g)
    w = torch.randn(Ci, Co, K, generator=g) / (Ci * K) ** 0.5
    b = torch.randn(Co, generator=g)
    gy = torch.randn(B, Co, OH, OW, generator=g)
    y_o = O.mapped_transposed_conv_forward(x, smap, w, b, OH, OW, K, interp)
    g_o = O.mapped_transposed_conv_backward(gy, smap, x, w, b, K, interp)
    for dtype in (torch.float32, torch.bfloat16):
        c = lambda t: t.to(dtype).cuda()
        if dtype == torch.bfloat16:
            y_o = O.mapped_transposed_conv_forward(x.bfloat16().float(), smap, w.bfloat16().float(),
                                                   b.bfloat16().float(), OH, OW, K, interp)
            g_o = O.mapped_transposed_conv_backward(gy.bfloat16().float(), smap,
                                                    x.bfloat16().float(), w.bfloat16().float(),
                                                    b.bfloat16().float(), K, interp)
        y = _C.mapped_transposed_conv_forward(c(x), smap.cuda(), c(w), c(b), OH, OW, K, interp)
        gr = _C.mapped_transposed_conv_backward(c(gy), smap.cuda(), c(x), c(w), c(b), K, interp)
        assert rel_err(y.float(), y_o) < TOL[dtype]
        for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
            assert rel_err(a.float(), r) < TOL[dtype], nm


# ----------------------------------------------- scalar fp32 kernels, single tap, P > 4 in bf16
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("k,p", [(5, 5), (1, 0), (1, 2), (3, 6)])
def test_conv_and_tconv_fp32_many_points_or_one_tap(k, p, interp, device):
    """More than four interpolation points per tap runs the scalar fp32 kernels; K = 1 is the
    smallest tap group of the matrix-core kernels."""
    g = torch.Generator().manual_seed(1300 + 10 * k + p + interp)
    B, Ci, Co, IH, IW, OH, OW = 2, 6, 9, 9, 12, 7, 10
    x = torch.randn(B, Ci, IH, IW, generator=g)
    smap, iw = helpers.random_map(g, OH, OW, k, p, IH, IW, torch.float32)
    w = torch.randn(Co, Ci, k, generator=g)
    b = torch.randn(Co, generator=g)
    gy = torch.randn(B, Co, OH, OW, generator=g)
    y_o = O.weighted_mapped_conv_forward(x, smap, iw, w, b, k, interp)
    g_o = O.weighted_mapped_conv_backward(gy, smap, iw, x, w, b, k, interp)
    xd, sd, iwd, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    if p:
        y = _C.weighted_mapped_conv_forward(xd, sd, iwd, wd_, bd, k, interp)
        gr = _C.weighted_mapped_conv_backward(gyd, sd, iwd, xd, wd_, bd, k, interp)
    else:
        y = _C.mapped_conv_forward(xd, sd, wd_, bd, k, interp)
        gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, k, interp)
    assert rel_err(y, y_o) < 1e-5
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a, r) < 1e-5, nm
    # transposed: the same map read as [IH', IW'] = [OH, OW] pointing into an IH x IW output
    xt = torch.randn(B, Ci, OH, OW, generator=g)
    wt = torch.randn(Ci, Co, k, generator=g)
    gyt = torch.randn(B, Co, IH, IW, generator=g)
    t_o = O.weighted_mapped_transposed_conv_forward(xt, smap, iw, wt, b, IH, IW, k, interp)
    tg_o = O.weighted_mapped_transposed_conv_backward(gyt, smap, iw, xt, wt, b, k, interp)
    xtd, wtd, gytd = dev(xt, wt, gyt)
    if p:
        t = _C.weighted_mapped_transposed_conv_forward(xtd, sd, iwd, wtd, bd, IH, IW, k, interp)
        tg = _C.weighted_mapped_transposed_conv_backward(gytd, sd, iwd, xtd, wtd, bd, k, interp)
    else:
        t = _C.mapped_transposed_conv_forward(xtd, sd, wtd, bd, IH, IW, k, interp)
        tg = _C.mapped_transposed_conv_backward(gytd, sd, xtd, wtd, bd, k, interp)
    assert rel_err(t, t_o) < 1e-5
    for a, r, nm in zip(tg, tg_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a, r) < 1e-5, "transposed " + nm


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("with_plan", [False, True])
def test_input_gradient_with_border_rows_beyond_two_entries(with_plan, dtype, device):
    """5x5 latitude map: the clamped rows at the top and the bottom put three and more
    contributions into cells of the first and the last input row, every other row holds at most
    two per cell.  The input gradient then runs its two-entry form on the tiles whose rows are
    clear and the general form on the others, several tiles per row and per image here."""
    B, Ci, Co, H, W, K = 2, 24, 40, 24, 288, 25
    g = torch.Generator().manual_seed(77)
    cast = lambda t: t.to(dtype)
    x, gy = cast(torch.randn(B, Ci, H, W, generator=g)), cast(torch.randn(B, Co, H, W, generator=g))
    w = cast(torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5)
    b = cast(torch.randn(Co, generator=g))
    smap = synthetic.latitude_map(H, W, 2)
    # the premise: cells of the border rows receive more than two contributions, no others do
    cnt = torch.bincount(helpers.map_contributions(smap, None, H, W, 1), minlength=H * W * K)
    rows = (cnt.view(H, W * K) > 2).any(1)
    assert rows[0] and rows[-1] and not rows[2:-2].any()
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, 1)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    plan = _C.conv_map_plan(sd, None, H, W, 1, dtype) if with_plan else None
    for _ in range(2):
        gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 1, plan=plan)
        for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
            assert rel_err(a.float().cpu(), r) < TOL[dtype], nm
        assert_close_elementwise(gr[0].float().cpu(), g_o[0], TOL[dtype])


@pytest.mark.parametrize("interp", [1, 2])
@pytest.mark.parametrize("row_shift", [0.0, 0.37])
@pytest.mark.parametrize("shape", [(4, 130, 96, 40, 392, 2), (2, 72, 200, 33, 264, 1),
                                   (3, 128, 128, 16, 1024, 2)])
def test_bf16_weight_gradient_over_many_tiles_per_workgroup(shape, row_shift, interp, device):
    """bf16 storage under a latitude map, with integral rows (two pairs per tap) and with the
    rows shifted by a fraction (all four): the weight gradient's workgroups walk runs of several
    row tiles (with two pairs: their gathers in flight across tile boundaries, runs padded to a
    whole number of ring periods), ragged channel counts on both sides, rows that end inside a
    tile, 9 and 25 taps (passes of 5 + 4 and 5 x 5).  Checked against the fp32 kernels on
    the same bf16-valued inputs (themselves checked against the oracle), which differ by the
    rounding of the samples to bf16 only; the oracle itself runs on the small cases elsewhere in
    this file and on sampled positions at full size."""
    B, Co, Ci, H, W, radius = shape
    K = (2 * radius + 1) ** 2
    g = torch.Generator().manual_seed(91)
    x = torch.randn(B, Ci, H, W, generator=g).bfloat16().cuda()
    gy = torch.randn(B, Co, H, W, generator=g).bfloat16().cuda()
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).bfloat16().cuda()
    b = torch.randn(Co, generator=g).bfloat16().cuda()
    smap = synthetic.latitude_map(H, W, radius)
    smap[..., 1] = (smap[..., 1] + row_shift).clamp(0, H - 1)
    smap = smap.cuda()
    got = _C.mapped_conv_backward(gy, smap, x, w, b, K, interp)
    ref = _C.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, interp)
    for a, r, nm in zip(got, ref, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm
    assert_close_elementwise(got[1].float(), ref[1], 2e-2, "grad_weight")
    # the same bits on every call (fixed summation order)
    again = _C.mapped_conv_backward(gy, smap, x, w, b, K, interp)
    assert torch.equal(got[1], again[1]) and torch.equal(got[2], again[2])


@pytest.mark.parametrize("row_shift", [0.0, 0.37])
@pytest.mark.parametrize("radius", [1, 2])
def test_bf16_weight_gradient_over_many_tiles_against_the_oracle(radius, row_shift, device):
    """The same walk over several row tiles per workgroup, against the ORACLE: 24 x 8192 pixels
    are 1536 tiles of 128, which the 1280 (9 taps) or 512 (25 taps) pixel ranges of this channel
    split take two or three at a time (three: a run padded to a whole ring period), with ragged
    channel groups on both sides (24 of 128 plain, 40 = 32 + 8 gathered) and both forms of the
    kernel (integral rows: two pairs per tap; shifted rows: four)."""
    B, Co, Ci, H, W = 1, 24, 40, 24, 8192
    K = (2 * radius + 1) ** 2
    g = torch.Generator().manual_seed(191 + radius)
    bf = lambda t: t.to(torch.bfloat16)
    x, gy = bf(torch.randn(B, Ci, H, W, generator=g)), bf(torch.randn(B, Co, H, W, generator=g))
    w = bf(torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5)
    b = bf(torch.randn(Co, generator=g))
    smap = synthetic.latitude_map(H, W, radius)
    smap[..., 1] = (smap[..., 1] + row_shift).clamp(0, H - 1)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, 1)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 1)
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm
    assert_close_elementwise(gr[1].float(), g_o[1], 2e-2, "grad_weight")


@pytest.mark.parametrize("interp", [1, 2])
@pytest.mark.parametrize("with_plan", [False, True])
def test_bf16_transposed_conv_under_a_map_with_integral_rows(with_plan, interp, device):
    """Transposed convolution, bf16 storage, latitude map: its weight gradient (plain operand the
    input, gathered operand grad_output) takes the same bf16 kernel as the convolution's, and
    its input gradient the two-pair gather-product."""
    B, Ci, Co, H, W, K = 2, 20, 36, 12, 136, 9
    g = torch.Generator().manual_seed(123 + interp)
    bf = lambda t: t.to(torch.bfloat16)
    x, gy = bf(torch.randn(B, Ci, H, W, generator=g)), bf(torch.randn(B, Co, H, W, generator=g))
    w = bf(torch.randn(Ci, Co, K, generator=g) / (Ci * K) ** 0.5)
    b = bf(torch.randn(Co, generator=g))
    smap = synthetic.latitude_map(H, W, 1)
    y_o = O.mapped_transposed_conv_forward(x.float(), smap, w.float(), b.float(), H, W, K, interp)
    g_o = O.mapped_transposed_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K,
                                            interp)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    plan = _C.conv_map_plan(sd, None, H, W, interp, torch.bfloat16) if with_plan else None
    y = _C.mapped_transposed_conv_forward(xd, sd, wd_, bd, H, W, K, interp, plan=plan)
    gr = _C.mapped_transposed_conv_backward(gyd, sd, xd, wd_, bd, K, interp, plan=plan)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm
    assert_close_elementwise(gr[1].float(), g_o[1], 2e-2, "grad_weight")


@pytest.mark.parametrize("interp", [1, 2])
@pytest.mark.parametrize("radius", [1, 2])
def test_bf16_backward_under_a_map_with_fractional_rows(radius, interp, device):
    """bf16 storage, rows of the latitude map shifted by a fraction so that all four corners of
    every tap weigh something, image rows a multiple of 8 pixels: the weight gradient's
    four-pair form on the 8-channel block copy, against the oracle."""
    B, Ci, Co, H, W = 2, 24, 40, 14, 136
    K = (2 * radius + 1) ** 2
    g = torch.Generator().manual_seed(321 + radius)
    bf = lambda t: t.to(torch.bfloat16)
    x, gy = bf(torch.randn(B, Ci, H, W, generator=g)), bf(torch.randn(B, Co, H, W, generator=g))
    w = bf(torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5)
    b = bf(torch.randn(Co, generator=g))
    smap = synthetic.latitude_map(H, W, radius)
    smap[..., 1] = (smap[..., 1] + 0.37).clamp(0, H - 1)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, interp)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, interp)
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm
    assert_close_elementwise(gr[1].float(), g_o[1], 2e-2, "grad_weight")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("row_shift", [0.0, 0.37])
def test_weight_gradient_with_staged_operands_over_ragged_channel_groups(row_shift, dtype, device):
    """More plain channels than one workgroup takes (136 = 128 + 8: the second group's staged
    fragments end after one slab), gathered channels that do not fill their last group, 25 taps
    (three passes over a resolved-tap table, the last one short) and image sizes that leave
    ragged pixel tiles, with integral map rows (two-pair forms, which read the tap tables) and
    with fractional ones (four-pair forms): all three gradients against the oracle."""
    B, Ci, Co, H, W, radius = 2, 40, 136, 14, 136, 2
    K = (2 * radius + 1) ** 2
    g = torch.Generator().manual_seed(99)
    cast = lambda t: t.to(dtype)
    x, gy = cast(torch.randn(B, Ci, H, W, generator=g)), cast(torch.randn(B, Co, H, W, generator=g))
    w = cast(torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5)
    b = cast(torch.randn(Co, generator=g))
    smap = synthetic.latitude_map(H, W, radius)
    if row_shift:
        smap[..., 1] = (smap[..., 1] + row_shift).clamp(0, H - 1)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, 1)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 1)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm
    assert_close_elementwise(gr[1].float(), g_o[1], tol, "grad_weight")


@pytest.mark.parametrize("row_shift", [0.0, 0.5])
@pytest.mark.parametrize("shape", [(1, 3, 5, 6, 16), (2, 1, 2, 3, 8), (1, 9, 17, 5, 264)])
def test_bf16_backward_with_very_few_channels(shape, row_shift, device):
    """bf16 storage, rows a multiple of 8 pixels, fewer channels than one 8-channel block or one
    MFMA tile on either side, images of a few rows: the block copy's padding channels and the
    workgroups' idle channel groups must add nothing.  Against the oracle."""
    B, Ci, Co, H, W = shape
    K = 9
    g = torch.Generator().manual_seed(7 + Ci)
    bf = lambda t: t.to(torch.bfloat16)
    x, gy = bf(torch.randn(B, Ci, H, W, generator=g)), bf(torch.randn(B, Co, H, W, generator=g))
    w = bf(torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5)
    b = bf(torch.randn(Co, generator=g))
    smap = synthetic.latitude_map(H, W, 1)
    smap[..., 1] = (smap[..., 1] + row_shift).clamp(0, H - 1)
    y_o = O.mapped_conv_forward(x.float(), smap, w.float(), b.float(), K, 1)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, 1)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    y = _C.mapped_conv_forward(xd, sd, wd_, bd, K, 1)
    gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 1)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


def test_bf16_with_more_than_four_points_is_rejected(device):
    """bf16 storage exists on the matrix-core kernels only, which take at most four points."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, 4, 5, 6, generator=g).bfloat16().cuda()
    smap, iw = helpers.random_map(g, 5, 6, 3, 5, 5, 6, torch.float32)
    w = torch.randn(8, 4, 3, generator=g).bfloat16().cuda()
    b = torch.zeros(8).bfloat16().cuda()
    with pytest.raises(RuntimeError, match="dtype"):
        _C.weighted_mapped_conv_forward(x, smap.cuda(), iw.cuda(), w, b, 3, 1)
    gy = torch.randn(1, 8, 5, 6, generator=g).bfloat16().cuda()
    with pytest.raises(RuntimeError, match="dtype"):
        _C.weighted_mapped_conv_backward(gy, smap.cuda(), iw.cuda(), x, w, b, 3, 1)


# --------------------------------------- reference known answers through the matrix-core kernels
def _layer_for(case):
    k, ci, co = KNOWN["kernel_size"], KNOWN["in_channels"], KNOWN["out_channels"]
    op, interp = case["op"], case["interpolation"]
    if op == "conv":
        return nn.MappedConvolution(ci, co, k, interpolation=interp)
    if op == "tconv":
        return nn.MappedTransposedConvolution(ci, co, k, interpolation=interp)
    if op == "max_pool":
        return nn.MappedMaxPool(k, interpolation=interp)
    if op == "avg_pool":
        return nn.MappedAvgPool(k, interpolation=interp)
    return nn.Unresample(interp)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(CASES))
def test_known_answers_through_fp32_and_bf16_kernels(name, dtype, device):
    """The reference's hand-computed cases (Ci=2, Co=3, K=4 on 4x5 images: every tile ragged)
    in the storage types the matrix-core kernels serve.  Inputs and expected values are small
    integers and quarters, exact in fp32; bf16 keeps 8 bits of the outputs."""
    case = CASES[name]
    if dtype == torch.bfloat16 and case["op"] not in ("conv", "tconv"):
        pytest.skip("bf16 storage exists for the convolutions only")
    x, smap, iw, exp = helpers.case_tensors(case, torch.float32)
    x = x.to(dtype).cuda().requires_grad_(True)
    smap, iw = dev(smap, iw)
    layer = _layer_for(case).to(device)
    if case["op"] in ("conv", "tconv"):
        w, b = helpers.case_weights(case, torch.float32)
        layer.weight.data, layer.bias.data = w.cuda(), b.cuda()
    layer = layer.to(dtype)
    if case["op"] == "tconv":
        oh, ow = case["output_shape"]
        out = layer(x, oh, ow, smap, iw)
    else:
        out = layer(x, smap, iw)
    assert out.dtype == dtype
    want = exp.expand_as(out)
    if dtype == torch.float32:
        torch.testing.assert_close(out.float().cpu(), want, rtol=1e-5, atol=1e-5)
    else:
        torch.testing.assert_close(out.float().cpu(), want, rtol=2e-2, atol=2e-2)
    gout = torch.arange(out.numel(), dtype=torch.float32).view(out.shape).remainder(7).sub(3)
    out.backward(gout.to(dtype).cuda())
    # every gradient against the oracle's backward of the same case (the reference runs
    # gradcheck on these cases, package/tests/utils.py:63-96; gout holds small integers so that
    # the bf16 inputs of the backward are exact too)
    xf, sm, iwc = x.detach().float().cpu(), smap.cpu(), None if iw is None else iw.cpu()
    k, interp = KNOWN["kernel_size"], helpers.INTERP[case["interpolation"]]
    tol = TOL[dtype]
    op = case["op"]
    if op in ("conv", "tconv"):
        if op == "conv":
            want = O.weighted_mapped_conv_backward(gout, sm, iwc, xf, w, b, k, interp)
        else:
            want = O.weighted_mapped_transposed_conv_backward(gout, sm, iwc, xf, w, b, k, interp)
        got = (x.grad, layer.weight.grad, layer.bias.grad)
        for a, r, nm in zip(got, want, ("grad_input", "grad_weight", "grad_bias")):
            assert a is not None and a.dtype == dtype
            assert rel_err(a.float(), r) < tol, nm
            assert_close_elementwise(a.float(), r, 2 * tol, nm)
    else:
        H, W = xf.shape[2:]
        if op == "max_pool":
            _, idx = O.weighted_mapped_max_pool(xf, sm, iwc, k, interp)
            want = O.weighted_mapped_max_unpool(gout, idx, sm, iwc, H, W, k, interp)
        elif op == "avg_pool":
            want = O.weighted_mapped_avg_unpool(gout, sm, iwc, H, W, k, interp)
        else:  # Unresample: the gradient of a gather is the scatter through the same map
            want = O.weighted_resample_to_map(gout, sm, iwc, H, W, interp)
        assert rel_err(x.grad.float(), want) < tol, "grad_input"
        assert_close_elementwise(x.grad.float(), want, 2 * tol, "grad_input")


# ------------------------------------------------------------ full-size configurations 3 and 5
def _sampled_conv_check(x, w, b, smap, iw, K, interp, picks, images, tol, seed):
    """Full-size forward and backward on the GPU against the oracle evaluated on `picks`
    (flat output-pixel indices) of `images` only.

    Forward: the oracle runs on a map holding just the picked pixels' taps.  Backward: the
    GPU gets a grad_output that is zero except at the picked pixels of the chosen images, so
    that grad_input / grad_weight / grad_bias equal the oracle's on that sub-problem."""
    B, Ci = x.shape[:2]
    Co = w.shape[0]
    OH, OW = smap.shape[:2]
    N = OH * OW
    sub_map = smap.reshape((N,) + tuple(smap.shape[2:]))[picks].unsqueeze(0).contiguous().cpu()
    sub_iw = None if iw is None else \
        iw.reshape((N,) + tuple(iw.shape[2:]))[picks].unsqueeze(0).contiguous().cpu()
    x_sub = x[images].float().cpu()
    wf, bf = w.float().cpu(), b.float().cpu()
    y = _C.weighted_mapped_conv_forward(x, smap, iw, w, b, K, interp) if iw is not None else \
        _C.mapped_conv_forward(x, smap, w, b, K, interp)
    y_o = O.weighted_mapped_conv_forward(x_sub, sub_map, sub_iw, wf, bf, K, interp)
    got = y.view(B, Co, N)[images][:, :, picks.to(y.device)].float().cpu()
    assert rel_err(got, y_o[:, :, 0, :]) < tol, "forward at sampled positions"
    assert_close_elementwise(got, y_o[:, :, 0, :], 4 * tol, "forward at sampled positions")

    g = torch.Generator().manual_seed(seed)
    g_sub = torch.randn(len(images), Co, 1, len(picks), generator=g).to(x.dtype)
    gy = torch.zeros(B, Co, N, dtype=x.dtype, device=x.device)
    gy[torch.tensor(images, device=x.device)[:, None, None],
       torch.arange(Co, device=x.device)[None, :, None],
       picks.to(x.device)[None, None, :]] = g_sub[:, :, 0, :].to(x.device)
    gy = gy.view(B, Co, OH, OW)
    if iw is not None:
        gx, gw, gb = _C.weighted_mapped_conv_backward(gy, smap, iw, x, w, b, K, interp)
    else:
        gx, gw, gb = _C.mapped_conv_backward(gy, smap, x, w, b, K, interp)
    gx_o, gw_o, gb_o = O.weighted_mapped_conv_backward(g_sub.float(), sub_map, sub_iw, x_sub, wf,
                                                       bf, K, interp)
    assert rel_err(gx[images].float(), gx_o) < tol, "grad_input"
    others = [i for i in range(B) if i not in images]
    if others:
        assert gx[others].float().abs().max().item() == 0, "images without gradient stay zero"
    assert rel_err(gw.float(), gw_o) < tol, "grad_weight"
    assert rel_err(gb.float(), gb_o) < tol, "grad_bias"
    return y


def _dense_properties(x, w, b, smap, iw, K, interp, y, tol, seed):
    """Adjointness of forward and input gradient, the weight gradient as the derivative of
    <conv(x), g> along a random direction, the bias gradient as the plain sum."""
    torch.manual_seed(seed)
    fwd = (lambda x_, w_, b_: _C.weighted_mapped_conv_forward(x_, smap, iw, w_, b_, K, interp)) \
        if iw is not None else (lambda x_, w_, b_: _C.mapped_conv_forward(x_, smap, w_, b_, K, interp))
    gy = torch.randn(y.shape, device=x.device, dtype=torch.float32).to(x.dtype)
    if iw is not None:
        gx, gw, gb = _C.weighted_mapped_conv_backward(gy, smap, iw, x, w, b, K, interp)
    else:
        gx, gw, gb = _C.mapped_conv_backward(gy, smap, x, w, b, K, interp)
    zero = torch.zeros_like(b)
    y0 = fwd(x, w, zero)

    def dot(a, c):
        return sum((a[i].double() * c[i].double()).sum() for i in range(a.shape[0]))

    def scale(a, c):  # size of a sum of len(a) terms of random sign
        return sum((a[i].double() * c[i].double()).pow(2).sum() for i in range(a.shape[0])).sqrt()

    lhs, rhs = dot(y0, gy), dot(x, gx)
    assert abs(lhs - rhs) <= 40 * tol * scale(y0, gy), "adjointness"
    dw = torch.randn(w.shape, device=x.device).to(x.dtype)
    y2 = fwd(x, dw, zero)
    lhs, rhs = dot(y2, gy), (gw.double() * dw.double()).sum()
    assert abs(lhs - rhs) <= 40 * tol * scale(y2, gy), "weight gradient along a direction"
    want_gb = sum(gy[i].double().sum((1, 2)) for i in range(gy.shape[0]))
    assert rel_err(gb.float(), want_gb) < tol, "bias gradient"


def _picks(OH, OW, count, seed):
    """Flat pixel indices: the four corners, the seam columns, the pole rows and random ones."""
    g = torch.Generator().manual_seed(seed)
    n = OH * OW
    fixed = [0, OW - 1, n - OW, n - 1, OW, 2 * OW - 1, (OH // 2) * OW, (OH // 2) * OW + OW - 1]
    rnd = torch.randperm(n, generator=g)[:count].tolist()
    return torch.tensor(sorted(set(p for p in fixed + rnd if p < n)), dtype=torch.int64)


def test_config5_full_size_weight_gradient_two_ways(device):
    """Configuration 5 at full size, weight gradient element by element: the fast form (staged
    operands, tap table, 5 120 workgroups, images beyond 2^31 bytes) against the general kernel,
    which the same call takes when grad_output is not 16-byte aligned.  The two differ in where
    they round (bf16 interpolation weights in the fast form) and in the order of their fp32
    sums, nothing else."""
    B, C, H, W, K = 16, 128, 512, 1024, 25
    smap = synthetic.latitude_map(H, W, 2).cuda()
    torch.manual_seed(58)
    x = torch.randn(B, C, H, W, device=device, dtype=torch.bfloat16)
    w = (torch.randn(C, C, K, device=device) / (C * K) ** 0.5).bfloat16()
    b = torch.zeros(C, device=device, dtype=torch.bfloat16)
    n = B * C * H * W
    buf = torch.empty(n + 8, device=device, dtype=torch.bfloat16)
    buf[:n].copy_(torch.randn(n // 64, device=device).bfloat16().repeat(64))
    gy = buf[:n].view(B, C, H, W)
    assert gy.data_ptr() % 16 == 0
    needs = (False, True, True)
    _, gw_fast, gb_fast = _C.mapped_conv_backward(gy, smap, x, w, b, K, 1, needs=needs)
    buf[1:n + 1].copy_(buf[:n].clone())
    gy_off = buf[1:n + 1].view(B, C, H, W)
    assert gy_off.data_ptr() % 16 != 0 and gy_off.is_contiguous()
    _, gw_gen, gb_gen = _C.mapped_conv_backward(gy_off, smap, x, w, b, K, 1, needs=needs)
    assert rel_err(gw_fast.float(), gw_gen.float()) < 2e-2
    assert_close_elementwise(gw_fast.float(), gw_gen.float(), 2e-2, "grad_weight")
    assert rel_err(gb_fast.float(), gb_gen.float()) < 2e-2


@pytest.mark.parametrize("interp", [0, 1])
def test_config2_full_size(interp, device):
    """The headline shape: B=8, 64 -> 64 channels, 256 x 512, 3 x 3 latitude map, fp32, nearest
    and bilinear: forward and all three gradients at 2 048 sampled output pixels (corners,
    seam columns, pole rows, random ones) of the first and the last image against the oracle."""
    B, C, H, W, K = 8, 64, 256, 512, 9
    smap = synthetic.latitude_map(H, W, 1).cuda()
    torch.manual_seed(22 + interp)
    x = torch.randn(B, C, H, W, device=device)
    w = torch.randn(C, C, K, device=device) / (C * K) ** 0.5
    b = torch.randn(C, device=device)
    y = _sampled_conv_check(x, w, b, smap, None, K, interp, _picks(H, W, 2040, 2), [0, B - 1],
                            1e-5, 23)
    _dense_properties(x, w, b, smap, None, K, interp, y, 1e-5, 24)


def test_layers_skip_the_gradients_nobody_asks_for(device):
    """A layer whose input needs no gradient (a network's first layer) or whose parameters are
    frozen gets None for those gradients from the op and the right values for the others;
    cache_plan=True layers build one plan per map and give the same results."""
    g = torch.Generator().manual_seed(808)
    B, Ci, Co, H, W, K = 2, 12, 20, 10, 40, 9
    smap = synthetic.latitude_map(H, W, 1).cuda()
    x = torch.randn(B, Ci, H, W, generator=g).cuda()
    gy = torch.randn(B, Co, H, W, generator=g).cuda()
    for make in (lambda **kw: nn.MappedConvolution(Ci, Co, K, **kw),
                 lambda **kw: nn.MappedTransposedConvolution(Ci, Co, K, **kw)):
        layer = make().cuda()
        call = (lambda l, inp: l(inp, smap)) if isinstance(layer, nn.MappedConvolution) else \
            (lambda l, inp: l(inp, H, W, smap))
        xr = x.clone().requires_grad_(True)
        call(layer, xr).backward(gy)
        full = (xr.grad.clone(), layer.weight.grad.clone(), layer.bias.grad.clone())
        # first layer: no input gradient
        layer.zero_grad()
        call(layer, x).backward(gy)
        assert torch.equal(layer.weight.grad, full[1]) and torch.equal(layer.bias.grad, full[2])
        # frozen parameters: the input gradient alone
        layer.zero_grad()
        layer.weight.requires_grad_(False)
        layer.bias.requires_grad_(False)
        xr = x.clone().requires_grad_(True)
        call(layer, xr).backward(gy)
        # (the slots of a transposed-map cell are handed out in the order the builder's atomics
        # land, so the input gradient's additions may be reordered from call to call)
        assert rel_err(xr.grad, full[0]) < 1e-6 and layer.weight.grad is None
        # the op itself
        bwd = _C.mapped_conv_backward if isinstance(layer, nn.MappedConvolution) else \
            _C.mapped_transposed_conv_backward
        got = bwd(gy, smap, x, layer.weight.data, layer.bias.data, K, 1,
                  needs=(False, True, False))
        assert got[0] is None and got[2] is None and torch.equal(got[1], full[1])
        got = bwd(gy, smap, x, layer.weight.data, layer.bias.data, K, 1,
                  needs=(False, False, True))
        assert got[0] is None and got[1] is None and rel_err(got[2], full[2]) < 1e-6
        # a layer that owns its plan
        owner = make(cache_plan=True).cuda()
        owner.load_state_dict(layer.state_dict())
        xr = x.clone().requires_grad_(True)
        for _ in range(2):
            owner.zero_grad()
            xr.grad = None
            call(owner, xr).backward(gy)
        first_plan = owner._plan.plan
        assert first_plan is not None
        for a, r in zip((xr.grad, owner.weight.grad, owner.bias.grad), full):
            assert rel_err(a, r) < 1e-5
        smap2 = (smap + 0.5).contiguous()    # another map: the layer builds another plan
        call(owner, x)
        assert owner._plan.plan is first_plan
        if isinstance(owner, nn.MappedConvolution):
            owner(x, smap2)
        else:
            owner(x, H, W, smap2)
        assert owner._plan.plan is not first_plan


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_config3_full_size(dtype, device):
    """B=4, 64 -> 128 channels, V=40962 vertices, K=7 taps x P=4 points, nearest."""
    B, Ci, Co, V, K, P = 4, 64, 128, 40962, 7, 4
    smap, iw = synthetic.mesh_weighted_map(V, K, P, seed=3)
    g = torch.Generator().manual_seed(33)
    x = torch.randn(B, Ci, 1, V, generator=g).to(dtype).cuda()
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dtype).cuda()
    b = torch.randn(Co, generator=g).to(dtype).cuda()
    tol = TOL[dtype]
    y = _sampled_conv_check(x, w, b, smap.cuda(), iw.cuda(), K, 0, _picks(1, V, 2048, 3), [0, 3],
                            tol, 34)
    _dense_properties(x, w, b, smap.cuda(), iw.cuda(), K, 0, y, tol, 35)


def test_config5_full_size_bf16(device):
    """B=16, 128 -> 128 channels, 512x1024, 5x5 latitude map, bilinear, bf16 storage: tensors
    of 2 GiB whose last image lies beyond 2^31 bytes."""
    B, C, H, W, K = 16, 128, 512, 1024, 25
    smap = synthetic.latitude_map(H, W, 2).cuda()
    torch.manual_seed(55)
    x = torch.randn(B, C, H, W, device=device, dtype=torch.bfloat16)
    w = (torch.randn(C, C, K, device=device) / (C * K) ** 0.5).bfloat16()
    b = torch.randn(C, device=device).bfloat16()
    y = _sampled_conv_check(x, w, b, smap, None, K, 1, _picks(H, W, 1016, 5), [0, B - 1], 2e-2, 56)
    _dense_properties(x, w, b, smap, None, K, 1, y, 2e-2, 57)
    del y
    # the regular 5x5 grid map turns the op into a zero-padded convolution: library routine
    # on the first and the last image
    grid = synthetic.identity_grid_map(H, W, 2).cuda()
    yg = _C.mapped_conv_forward(x, grid, w, b, K, 1)
    for i in (0, B - 1):
        ref = F.conv2d(x[i:i + 1].float(), w.float().view(C, C, 5, 5), b.float(), padding=2)
        assert rel_err(yg[i:i + 1].float(), ref) < 2e-2
