"""GPU parity tests (run on the MI355X box): every op of the HIP boundary against
the CPU oracle on the same seeded inputs, the reference's known answers and
gradcheck through the layers (float64, as the reference's *_cuda tests do), and
size-independent properties at larger shapes.

Bars: gathers (resample_from_map, pools) are bit-exact against the oracle in
every interpolation mode for fp32/fp64, max-pool argmax and KNN indices are
bit-exact; scatters and convolutions (atomic / blocked accumulation order) agree
within 1e-5 of the result's magnitude in fp32 and 1e-12 in fp64."""
import pytest
import torch
import torch.nn.functional as F
from torch.autograd import gradcheck

import helpers
from helpers import CASES, KNOWN, INTERP, rel_err
from oracle import ops as O

from mappedconvolutions_amd import _C, nn
from mappedconvolutions_amd.util import knn, synthetic

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float64]
TOL = {torch.float32: 1e-5, torch.float64: 1e-12}


def dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


# ------------------------------------------------- reference known answers + gradcheck
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


@pytest.mark.parametrize("name", sorted(CASES))
def test_known_answers_and_gradcheck_through_layers(name, device):
    case = CASES[name]
    x, smap, iw, exp = helpers.case_tensors(case)
    x, smap, iw = dev(x, smap, iw)
    x.requires_grad_(True)
    layer = _layer_for(case).double().to(device)
    if case["op"] in ("conv", "tconv"):
        w, b = helpers.case_weights(case)
        layer.weight.data, layer.bias.data = w.cuda(), b.cuda()
    if case["op"] == "tconv":
        oh, ow = case["output_shape"]
        args = (x, oh, ow, smap, iw)
    else:
        args = (x, smap, iw)
    out = layer(*args)
    torch.testing.assert_close(out.cpu(), exp.expand_as(out), rtol=1e-9, atol=1e-9)
    out.backward(torch.ones_like(out))
    assert gradcheck(layer, args)


# ------------------------------------------------------------------ op-level parity
def _conv_problem(dtype, seed, p, B=2, Ci=5, Co=7, IH=9, IW=11, OH=6, OW=10, K=5):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, Ci, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, wts = helpers.random_map(g, OH, OW, K, p, IH, IW, dtype)
    w = torch.randn(Co, Ci, K, generator=g, dtype=torch.float64).to(dtype)
    b = torch.randn(Co, generator=g, dtype=torch.float64).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    return x, smap, wts, w, b, gy, K


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_conv_forward_backward(dtype, interp, p, device):
    x, smap, wts, w, b, gy, K = _conv_problem(dtype, 100 + interp + 10 * p, p)
    y_o = O.weighted_mapped_conv_forward(x, smap, wts, w, b, K, interp)
    g_o = O.weighted_mapped_conv_backward(gy, smap, wts, x, w, b, K, interp)
    xd, sd, wd_, wgt, bd, gyd = dev(x, smap, wts, w, b, gy)
    if p:
        y = _C.weighted_mapped_conv_forward(xd, sd, wd_, wgt, bd, K, interp)
        g = _C.weighted_mapped_conv_backward(gyd, sd, wd_, xd, wgt, bd, K, interp)
    else:
        y = _C.mapped_conv_forward(xd, sd, wgt, bd, K, interp)
        g = _C.mapped_conv_backward(gyd, sd, xd, wgt, bd, K, interp)
    assert rel_err(y, y_o) < TOL[dtype]
    for a, r, nm in zip(g, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a, r) < TOL[dtype], nm


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_transposed_conv_forward_backward(dtype, interp, p, device):
    g = torch.Generator().manual_seed(200 + interp + 10 * p)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 5, 6, 6, 7, 9, 12, 4
    x = torch.randn(B, Ci, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, wts = helpers.random_map(g, IH, IW, K, p, OH, OW, dtype)
    w = torch.randn(Ci, Co, K, generator=g, dtype=torch.float64).to(dtype)
    b = torch.randn(Co, generator=g, dtype=torch.float64).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    y_o = O.weighted_mapped_transposed_conv_forward(x, smap, wts, w, b, OH, OW, K, interp)
    g_o = O.weighted_mapped_transposed_conv_backward(gy, smap, wts, x, w, b, K, interp)
    xd, sd, wd_, wgt, bd, gyd = dev(x, smap, wts, w, b, gy)
    if p:
        y = _C.weighted_mapped_transposed_conv_forward(xd, sd, wd_, wgt, bd, OH, OW, K, interp)
        gr = _C.weighted_mapped_transposed_conv_backward(gyd, sd, wd_, xd, wgt, bd, K, interp)
    else:
        y = _C.mapped_transposed_conv_forward(xd, sd, wgt, bd, OH, OW, K, interp)
        gr = _C.mapped_transposed_conv_backward(gyd, sd, xd, wgt, bd, K, interp)
    assert rel_err(y, y_o) < TOL[dtype]
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a, r) < TOL[dtype], nm


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("form", ["gather", "atomic"])
def test_pools(dtype, interp, p, half, form, device, monkeypatch):
    monkeypatch.setattr(_C, "scatter_as_gather", form == "gather")
    g = torch.Generator().manual_seed(300 + interp + 10 * p)
    B, C, IH, IW, OH, OW, K = 2, 11, 9, 13, 7, 9, 5   # C=11: a ragged channel chunk
    x = torch.randn(B, C, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, wts = helpers.random_map(g, OH, OW, K, p, IH, IW, dtype, half=half)
    gy = torch.randn(B, C, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    xd, sd, wd_, gyd = dev(x, smap, wts, gy)
    mo, mi = O.weighted_mapped_max_pool(x, smap, wts, K, interp)
    ao = O.weighted_mapped_avg_pool(x, smap, wts, K, interp)
    if p:
        m, i = _C.weighted_mapped_max_pool(xd, sd, wd_, K, interp)
        a = _C.weighted_mapped_avg_pool(xd, sd, wd_, K, interp)
        mu = _C.weighted_mapped_max_unpool(gyd, i, sd, wd_, IH, IW, K, interp)
        au = _C.weighted_mapped_avg_unpool(gyd, sd, wd_, IH, IW, K, interp)
    else:
        m, i = _C.mapped_max_pool(xd, sd, K, interp)
        a = _C.mapped_avg_pool(xd, sd, K, interp)
        mu = _C.mapped_max_unpool(gyd, i, sd, IH, IW, K, interp)
        au = _C.mapped_avg_unpool(gyd, sd, IH, IW, K, interp)
    assert torch.equal(m.cpu(), mo), "max-pool values must be bit-exact"
    assert torch.equal(i.cpu(), mi), "max-pool argmax must be bit-exact"
    assert torch.equal(a.cpu(), ao), "avg-pool gather must be bit-exact"
    muo = O.weighted_mapped_max_unpool(gy, mi, smap, wts, IH, IW, K, interp)
    auo = O.weighted_mapped_avg_unpool(gy, smap, wts, IH, IW, K, interp)
    assert rel_err(mu, muo) < TOL[dtype]
    assert rel_err(au, auo) < TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 4])
@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("form", ["gather", "atomic"])
def test_resample(dtype, interp, p, half, form, device, monkeypatch):
    monkeypatch.setattr(_C, "scatter_as_gather", form == "gather")
    g = torch.Generator().manual_seed(400 + interp + 10 * p)
    B, C, IH, IW, OH, OW = 2, 9, 10, 12, 8, 15
    x = torch.randn(B, C, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, wts = helpers.random_map(g, IH, IW, 1, p, OH, OW, dtype, half=half)
    smap = smap[:, :, 0].contiguous()
    wts = None if wts is None else wts[:, :, 0].contiguous()
    y = torch.randn(B, C, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    xd, sd, wd_, yd = dev(x, smap, wts, y)
    to_o = O.weighted_resample_to_map(x, smap, wts, OH, OW, interp)
    fr_o = O.weighted_resample_from_map(y, smap, wts, interp)
    if p:
        to = _C.weighted_resample_to_map(xd, sd, wd_, OH, OW, interp)
        fr = _C.weighted_resample_from_map(yd, sd, wd_, interp)
    else:
        to = _C.resample_to_map(xd, sd, OH, OW, interp)
        fr = _C.resample_from_map(yd, sd, interp)
    assert torch.equal(fr.cpu(), fr_o), "gather must be bit-exact"
    assert rel_err(to, to_o) < TOL[dtype]


def test_empty_and_degenerate_inputs(device):
    """Taps that all fall outside give zeros / -FLT_MAX with index -1; 1x1 images work."""
    x = torch.rand(1, 2, 3, 3, device=device) + 1
    far = torch.full((2, 2, 3, 2), 100.0, device=device)
    assert _C.mapped_avg_pool(x, far, 3, 1).abs().sum() == 0
    m, i = _C.mapped_max_pool(x, far, 3, 1)
    # the zero of the padding beats -FLT_MAX at tap 0 of every pixel: offset n * K * 2
    assert (m == 0).all() and i[0, 0].flatten().tolist() == [0, 6, 12, 18]
    g = torch.ones(1, 2, 2, 2, device=device)
    assert _C.mapped_max_unpool(g, i, far, 3, 3, 3, 1).abs().sum() == 0
    neg = torch.full((1, 2, 2, 2), -1, device=device, dtype=torch.int64)
    assert _C.mapped_max_unpool(g, neg, far, 3, 3, 3, 1).abs().sum() == 0
    one = torch.rand(1, 1, 1, 1, device=device)
    sm = torch.zeros(1, 1, 2, device=device)
    assert torch.equal(_C.resample_from_map(one, sm, 0), one)


# ------------------------------------------------------------- BASELINE config 1
def test_config1_forward_fp32(device):
    """B=1, 16->32, 64x128, 3x3 latitude map, bilinear, Kaiming weights, bias 0."""
    torch.manual_seed(0)
    x = torch.rand(1, 16, 64, 128) * 2 - 1
    w = torch.randn(32, 16, 9) * (2.0 / (16 * 9)) ** 0.5
    b = torch.zeros(32)
    smap = synthetic.latitude_map(64, 128, 1)
    ref = O.mapped_conv_forward(x, smap, w, b, 9, 1)
    out = _C.mapped_conv_forward(*dev(x, smap, w, b), 9, 1)
    assert rel_err(out, ref) < 1e-5


@pytest.mark.parametrize("interp", [0, 1])
def test_conv_medium_fp32_vs_oracle(interp, device):
    """A config-2-shaped problem scaled to what the CPU oracle finishes in seconds
    (B=2, 64->64, 32x64, 3x3 latitude map), forward and backward."""
    torch.manual_seed(1)
    B, C, H, W = 2, 64, 32, 64
    x, gy = torch.randn(B, C, H, W), torch.randn(B, C, H, W)
    w, b = torch.randn(C, C, 9) / 24, torch.randn(C)
    smap = synthetic.latitude_map(H, W, 1)
    y_o = O.mapped_conv_forward(x, smap, w, b, 9, interp)
    g_o = O.mapped_conv_backward(gy, smap, x, w, b, 9, interp)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    y = _C.mapped_conv_forward(xd, sd, wd_, bd, 9, interp)
    g = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, 9, interp)
    assert rel_err(y, y_o) < 1e-5
    for a, r, nm in zip(g, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a, r) < 1e-5, nm


# ------------------------------------------------------------------ bf16 storage
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 4])
def test_conv_bf16_vs_fp32_oracle(interp, p, device):
    """bf16 data / weights (fp32 maps, fp32 accumulation) against the fp32 oracle fed
    the same bf16-rounded values: within 2e-2 of the result's magnitude."""
    g = torch.Generator().manual_seed(700 + interp + 10 * p)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 24, 40, 20, 36, 12, 40, 5
    bf = lambda t: t.to(torch.bfloat16)
    x = bf(torch.randn(B, Ci, IH, IW, generator=g))
    smap, wts = helpers.random_map(g, OH, OW, K, p, IH, IW, torch.float32)
    w = bf(torch.randn(Co, Ci, K, generator=g) / 8)
    b = bf(torch.randn(Co, generator=g))
    gy = bf(torch.randn(B, Co, OH, OW, generator=g))
    y_o = O.weighted_mapped_conv_forward(x.float(), smap, wts, w.float(), b.float(), K, interp)
    g_o = O.weighted_mapped_conv_backward(gy.float(), smap, wts, x.float(), w.float(), b.float(),
                                          K, interp)
    xd, sd, wd_, wgt, bd, gyd = dev(x, smap, wts, w, b, gy)
    if p:
        y = _C.weighted_mapped_conv_forward(xd, sd, wd_, wgt, bd, K, interp)
        gr = _C.weighted_mapped_conv_backward(gyd, sd, wd_, xd, wgt, bd, K, interp)
    else:
        y = _C.mapped_conv_forward(xd, sd, wgt, bd, K, interp)
        gr = _C.mapped_conv_backward(gyd, sd, xd, wgt, bd, K, interp)
    assert y.dtype == torch.bfloat16 and all(t.dtype == torch.bfloat16 for t in gr)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


@pytest.mark.parametrize("interp", [0, 1])
def test_conv_bf16_two_leading_pairs(interp, device):
    """Maps that use only the first two (offset, weight) pairs of a tap take the weight
    gradient's reduced variant: nearest with P=4 whose last two interp weights are zero, and
    bilinear with integral rows (the lower corners weigh exactly zero)."""
    g = torch.Generator().manual_seed(720 + interp)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 40, 24, 18, 44, 14, 38, 7
    bf = lambda t: t.to(torch.bfloat16)
    p = 4 if interp == 0 else 0
    smap, wts = helpers.random_map(g, OH, OW, K, p, IH, IW, torch.float32)
    if interp == 0:
        wts[..., 2:] = 0
    else:
        smap[..., 1] = smap[..., 1].round()
    x = bf(torch.randn(B, Ci, IH, IW, generator=g))
    w = bf(torch.randn(Co, Ci, K, generator=g) / 8)
    b = bf(torch.randn(Co, generator=g))
    gy = bf(torch.randn(B, Co, OH, OW, generator=g))
    if p:
        g_o = O.weighted_mapped_conv_backward(gy.float(), smap, wts, x.float(), w.float(),
                                              b.float(), K, interp)
        gr = _C.weighted_mapped_conv_backward(*dev(gy, smap, wts, x, w, b), K, interp)
    else:
        g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, interp)
        gr = _C.mapped_conv_backward(*dev(gy, smap, x, w, b), K, interp)
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


def test_transposed_conv_bf16(device):
    g = torch.Generator().manual_seed(720)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 16, 24, 10, 33, 14, 40, 4
    bf = lambda t: t.to(torch.bfloat16)
    x = bf(torch.randn(B, Ci, IH, IW, generator=g))
    smap, _ = helpers.random_map(g, IH, IW, K, 0, OH, OW, torch.float32)
    w = bf(torch.randn(Ci, Co, K, generator=g) / 8)
    b = bf(torch.randn(Co, generator=g))
    gy = bf(torch.randn(B, Co, OH, OW, generator=g))
    y_o = O.mapped_transposed_conv_forward(x.float(), smap, w.float(), b.float(), OH, OW, K, 1)
    g_o = O.mapped_transposed_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, 1)
    xd, sd, wgt, bd, gyd = dev(x, smap, w, b, gy)
    y = _C.mapped_transposed_conv_forward(xd, sd, wgt, bd, OH, OW, K, 1)
    gr = _C.mapped_transposed_conv_backward(gyd, sd, xd, wgt, bd, K, 1)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


def test_conv_bf16_latitude_map_uses_both_backward_paths(device):
    """Latitude map (transposed-map gather path of the input gradient) in bf16."""
    torch.manual_seed(5)
    B, C, H, W = 2, 32, 32, 64
    bf = lambda t: t.to(torch.bfloat16)
    x, gy = bf(torch.randn(B, C, H, W)), bf(torch.randn(B, C, H, W))
    w, b = bf(torch.randn(C, C, 9) / 17), bf(torch.randn(C))
    smap = synthetic.latitude_map(H, W, 1)
    y_o = O.mapped_conv_forward(x.float(), smap, w.float(), b.float(), 9, 1)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), 9, 1)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    y = _C.mapped_conv_forward(xd, sd, wd_, bd, 9, 1)
    gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, 9, 1)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


# ------------------------------------------------------------------ map plans
@pytest.mark.parametrize("case", ["latitude_fp32", "random_fp32", "mesh_bf16", "latitude_bf16"])
def test_conv_backward_with_map_plan(case, device):
    """A plan built once from the map (conv_map_plan) replaces the per-call build of the
    transposed map and of the pair masks: same gradients as without it, and as the oracle."""
    g = torch.Generator().manual_seed(900)
    if case == "mesh_bf16":
        B, Ci, Co, V, K, P = 2, 32, 48, 1500, 7, 4
        smap, iw = synthetic.mesh_weighted_map(V, K, P, seed=9)
        shape_in, shape_out, interp, dtype, tol = (B, Ci, 1, V), (B, Co, 1, V), 0, torch.bfloat16, 2e-2
    else:
        B, Ci, Co, H, W, K = 2, 24, 40, 24, 48, 9
        iw = None
        if case.startswith("latitude"):
            smap = synthetic.latitude_map(H, W, 1)
        else:
            smap, _ = helpers.random_map(g, H, W, K, 0, H, W, torch.float32)
        shape_in, shape_out, interp, dtype, tol = (B, Ci, H, W), (B, Co, H, W), 1, torch.float32, 1e-5
        if case == "latitude_bf16":  # the gathered operand goes through its channel-block copy
            dtype, tol = torch.bfloat16, 2e-2
    x = torch.randn(shape_in, generator=g).to(dtype)
    gy = torch.randn(shape_out, generator=g).to(dtype)
    w = (torch.randn(Co, Ci, K, generator=g) / 8).to(dtype)
    b = torch.randn(Co, generator=g).to(dtype)
    xd, sd, iwd, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    plan = _C.conv_map_plan(sd, iwd, shape_in[2], shape_in[3], interp, dtype)
    assert plan is not None and plan.buffer.is_cuda
    if iw is None:
        g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, interp)
        plain = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, interp)
        for _ in range(2):  # a plan is only read: it serves any number of calls
            planned = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, interp, plan=plan)
    else:
        g_o = O.weighted_mapped_conv_backward(gy.float(), smap, iw, x.float(), w.float(),
                                              b.float(), K, interp)
        plain = _C.weighted_mapped_conv_backward(gyd, sd, iwd, xd, wd_, bd, K, interp)
        for _ in range(2):
            planned = _C.weighted_mapped_conv_backward(gyd, sd, iwd, xd, wd_, bd, K, interp,
                                                       plan=plan)
    for a, p_, r, nm in zip(planned, plain, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm
        assert rel_err(a.float(), p_.float()) < tol, nm


def test_map_plan_cache_follows_in_place_changes(device):
    """With the cache on, the second backward reuses the plan of the first; changing the map
    in place bumps its version counter and the plan is rebuilt."""
    g = torch.Generator().manual_seed(901)
    B, C, H, W, K = 1, 16, 16, 32, 9
    x, gy = torch.randn(B, C, H, W, generator=g), torch.randn(B, C, H, W, generator=g)
    w, b = torch.randn(C, C, K, generator=g) / 8, torch.randn(C, generator=g)
    smap = synthetic.latitude_map(H, W, 1)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    _C.enable_map_plan_cache(True)
    try:
        for _ in range(2):
            got = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 1)
        assert len(_C.map_plan_cache) == 1
        ref = O.mapped_conv_backward(gy, smap, x, w, b, K, 1)
        for a, r in zip(got, ref):
            assert rel_err(a, r) < 1e-5
        sd[..., 0] += 0.25  # in place: same storage, new version
        smap2 = sd.cpu()
        got = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 1)
        assert len(_C.map_plan_cache) == 2
        ref = O.mapped_conv_backward(gy, smap2, x, w, b, K, 1)
        for a, r in zip(got, ref):
            assert rel_err(a, r) < 1e-5
    finally:
        _C.enable_map_plan_cache(False)
    assert _C.map_plan_cache is None


# ------------------------------------------------- BASELINE configs 3, 4, 5 (scaled)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_config3_weighted_mesh_conv(dtype, device):
    """Weighted conv on a mesh signal [B, C, 1, V]: K=7 taps x P=4 random vertices,
    Dirichlet weights, nearest.  V and channels scaled so the oracle runs in seconds."""
    B, Ci, Co, V, K, P = 2, 64, 128, 4098, 7, 4
    smap, iw = synthetic.mesh_weighted_map(V, K, P, seed=3)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(B, Ci, 1, V, generator=g).to(dtype)
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dtype)
    b = torch.randn(Co, generator=g).to(dtype)
    gy = torch.randn(B, Co, 1, V, generator=g).to(dtype)
    y_o = O.weighted_mapped_conv_forward(x.float(), smap, iw, w.float(), b.float(), K, 0)
    g_o = O.weighted_mapped_conv_backward(gy.float(), smap, iw, x.float(), w.float(), b.float(),
                                          K, 0)
    xd, sd, id_, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    y = _C.weighted_mapped_conv_forward(xd, sd, id_, wd_, bd, K, 0)
    gr = _C.weighted_mapped_conv_backward(gyd, sd, id_, xd, wd_, bd, K, 0)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert rel_err(y.float(), y_o) < tol
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", [0, 3])
def test_mesh_conv_ragged_channels(dtype, p, device):
    """Single-row (mesh) source with channel counts that are no multiple of 16 and an output
    count past one 64-channel group: the channel-last staging pads with zeros, taps outside
    [0, V) contribute nothing.  Forward, backward and the transposed convolution."""
    B, Ci, Co, V, K = 2, 20, 70, 777, 5
    g = torch.Generator().manual_seed(31 + p)
    smap, iw = helpers.random_map(g, 1, V, K, p, 1, V, torch.float32, integer=True)
    x = torch.randn(B, Ci, 1, V, generator=g).to(dtype)
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dtype)
    b = torch.randn(Co, generator=g).to(dtype)
    gy = torch.randn(B, Co, 1, V, generator=g).to(dtype)
    y_o = O.weighted_mapped_conv_forward(x.float(), smap, iw, w.float(), b.float(), K, 0)
    g_o = O.weighted_mapped_conv_backward(gy.float(), smap, iw, x.float(), w.float(), b.float(),
                                          K, 0)
    xd, sd, id_, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    if p:
        y = _C.weighted_mapped_conv_forward(xd, sd, id_, wd_, bd, K, 0)
        gr = _C.weighted_mapped_conv_backward(gyd, sd, id_, xd, wd_, bd, K, 0)
    else:
        y = _C.mapped_conv_forward(xd, sd, wd_, bd, K, 0)
        gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 0)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert rel_err(y.float(), y_o) < tol
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm
    # transposed convolution: its backward-input is the gather-product over grad_output
    wt = (torch.randn(Ci, Co, K, generator=g) / (Ci * K) ** 0.5).to(dtype)
    t_o = O.weighted_mapped_transposed_conv_backward(gy.float(), smap, iw, x.float(), wt.float(),
                                                     b.float(), K, 0)
    if p:
        t = _C.weighted_mapped_transposed_conv_backward(gyd, sd, id_, xd, wt.cuda(), bd, K, 0)
    else:
        t = _C.mapped_transposed_conv_backward(gyd, sd, xd, wt.cuda(), bd, K, 0)
    for a, r, nm in zip(t, t_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, "transposed " + nm


@pytest.mark.parametrize("co", [128, 192, 130])
def test_conv_bf16_wide_outputs(co, device):
    """bf16 storage with 128 output channels per workgroup (Co = 128), with Co padded to a
    multiple of 64 but not of 128 (192) and ragged (130), input channels ragged too."""
    B, Ci, H, W, K = 1, 40, 12, 40, 9
    g = torch.Generator().manual_seed(co)
    smap = synthetic.latitude_map(H, W, 1)
    x = torch.randn(B, Ci, H, W, generator=g).bfloat16()
    w = (torch.randn(co, Ci, K, generator=g) / (Ci * K) ** 0.5).bfloat16()
    b = torch.randn(co, generator=g).bfloat16()
    gy = torch.randn(B, co, H, W, generator=g).bfloat16()
    y_o = O.mapped_conv_forward(x.float(), smap, w.float(), b.float(), K, 1)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, 1)
    y = _C.mapped_conv_forward(x.cuda(), smap.cuda(), w.cuda(), b.cuda(), K, 1)
    gr = _C.mapped_conv_backward(gy.cuda(), smap.cuda(), x.cuda(), w.cuda(), b.cuda(), K, 1)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


@pytest.mark.parametrize("interp", [0, 1])
@pytest.mark.parametrize("w_img", [256, 300])
def test_conv_bf16_wide_rows(interp, w_img, device):
    """bf16 storage on images at least 256 pixels wide: 1 x 128 pixel tiles (ragged at the
    right edge for W = 300), the channel-block copy of the gathered operand with channels
    padded (Ci = 24, Co = 40) and the ring of in-flight gathers."""
    B, Ci, Co, H, K = 2, 24, 40, 6, 9
    g = torch.Generator().manual_seed(900 + interp + w_img)
    smap = synthetic.latitude_map(H, w_img, 1)
    x = torch.randn(B, Ci, H, w_img, generator=g).bfloat16()
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).bfloat16()
    b = torch.randn(Co, generator=g).bfloat16()
    gy = torch.randn(B, Co, H, w_img, generator=g).bfloat16()
    y_o = O.mapped_conv_forward(x.float(), smap, w.float(), b.float(), K, interp)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, interp)
    y = _C.mapped_conv_forward(*dev(x, smap, w, b), K, interp)
    gr = _C.mapped_conv_backward(*dev(gy, smap, x, w, b), K, interp)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


def test_scatter_forms_many_to_one(device):
    """Every source pixel lands on the same few destination pixels: destination lists far
    longer than the length up to which they are sorted, empty lists everywhere else."""
    B, C, IH, IW, OH, OW = 2, 5, 40, 50, 6, 7
    g = torch.Generator().manual_seed(77)
    x = torch.randn(B, C, IH, IW, generator=g)
    smap = torch.zeros(IH, IW, 2)
    smap[..., 0] = 2.25
    smap[..., 1] = 3.5
    smap[::7, ::5, 0] = 5.0   # a few land elsewhere, some outside
    smap[::9, ::4, 1] = 40.0
    for interp in (0, 1, 2):
        want = O.resample_to_map(x, smap, OH, OW, interp)
        got = _C.resample_to_map(x.cuda(), smap.cuda(), OH, OW, interp)
        assert rel_err(got, want) < 1e-5
    K = 3
    pmap = smap[:, :, None, :].repeat(1, 1, K, 1).contiguous()
    gy = torch.randn(B, C, IH, IW, generator=g)
    want = O.mapped_avg_unpool(gy, pmap, OH, OW, K, 1)
    assert rel_err(_C.mapped_avg_unpool(gy.cuda(), pmap.cuda(), OH, OW, K, 1), want) < 1e-5


@pytest.mark.parametrize("interp", [1, 2])
def test_config4_cube_resample_and_pools(interp, device):
    """Cube map [B, C, F, 6F] -> equirect [2F, 4F] through the exact gnomonic map:
    resample_to_map (scatter), its adjoint gather, then mapped max / avg pooling with
    the latitude map on the equirect image.  F scaled to 32."""
    B, C, F = 2, 8, 32
    H, W = 2 * F, 4 * F
    g = torch.Generator().manual_seed(4)
    cube = torch.rand(B, C, F, 6 * F, generator=g)
    cmap = synthetic.cube_to_equirect_map(F, H, W)
    eq_o = O.resample_to_map(cube, cmap, H, W, interp)
    eq = _C.resample_to_map(cube.cuda(), cmap.cuda(), H, W, interp)
    assert rel_err(eq, eq_o) < 1e-5
    back_o = O.resample_from_map(eq_o, cmap, interp)
    back = _C.resample_from_map(eq_o.cuda(), cmap.cuda(), interp)
    assert torch.equal(back.cpu(), back_o)
    lmap = synthetic.latitude_map(H, W, 1)
    mo, mi = O.mapped_max_pool(eq_o, lmap, 9, 1)
    m, i = _C.mapped_max_pool(eq_o.cuda(), lmap.cuda(), 9, 1)
    assert torch.equal(m.cpu(), mo) and torch.equal(i.cpu(), mi)
    assert torch.equal(_C.mapped_avg_pool(eq_o.cuda(), lmap.cuda(), 9, 1).cpu(),
                       O.mapped_avg_pool(eq_o, lmap, 9, 1))
    gy = torch.randn(B, C, H, W, generator=g)
    assert rel_err(_C.mapped_max_unpool(gy.cuda(), i, lmap.cuda(), H, W, 9, 1),
                   O.mapped_max_unpool(gy, mi, lmap, H, W, 9, 1)) < 1e-5
    assert rel_err(_C.mapped_avg_unpool(gy.cuda(), lmap.cuda(), H, W, 9, 1),
                   O.mapped_avg_unpool(gy, lmap, H, W, 9, 1)) < 1e-5


@pytest.mark.parametrize("interp", [0, 1])
def test_pools_with_more_channels_than_one_thread_takes(interp, device):
    """3x3 pooling and unpooling with 72 channels and 2 images: the pooling gather takes 64
    channels per thread (72 = 64 + 8) and the unpooling gather 64 planes (144 = 64 + 64 + 16),
    so both see full and ragged groups.  Bit-exact pooling outputs and argmax, 1e-5 on the
    unpoolings."""
    B, C, H, W, K = 2, 72, 8, 64, 9
    g = torch.Generator().manual_seed(60 + interp)
    lmap = synthetic.latitude_map(H, W, 1)
    x = torch.randn(B, C, H, W, generator=g)
    gy = torch.randn(B, C, H, W, generator=g)
    mo, mi = O.mapped_max_pool(x, lmap, K, interp)
    ao = O.mapped_avg_pool(x, lmap, K, interp)
    xd, ld, gyd = x.cuda(), lmap.cuda(), gy.cuda()
    m, i = _C.mapped_max_pool(xd, ld, K, interp)
    a = _C.mapped_avg_pool(xd, ld, K, interp)
    assert torch.equal(m.cpu(), mo) and torch.equal(i.cpu(), mi) and torch.equal(a.cpu(), ao)
    assert rel_err(_C.mapped_avg_unpool(gyd, ld, H, W, K, interp),
                   O.mapped_avg_unpool(gy, lmap, H, W, K, interp)) < 1e-5
    assert rel_err(_C.mapped_max_unpool(gyd, i, ld, H, W, K, interp),
                   O.mapped_max_unpool(gy, mi, lmap, H, W, K, interp)) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("K", [10, 18, 25, 28])
def test_pools_with_more_than_nine_taps(K, interp, dtype, device):
    """Pooling maps of more than nine taps run nine taps at a time, every pass continuing from
    the sum or the winner the pass before left in the output: values, argmax and averages must
    still be those of one pass over all taps in order, bit for bit - also where every tap of a
    pixel lies outside the image (zeros, the first tap wins) and where one large value wins."""
    g = torch.Generator().manual_seed(700 + K + interp)
    B, C, IH, IW, OH, OW = 2, 5, 9, 40, 7, 33
    x = torch.randn(B, C, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, _ = helpers.random_map(g, OH, OW, K, 0, IH, IW, dtype)
    smap[0, :3] = -7.0          # pixels all of whose taps lie outside
    x[:, :, 0, 0] = 50.0        # a value that wins wherever it is sampled
    xd, sd = dev(x, smap)
    mo, mi = O.mapped_max_pool(x, smap, K, interp)
    ao = O.mapped_avg_pool(x, smap, K, interp)
    m, i = _C.mapped_max_pool(xd, sd, K, interp)
    a = _C.mapped_avg_pool(xd, sd, K, interp)
    assert torch.equal(m.cpu(), mo), "max-pool values must be bit-exact"
    assert torch.equal(i.cpu(), mi), "max-pool argmax must be bit-exact"
    assert torch.equal(a.cpu(), ao), "avg-pool gather must be bit-exact"


@pytest.mark.parametrize("radius,interp", [(1, 1), (2, 0), (2, 1), (3, 1)])
def test_unpool_list_lengths_for_both_sorting_networks(radius, interp, device):
    """Unpooling through latitude maps whose per-pixel contribution lists are 9 to 16 entries
    long (3x3 bilinear: the 16-key sorting network) and 17 to 32 (5x5 nearest: 25 entries,
    the 32-key network) or longer (5x5 bilinear: 50 - sorted by rank, a lane per entry, and
    gathered in passes of 24 entries that continue from the destination; 7x7 bilinear: 98, the
    insertion sort and five passes): same values as the oracle, and the same bits on every call."""
    B, C, H, W = 2, 3, 24, 128
    K = (2 * radius + 1) ** 2
    g = torch.Generator().manual_seed(40 + radius + interp)
    lmap = synthetic.latitude_map(H, W, radius)
    x = torch.randn(B, C, H, W, generator=g)
    gy = torch.randn(B, C, H, W, generator=g)
    _, mi = O.mapped_max_pool(x, lmap, K, interp)
    want_a = O.mapped_avg_unpool(gy, lmap, H, W, K, interp)
    want_m = O.mapped_max_unpool(gy, mi, lmap, H, W, K, interp)
    gyd, ld, mid = gy.cuda(), lmap.cuda(), mi.cuda()
    got_a = _C.mapped_avg_unpool(gyd, ld, H, W, K, interp)
    got_m = _C.mapped_max_unpool(gyd, mid, ld, H, W, K, interp)
    assert rel_err(got_a, want_a) < 1e-5
    assert rel_err(got_m, want_m) < 1e-5
    assert torch.equal(got_a, _C.mapped_avg_unpool(gyd, ld, H, W, K, interp))
    assert torch.equal(got_m, _C.mapped_max_unpool(gyd, mid, ld, H, W, K, interp))


def test_config4_full_size_scatter_properties(device):
    """Full spatial size of the cube -> equirect resampling (256x1536 -> 512x1024) and of the
    512x1024 unpoolings, fewer planes: the gather form against the atomic form, and
    adjointness <R_to(x), y> == <x, R_from(y)> (the oracle would take minutes here)."""
    F, H, W, B, C = 256, 512, 1024, 1, 16
    g = torch.Generator().manual_seed(44)
    cube = torch.rand(B, C, F, 6 * F, generator=g).cuda()
    y = torch.randn(B, C, H, W, generator=g).cuda()
    cmap = synthetic.cube_to_equirect_map(F, H, W).cuda()
    lmap = synthetic.latitude_map(H, W, 1).cuda()
    for interp in (1, 2):
        _C.scatter_as_gather = True
        to = _C.resample_to_map(cube, cmap, H, W, interp)
        back = _C.resample_from_map(y, cmap, interp)
        lhs = (to.double() * y.double()).sum()
        rhs = (cube.double() * back.double()).sum()
        assert abs(lhs - rhs) < 1e-6 * (cube.double() * back.double()).abs().sum()
        _C.scatter_as_gather = False
        try:
            to_atomic = _C.resample_to_map(cube, cmap, H, W, interp)
        finally:
            _C.scatter_as_gather = True
        assert rel_err(to, to_atomic.cpu()) < 1e-5
    m, i = _C.mapped_max_pool(y, lmap, 9, 1)
    au, mu = _C.mapped_avg_unpool(y, lmap, H, W, 9, 1), _C.mapped_max_unpool(y, i, lmap, H, W, 9, 1)
    _C.scatter_as_gather = False
    try:
        au_a = _C.mapped_avg_unpool(y, lmap, H, W, 9, 1)
        mu_a = _C.mapped_max_unpool(y, i, lmap, H, W, 9, 1)
    finally:
        _C.scatter_as_gather = True
    assert rel_err(au, au_a.cpu()) < 1e-5 and rel_err(mu, mu_a.cpu()) < 1e-5
    x = torch.randn(B, C, H, W, generator=g).cuda()
    lhs = (_C.mapped_avg_pool(x, lmap, 9, 1).double() * y.double()).sum()
    rhs = (x.double() * au.double()).sum()
    assert abs(lhs - rhs) < 1e-6 * (x.double() * au.double()).abs().sum()
    # sorted entry lists: the gather form gives the same bits on every call
    assert torch.equal(au, _C.mapped_avg_unpool(y, lmap, H, W, 9, 1))


def _sub_map(smap, picks):
    """The entries of `picks` (flat locations) of a map [H, W, ...] as a one-row map [1, n, ...]."""
    flat = smap.reshape((smap.shape[0] * smap.shape[1],) + tuple(smap.shape[2:]))
    return flat[picks].unsqueeze(0).contiguous()


def _random_picks(n, count, seed):
    g = torch.Generator().manual_seed(seed)
    fixed = torch.tensor([0, 1, n // 2, n - 2, n - 1])
    return torch.unique(torch.cat([fixed, torch.randperm(n, generator=g)[:count]]))


def test_config4_full_size_against_the_oracle_at_sampled_positions(device):
    """Configuration 4 at its own size - B=4, C=64, cube map 256 x 1536 <-> equirectangular
    512 x 1024, 3 x 3 latitude-map pooling - against the oracle evaluated on sampled positions
    only (a one-row map holding the sampled locations' entries):
    gathers (resample_from_map, pooled values, argmax) bit-exact at about 4 000 positions;
    scatters (resample_to_map, both unpoolings) within 1e-5 on inputs that are zero except at
    the sampled source positions, compared over the whole destination."""
    F, H, W, B, C, K = 256, 512, 1024, 4, 64, 9
    g = torch.Generator().manual_seed(404)
    cmap = synthetic.cube_to_equirect_map(F, H, W)
    lmap = synthetic.latitude_map(H, W, 1)
    y = torch.rand(B, C, H, W, generator=g)
    yd = y.cuda()
    for interp in (1, 2):
        # resample_from_map: equirectangular image sampled at the cube map's pixels
        picks = _random_picks(F * 6 * F, 4000, 10 + interp)
        want = O.resample_from_map(y, _sub_map(cmap, picks), interp)
        got = _C.resample_from_map(yd, cmap.cuda(), interp).view(B, C, -1)[:, :, picks.cuda()]
        assert torch.equal(got.cpu(), want[:, :, 0]), "resample_from_map at sampled positions"
        del got
        # resample_to_map: a cube image that is zero except at the sampled pixels
        vals = torch.rand(B, C, 1, len(picks), generator=g)
        cube = torch.zeros(B, C, F * 6 * F)
        cube[:, :, picks] = vals[:, :, 0]
        want = O.resample_to_map(vals, _sub_map(cmap, picks), H, W, interp)
        got = _C.resample_to_map(cube.view(B, C, F, 6 * F).cuda(), cmap.cuda(), H, W, interp)
        assert rel_err(got, want) < 1e-5, "resample_to_map"
        helpers.assert_close_elementwise(got, want, 1e-5, "resample_to_map")
        del got, cube
    # pooling over the equirectangular image
    picks = _random_picks(H * W, 4000, 20)
    sub = _sub_map(lmap, picks)
    ld = lmap.cuda()
    for interp in (0, 1):
        mo, mi = O.mapped_max_pool(y, sub, K, interp)
        ao = O.mapped_avg_pool(y, sub, K, interp)
        m, i = _C.mapped_max_pool(yd, ld, K, interp)
        a = _C.mapped_avg_pool(yd, ld, K, interp)
        pc = picks.cuda()
        assert torch.equal(m.view(B, C, -1)[:, :, pc].cpu(), mo[:, :, 0]), "max-pool values"
        assert torch.equal(a.view(B, C, -1)[:, :, pc].cpu(), ao[:, :, 0]), "avg-pool values"
        # the oracle's winners are offsets into its one-row map: the tap is (offset / 2) % K
        tap = (mi[:, :, 0] // 2) % K
        full_idx = torch.where(mi[:, :, 0] >= 0, (picks.view(1, 1, -1) * K + tap) * 2, mi[:, :, 0])
        assert torch.equal(i.view(B, C, -1)[:, :, pc].cpu(), full_idx), "max-pool argmax"
        # unpoolings: a gradient that is zero except at the sampled pooled pixels
        gvals = torch.randn(B, C, 1, len(picks), generator=g)
        gout = torch.zeros(B, C, H * W)
        gout[:, :, picks] = gvals[:, :, 0]
        goutd = gout.view(B, C, H, W).cuda()
        want_a = O.mapped_avg_unpool(gvals, sub, H, W, K, interp)
        got_a = _C.mapped_avg_unpool(goutd, ld, H, W, K, interp)
        assert rel_err(got_a, want_a) < 1e-5, "avg unpool"
        helpers.assert_close_elementwise(got_a, want_a, 1e-5, "avg unpool")
        del got_a, want_a
        want_m = O.mapped_max_unpool(gvals, mi, sub, H, W, K, interp)
        got_m = _C.mapped_max_unpool(goutd, i, ld, H, W, K, interp)
        assert rel_err(got_m, want_m) < 1e-5, "max unpool"
        helpers.assert_close_elementwise(got_m, want_m, 1e-5, "max unpool")
        del got_m, want_m, m, i, a, goutd


def test_config4_knn_full_size_against_the_oracle_at_sampled_queries(device):
    """524 288 queries against 40 962 reference points on the unit sphere, k = 8: indices and
    distances of 2 048 sampled queries bit-exact against the oracle."""
    ref = synthetic.sphere_points(40962, seed=1)
    qry = synthetic.sphere_points(524288, seed=2)
    idx, dist = knn(ref.cuda(), qry.cuda(), 8)
    g = torch.Generator().manual_seed(8)
    pick = torch.unique(torch.cat([torch.tensor([0, 524287]),
                                   torch.randint(0, 524288, (2046,), generator=g)]))
    io, do = O.knn_forward(ref, qry[:, :, pick].contiguous(), 8)
    assert torch.equal(idx[:, :, pick.cuda()].cpu(), io), "KNN indices must be bit-exact"
    assert torch.equal(dist[:, :, pick.cuda()].cpu(), do)


def test_config5_bf16_5x5(device):
    """Encoder-scale shape scaled down: 128 -> 128 channels, 5x5 latitude map (K=25),
    bf16 storage with fp32 accumulation, against the fp32 oracle."""
    B, C, H, W, K = 1, 128, 16, 64, 25
    g = torch.Generator().manual_seed(5)
    bf = lambda t: t.to(torch.bfloat16)
    x, gy = bf(torch.randn(B, C, H, W, generator=g)), bf(torch.randn(B, C, H, W, generator=g))
    w = bf(torch.randn(C, C, K, generator=g) / (C * K) ** 0.5)
    b = bf(torch.randn(C, generator=g))
    smap = synthetic.latitude_map(H, W, 2)
    y_o = O.mapped_conv_forward(x.float(), smap, w.float(), b.float(), K, 1)
    g_o = O.mapped_conv_backward(gy.float(), smap, x.float(), w.float(), b.float(), K, 1)
    xd, sd, wd_, bd, gyd = dev(x, smap, w, b, gy)
    y = _C.mapped_conv_forward(xd, sd, wd_, bd, K, 1)
    gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, 1)
    assert rel_err(y.float(), y_o) < 2e-2
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < 2e-2, nm


def test_headline_shape_properties(device):
    """B=8, 64->64, 256x512, 3x3 latitude map, fp32, at full size: linearity in the
    input, adjointness of forward and input gradient, bias gradient = plain sum, and
    the weight gradient as the derivative of <conv(x), g> along a random direction."""
    torch.manual_seed(6)
    B, C, H, W = 8, 64, 256, 512
    x = torch.randn(B, C, H, W, device=device)
    gy = torch.randn(B, C, H, W, device=device)
    w = torch.randn(C, C, 9, device=device) / 24
    zero = torch.zeros(C, device=device)
    smap = synthetic.latitude_map(H, W, 1).to(device)
    for interp in (0, 1):
        y = _C.mapped_conv_forward(x, smap, w, zero, 9, interp)
        gx, gw, gb = _C.mapped_conv_backward(gy, smap, x, w, zero, 9, interp)
        lhs, rhs = (y.double() * gy.double()).sum(), (x.double() * gx.double()).sum()
        assert abs(lhs - rhs) / abs(lhs) < 1e-5
        assert rel_err(gb, gy.double().sum((0, 2, 3))) < 1e-5
        dw = torch.randn_like(w)
        y2 = _C.mapped_conv_forward(x, smap, dw, zero, 9, interp)  # linear in the weight
        lhs, rhs = (y2.double() * gy.double()).sum(), (gw.double() * dw.double()).sum()
        assert abs(lhs - rhs) / abs(lhs) < 1e-4
        y3 = _C.mapped_conv_forward(2 * x, smap, w, zero, 9, interp)
        assert rel_err(y3, 2 * y) < 1e-6


# ----------------------------------------------------- size-independent properties
@pytest.mark.parametrize("interp", [0, 1])
def test_identity_map_equals_conv2d_large(interp, device):
    """With the regular-grid map a mapped convolution is a zero-padded 3x3
    convolution; checked against the library routine at B=2, 64->64, 128x256."""
    torch.manual_seed(2)
    B, C, H, W = 2, 64, 128, 256
    x = torch.randn(B, C, H, W, device=device)
    w = torch.randn(C, C, 9, device=device) / 24
    b = torch.randn(C, device=device)
    smap = synthetic.identity_grid_map(H, W, 1).to(device)
    gy = torch.randn(B, C, H, W, device=device)
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    ref = F.conv2d(xr, wr.view(C, C, 3, 3), b.double(), padding=1)
    gx_r, gw_r = torch.autograd.grad(ref, (xr, wr), gy.double())
    y = _C.mapped_conv_forward(x, smap, w, b, 9, interp)
    gx, gw, gb = _C.mapped_conv_backward(gy, smap, x, w, b, 9, interp)
    assert rel_err(y, ref.detach()) < 1e-5
    assert rel_err(gx, gx_r) < 1e-5
    assert rel_err(gw, gw_r) < 1e-5
    assert rel_err(gb, gy.double().sum((0, 2, 3))) < 1e-5


@pytest.mark.parametrize("interp", [0, 1, 2])
def test_adjointness_large(interp, device):
    """<conv(x), g> == <x, conv_backward_input(g)> and <from_map(s), g> == <s, to_map(g)>."""
    torch.manual_seed(3)
    B, C, H, W = 2, 32, 64, 128
    x = torch.randn(B, C, H, W, device=device)
    w = torch.randn(C, C, 9, device=device) / 17
    zero = torch.zeros(C, device=device)
    smap = synthetic.latitude_map(H, W, 1).to(device)
    g = torch.randn(B, C, H, W, device=device)
    y = _C.mapped_conv_forward(x, smap, w, zero, 9, interp)
    gx = _C.mapped_conv_backward(g, smap, x, w, zero, 9, interp)[0]
    lhs, rhs = (y.double() * g.double()).sum(), (x.double() * gx.double()).sum()
    assert abs(lhs - rhs) / abs(lhs) < 1e-5
    sm1 = smap[:, :, 3].contiguous()
    lhs = (_C.resample_from_map(x, sm1, interp).double() * g.double()).sum()
    rhs = (x.double() * _C.resample_to_map(g, sm1, H, W, interp).double()).sum()
    assert abs(lhs - rhs) / abs(lhs) < 1e-5


def test_linearity_of_forward(device):
    torch.manual_seed(4)
    B, C, H, W = 1, 16, 32, 64
    x1, x2 = torch.randn(B, C, H, W, device=device), torch.randn(B, C, H, W, device=device)
    w = torch.randn(8, C, 9, device=device)
    zero = torch.zeros(8, device=device)
    smap = synthetic.latitude_map(H, W, 1).to(device)
    y = _C.mapped_conv_forward(x1 + 2 * x2, smap, w, zero, 9, 1)
    y12 = _C.mapped_conv_forward(x1, smap, w, zero, 9, 1) + 2 * _C.mapped_conv_forward(
        x2, smap, w, zero, 9, 1)
    assert rel_err(y, y12) < 1e-5


# ---------------------------------------------------------------------------- knn
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [1, 8, 20])
def test_knn_vs_oracle(dtype, k, device):
    g = torch.Generator().manual_seed(500 + k)
    B, D, R, Q = 2, 3, 1000, 700
    ref = torch.randn(B, D, R, generator=g, dtype=torch.float64).to(dtype)
    qry = torch.randn(B, D, Q, generator=g, dtype=torch.float64).to(dtype)
    ref[:, :, 50] = ref[:, :, 10]
    qry[:, :, 0] = ref[:, :, 10]
    io, do = O.knn_forward(ref, qry, k)
    i, d = knn(ref.cuda(), qry.cuda(), k)
    assert torch.equal(i.cpu(), io), "KNN indices must be bit-exact"
    assert torch.equal(d.cpu(), do)


def test_knn_other_dimensions(device):
    for D in (1, 2, 4, 6):
        g = torch.Generator().manual_seed(D)
        ref = torch.randn(1, D, 299 + D, generator=g)   # not a multiple of the batch of 8
        qry = torch.randn(1, D, 260, generator=g)
        io, do = O.knn_forward(ref, qry, 5)
        i, d = knn(ref.cuda(), qry.cuda(), 5)
        assert torch.equal(i.cpu(), io) and torch.equal(d.cpu(), do)


def test_knn_sphere_invariants(device):
    """Unit-sphere points, 65536 queries x 40962 references, k=8: ascending
    distances, distances match the indexed points, and no excluded point is closer
    than the k-th on sampled queries."""
    ref = synthetic.sphere_points(40962, seed=1).to(device)
    qry = synthetic.sphere_points(65536, seed=2).to(device)
    idx, dist = knn(ref, qry, 8)
    assert idx.min() >= 1 and idx.max() <= 40962
    assert (dist[:, 1:] >= dist[:, :-1]).all()
    picked = ref[0][:, (idx[0] - 1).reshape(-1)].view(3, 8, -1)
    d2 = ((picked - qry[0][:, None, :]) ** 2).sum(0).sqrt()
    torch.testing.assert_close(d2, dist[0], rtol=1e-4, atol=1e-6)
    sample = torch.arange(0, 65536, 997, device=device)
    full = torch.cdist(qry[0][:, sample].t().double(), ref[0].t().double())
    kth = full.sort(-1).values[:, 7]
    torch.testing.assert_close(dist[0, 7, sample].double(), kth, rtol=1e-5, atol=1e-6)


def test_scatter_as_gather_keeps_infinities_where_they_belong(device):
    """A non-finite source value reaches the destinations its own taps touch and no others:
    destinations that receive nothing stay exactly zero (padded list entries are dropped, not
    multiplied by a zero weight)."""
    B, C, IH, IW, OH, OW = 1, 3, 12, 20, 9, 11
    x = torch.ones(B, C, IH, IW)
    x[:, :, 0, 0] = float("inf")       # source element 0: what an empty list would re-read
    smap = torch.zeros(IH, IW, 2)
    smap[..., 0] = 4.25
    smap[..., 1] = 5.5                  # everything lands around (5..6, 4..5)
    want = O.resample_to_map(x, smap, OH, OW, 1)
    got = _C.resample_to_map(x.cuda(), smap.cuda(), OH, OW, 1).cpu()
    assert torch.equal(torch.isinf(got), torch.isinf(want))
    assert (got[~torch.isinf(want)] == 0).all() and not torch.isnan(got).any()
    K = 2
    pmap = smap[:, :, None, :].repeat(1, 1, K, 1).contiguous()
    want = O.mapped_avg_unpool(x, pmap, OH, OW, K, 1)
    got = _C.mapped_avg_unpool(x.cuda(), pmap.cuda(), OH, OW, K, 1).cpu()
    assert torch.equal(torch.isinf(got), torch.isinf(want)) and not torch.isnan(got).any()
