"""Map plans (no counterpart in the reference): what an operator derives from sample_map alone,
built once and reused.  For every op that takes one: planned == unplanned == oracle, the plan
serves repeated calls, and the cache in the Python mirror picks plans up by itself."""
import pytest
import torch

import helpers
from helpers import rel_err
from oracle import ops as O

from mappedconvolutions_amd import _C
from mappedconvolutions_amd.util import synthetic

pytestmark = pytest.mark.gpu


def dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("interp,p", [(0, 0), (0, 4), (1, 0), (2, 0), (1, 2)])
def test_conv_forward_and_backward_with_one_plan(interp, p, dtype, device):
    """One plan per (map, input size) serves the forward (resolved taps), the input gradient
    (transposed map) and the weight gradient (pair masks).  (1, 2): bilinear with two points
    is eight pairs per tap: no gather part, the forward decodes the map as without a plan."""
    g = torch.Generator().manual_seed(2000 + 10 * interp + p)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 20, 36, 14, 40, 11, 37, 5
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    smap, iw = helpers.random_map(g, OH, OW, K, p, IH, IW, torch.float32)
    x = torch.randn(B, Ci, IH, IW, generator=g).to(dtype)
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dtype)
    b = torch.randn(Co, generator=g).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g).to(dtype)
    y_o = O.weighted_mapped_conv_forward(x.float(), smap, iw, w.float(), b.float(), K, interp)
    g_o = O.weighted_mapped_conv_backward(gy.float(), smap, iw, x.float(), w.float(), b.float(),
                                          K, interp)
    xd, sd, iwd, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    plan = _C.conv_map_plan(sd, iwd, IH, IW, interp, dtype)
    assert plan is not None
    for _ in range(2):
        if p:
            y = _C.weighted_mapped_conv_forward(xd, sd, iwd, wd_, bd, K, interp, plan=plan)
            gr = _C.weighted_mapped_conv_backward(gyd, sd, iwd, xd, wd_, bd, K, interp, plan=plan)
        else:
            y = _C.mapped_conv_forward(xd, sd, wd_, bd, K, interp, plan=plan)
            gr = _C.mapped_conv_backward(gyd, sd, xd, wd_, bd, K, interp, plan=plan)
    y_plain = _C.weighted_mapped_conv_forward(xd, sd, iwd, wd_, bd, K, interp) if p else \
        _C.mapped_conv_forward(xd, sd, wd_, bd, K, interp)
    assert rel_err(y.float(), y_o) < tol
    assert rel_err(y.float(), y_plain.float()) < tol
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("interp,p", [(0, 3), (1, 0), (2, 0)])
def test_transposed_conv_with_one_plan(interp, p, dtype, device):
    """A transposed convolution's map samples its OUTPUT: the plan is built for that size and
    serves its forward (scatter), its input gradient (gather) and its weight gradient."""
    g = torch.Generator().manual_seed(2100 + 10 * interp + p)
    B, Ci, Co, IH, IW, OH, OW, K = 2, 18, 24, 9, 21, 13, 30, 4
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    smap, iw = helpers.random_map(g, IH, IW, K, p, OH, OW, torch.float32)
    x = torch.randn(B, Ci, IH, IW, generator=g).to(dtype)
    w = (torch.randn(Ci, Co, K, generator=g) / (Ci * K) ** 0.5).to(dtype)
    b = torch.randn(Co, generator=g).to(dtype)
    gy = torch.randn(B, Co, OH, OW, generator=g).to(dtype)
    y_o = O.weighted_mapped_transposed_conv_forward(x.float(), smap, iw, w.float(), b.float(),
                                                    OH, OW, K, interp)
    g_o = O.weighted_mapped_transposed_conv_backward(gy.float(), smap, iw, x.float(), w.float(),
                                                     b.float(), K, interp)
    xd, sd, iwd, wd_, bd, gyd = dev(x, smap, iw, w, b, gy)
    plan = _C.conv_map_plan(sd, iwd, OH, OW, interp, dtype)
    assert plan is not None
    for _ in range(2):
        if p:
            y = _C.weighted_mapped_transposed_conv_forward(xd, sd, iwd, wd_, bd, OH, OW, K, interp,
                                                           plan=plan)
            gr = _C.weighted_mapped_transposed_conv_backward(gyd, sd, iwd, xd, wd_, bd, K, interp,
                                                             plan=plan)
        else:
            y = _C.mapped_transposed_conv_forward(xd, sd, wd_, bd, OH, OW, K, interp, plan=plan)
            gr = _C.mapped_transposed_conv_backward(gyd, sd, xd, wd_, bd, K, interp, plan=plan)
    assert rel_err(y.float(), y_o) < tol
    for a, r, nm in zip(gr, g_o, ("grad_input", "grad_weight", "grad_bias")):
        assert rel_err(a.float(), r) < tol, nm


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_resample_and_unpool_plans(dtype, interp, p, device):
    """resample_to_map, avg unpool and max unpool through plans: the same bits as the per-call
    form (both sort every destination's contributions), the oracle's values."""
    g = torch.Generator().manual_seed(2200 + 10 * interp + p)
    B, C, IH, IW, OH, OW, K = 2, 11, 9, 13, 7, 9, 5
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    # resample_to_map: map [IH, IW, (P,) 2] into OH x OW
    x = torch.randn(B, C, IH, IW, generator=g, dtype=torch.float64).to(dtype)
    smap, iw = helpers.random_map(g, IH, IW, 1, p, OH, OW, dtype)
    smap = smap[:, :, 0].contiguous()
    iw = None if iw is None else iw[:, :, 0].contiguous()
    xd, sd, iwd = dev(x, smap, iw)
    plan = _C.scatter_map_plan(sd, iwd, OH, OW, interp)
    want = O.weighted_resample_to_map(x, smap, iw, OH, OW, interp)
    for _ in range(2):
        got = _C.weighted_resample_to_map(xd, sd, iwd, OH, OW, interp, plan=plan) if p else \
            _C.resample_to_map(xd, sd, OH, OW, interp, plan=plan)
    plain = _C.weighted_resample_to_map(xd, sd, iwd, OH, OW, interp) if p else \
        _C.resample_to_map(xd, sd, OH, OW, interp)
    assert rel_err(got, want) < tol and torch.equal(got, plain)
    # unpoolings: map [OH, OW, K, (P,) 2] into IH x IW
    pmap, piw = helpers.random_map(g, OH, OW, K, p, IH, IW, dtype)
    gy = torch.randn(B, C, OH, OW, generator=g, dtype=torch.float64).to(dtype)
    _, mi = O.weighted_mapped_max_pool(x, pmap, piw, K, interp)
    pd, pwd, gyd, mid = dev(pmap, piw, gy, mi)
    plan_a = _C.scatter_map_plan(pd, pwd, IH, IW, interp)
    plan_m = _C.scatter_map_plan(pd, pwd, IH, IW, interp, for_max_unpool=True)
    want_a = O.weighted_mapped_avg_unpool(gy, pmap, piw, IH, IW, K, interp)
    want_m = O.weighted_mapped_max_unpool(gy, mi, pmap, piw, IH, IW, K, interp)
    if p:
        got_a = _C.weighted_mapped_avg_unpool(gyd, pd, pwd, IH, IW, K, interp, plan=plan_a)
        got_m = _C.weighted_mapped_max_unpool(gyd, mid, pd, pwd, IH, IW, K, interp, plan=plan_m)
        plain_a = _C.weighted_mapped_avg_unpool(gyd, pd, pwd, IH, IW, K, interp)
        plain_m = _C.weighted_mapped_max_unpool(gyd, mid, pd, pwd, IH, IW, K, interp)
    else:
        got_a = _C.mapped_avg_unpool(gyd, pd, IH, IW, K, interp, plan=plan_a)
        got_m = _C.mapped_max_unpool(gyd, mid, pd, IH, IW, K, interp, plan=plan_m)
        plain_a = _C.mapped_avg_unpool(gyd, pd, IH, IW, K, interp)
        plain_m = _C.mapped_max_unpool(gyd, mid, pd, IH, IW, K, interp)
    assert rel_err(got_a, want_a) < tol and torch.equal(got_a, plain_a)
    assert rel_err(got_m, want_m) < tol and torch.equal(got_m, plain_m)


def test_plan_cache_serves_every_op(device):
    """With the cache on, conv / transposed conv / resample / unpool calls build their plans
    at first use and find them afterwards; results stay those of the plain calls."""
    g = torch.Generator().manual_seed(2300)
    B, C, H, W, K = 1, 16, 16, 32, 9
    x, gy = torch.randn(B, C, H, W, generator=g).cuda(), torch.randn(B, C, H, W, generator=g).cuda()
    w, b = (torch.randn(C, C, K, generator=g) / 12).cuda(), torch.randn(C, generator=g).cuda()
    smap = synthetic.latitude_map(H, W, 1).cuda()
    rmap = smap[:, :, 2].contiguous()
    _, idx = _C.mapped_max_pool(x, smap, K, 1)
    plain = [_C.mapped_conv_forward(x, smap, w, b, K, 1),
             _C.mapped_transposed_conv_forward(x, smap, w, b, H, W, K, 1),
             _C.resample_to_map(x, rmap, H, W, 1),
             _C.mapped_avg_unpool(gy, smap, H, W, K, 1),
             _C.mapped_max_unpool(gy, idx, smap, H, W, K, 1)]
    _C.enable_map_plan_cache(True)
    try:
        for _ in range(2):
            cached = [_C.mapped_conv_forward(x, smap, w, b, K, 1),
                      _C.mapped_transposed_conv_forward(x, smap, w, b, H, W, K, 1),
                      _C.resample_to_map(x, rmap, H, W, 1),
                      _C.mapped_avg_unpool(gy, smap, H, W, K, 1),
                      _C.mapped_max_unpool(gy, idx, smap, H, W, K, 1)]
            _C.mapped_conv_backward(gy, smap, x, w, b, K, 1)
            _C.mapped_transposed_conv_backward(gy, smap, x, w, b, K, 1)
        # conv and transposed conv share one plan here (same map, same sampled size)
        assert len(_C.map_plan_cache) == 4
    finally:
        _C.enable_map_plan_cache(False)
    for a, r in zip(cached, plain):
        assert rel_err(a, r) < 1e-5


def test_a_plan_is_refused_where_it_was_not_built_for(device):
    """Plans of equal size are not interchangeable: one built for bilinear does not serve
    bispherical, one built from another map tensor of the same shape does not serve this map,
    an average-unpool plan does not serve max unpooling (their source codes differ), a plan
    for another destination size or data type is not taken, and neither is a descriptor that
    was edited after the build.  Each is rejected before anything is enqueued."""
    g = torch.Generator().manual_seed(2400)
    B, C, H, W, K = 1, 8, 12, 24, 9
    x, gy = torch.randn(B, C, H, W, generator=g).cuda(), torch.randn(B, C, H, W, generator=g).cuda()
    w, b = (torch.randn(C, C, K, generator=g) / 9).cuda(), torch.randn(C, generator=g).cuda()
    smap = synthetic.latitude_map(H, W, 1).cuda()
    other = (smap + 0.25).contiguous()
    plan = _C.conv_map_plan(smap, None, H, W, 1)
    want = _C.mapped_conv_forward(x, smap, w, b, K, 1)
    assert torch.equal(_C.mapped_conv_forward(x, smap, w, b, K, 1, plan=plan), want)
    refused = dict(match="plan was not built for")
    with pytest.raises(RuntimeError, **refused):      # other interpolation, same sizes
        _C.mapped_conv_forward(x, smap, w, b, K, 2, plan=plan)
    with pytest.raises(RuntimeError, **refused):
        _C.mapped_conv_backward(gy, smap, x, w, b, K, 2, plan=plan)
    with pytest.raises(RuntimeError, **refused):      # other map of the same shape
        _C.mapped_conv_forward(x, other, w, b, K, 1, plan=plan)
    with pytest.raises(RuntimeError, **refused):      # a transposed conv's map samples its output:
        _C.mapped_transposed_conv_forward(x, smap, w, b, H, W // 2, K, 1, plan=plan)  # H x W/2 here
    with pytest.raises(RuntimeError, match="workspace missing or too small"):  # (too small a plan)
        _C.mapped_transposed_conv_forward(x, smap, w, b, H, 2 * W, K, 1, plan=plan)
    # (any code other than 1 or 2 is nearest: a plan built with 0 serves 7)
    plan0 = _C.conv_map_plan(smap, None, H, W, 0)
    assert torch.equal(_C.mapped_conv_forward(x, smap, w, b, K, 7, plan=plan0),
                       _C.mapped_conv_forward(x, smap, w, b, K, 0))
    # scatter plans
    _, idx = _C.mapped_max_pool(x, smap, K, 1)
    plan_a = _C.scatter_map_plan(smap, None, H, W, 1)
    plan_m = _C.scatter_map_plan(smap, None, H, W, 1, for_max_unpool=True)
    assert plan_a.numel() == plan_m.numel()
    _C.mapped_avg_unpool(gy, smap, H, W, K, 1, plan=plan_a)
    _C.mapped_max_unpool(gy, idx, smap, H, W, K, 1, plan=plan_m)
    with pytest.raises(RuntimeError, **refused):
        _C.mapped_max_unpool(gy, idx, smap, H, W, K, 1, plan=plan_a)
    with pytest.raises(RuntimeError, **refused):
        _C.mapped_avg_unpool(gy, smap, H, W, K, 1, plan=plan_m)
    with pytest.raises(RuntimeError, **refused):
        _C.mapped_avg_unpool(gy, smap, H, W, K, 2, plan=plan_a)
    with pytest.raises(RuntimeError, **refused):      # built for float32 weights
        _C.mapped_avg_unpool(gy.double(), smap.double(), H, W, K, 1, plan=plan_a)
    with pytest.raises(RuntimeError, **refused):      # a conv plan is not a scatter plan
        _C.mapped_avg_unpool(gy, smap, H, W, K, 1, plan=plan)
    # an edited descriptor no longer matches its own check word
    plan_a.desc.K = K + 1
    with pytest.raises(RuntimeError, **refused):
        _C.mapped_avg_unpool(gy, smap, H, W, K, 1, plan=plan_a)
    with pytest.raises(RuntimeError, match="plan must come from"):
        _C.mapped_avg_unpool(gy, smap, H, W, K, 1, plan=plan_m.buffer)
