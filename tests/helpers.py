"""Shared test helpers: the transcribed known-answer cases of the reference's
tests, random problem generators, and a runner that evaluates a case through any
ops namespace (the CPU oracle, the reference's CPU build, or the HIP boundary)."""
import json
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
INTERP = {'nearest': 0, 'bilinear': 1, 'bispherical': 2}

with open(os.path.join(HERE, "golden", "reference_known_answers.json")) as f:
    KNOWN = json.load(f)

CASES = {c["name"]: c for c in KNOWN["cases"]}


def case_tensors(case, dtype=torch.float64):
    """(input [B,C,H,W], sample_map, interp_weights or None, expected [.., H', W'] broadcastable)."""
    spec = KNOWN["inputs"][case["input"]]
    h, w = spec["shape"]
    if "fill" in spec:
        plane = torch.full((h, w), spec["fill"], dtype=dtype)
    else:
        plane = torch.arange(h * w, dtype=dtype).view(h, w)
    op = case["op"]
    ch = KNOWN["in_channels"] if op in ("conv", "tconv") else (3 if op == "unresample" else 1)
    x = plane.repeat(KNOWN["batch"], ch, 1, 1).contiguous()
    smap = torch.tensor(KNOWN["maps"][case["map"]], dtype=dtype)
    iw = case.get("interp_weights")
    iw = None if iw is None else torch.tensor(KNOWN["interp_weights"][iw], dtype=dtype)
    exp = torch.tensor(case["expected_plane"], dtype=dtype)
    if "expected_affine" in case:
        a, b = case["expected_affine"]
        exp = a + b * exp
    return x, smap, iw, exp


def case_weights(case, dtype=torch.float64):
    ci, co, k = KNOWN["in_channels"], KNOWN["out_channels"], KNOWN["kernel_size"]
    shape = (co, ci, k) if case["op"] == "conv" else (ci, co, k)
    w = torch.ones(shape, dtype=dtype)
    if case["weights"] == "first_half_0.25":
        w[..., :k // 2] *= 0.25
    bias = torch.full((co,), 2.0, dtype=dtype)
    return w, bias


def run_case(ops, case, device="cpu", dtype=torch.float64):
    """Evaluate a known-answer case through ops-level functions; returns (output, expected)."""
    x, smap, iw, exp = case_tensors(case, dtype)
    x, smap = x.to(device), smap.to(device)
    iw = None if iw is None else iw.to(device)
    interp = INTERP[case["interpolation"]]
    k = KNOWN["kernel_size"]
    op = case["op"]
    if op == "conv":
        w, b = case_weights(case, dtype)
        out = ops.mapped_conv_forward(x, smap, w.to(device), b.to(device), k, interp)
    elif op == "tconv":
        w, b = case_weights(case, dtype)
        oh, ow = case["output_shape"]
        out = ops.mapped_transposed_conv_forward(x, smap, w.to(device), b.to(device), oh, ow, k,
                                                 interp)
    elif op == "max_pool":
        out = ops.mapped_max_pool(x, smap, k, interp)[0]
    elif op == "avg_pool":
        out = ops.mapped_avg_pool(x, smap, k, interp)
    elif op == "unresample":
        if iw is None:
            out = ops.resample_from_map(x, smap, interp)
        else:
            out = ops.weighted_resample_from_map(x, smap, iw, interp)
    else:
        raise ValueError(op)
    return out, exp


def random_map(gen, oh, ow, k, p, ih, iw_, dtype, integer=False, half=False):
    """Random sample map [oh, ow, k, (p,) 2] with coordinates spilling outside the
    image on every side, plus interp weights [oh, ow, k, p] when p > 0."""
    shape = (oh, ow, k) + ((p,) if p else ())
    x = torch.rand(shape, generator=gen, dtype=torch.float64) * (iw_ + 3) - 2
    y = torch.rand(shape, generator=gen, dtype=torch.float64) * (ih + 3) - 2
    if integer:
        x, y = x.round(), y.round()
    if half:  # exact .5 coordinates exercise the round-half-away rule
        x, y = x.floor() + 0.5, y.floor() + 0.5
    smap = torch.stack([x, y], -1).to(dtype).contiguous()
    wts = None
    if p:
        wts = torch.rand(shape, generator=gen, dtype=torch.float64).to(dtype).contiguous()
    return smap, wts


def rel_err(a, b):
    """max |a-b| / max(|b|, tiny): error relative to the magnitude of the result."""
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def assert_close_elementwise(a, b, tol, what=""):
    """Every element: |a - b| <= tol * (|b| + rms(b)).  Unlike rel_err, an element that is small
    against the largest one still has to be right to `tol` of the result's typical size."""
    a, b = a.double().cpu(), b.double().cpu()
    rms = b.pow(2).mean().sqrt().clamp_min(1e-30)
    excess = (a - b).abs() - tol * (b.abs() + rms)
    worst = excess.max().item()
    assert worst <= 0, "%s: element off by %.3g beyond tol %.1e (rms %.3g)" % (
        what, worst + tol * rms.item(), tol, rms.item())


def map_contributions(smap, iw, dh, dw, interp):
    """Destination cells (pixel * K + tap) of every contribution with a nonzero weight that a
    scatter through `smap` [MH, MW, K, (P,) 2] makes into a dh x dw image: the entries of the
    map turned around.  Returns a 1-D int64 tensor of cell indices (with repeats)."""
    K = smap.shape[2]
    m = smap.double()
    if iw is None:
        m = m.unsqueeze(3)
        w = torch.ones(m.shape[:-1], dtype=torch.float64)
    else:
        w = iw.double()
    x, y = m[..., 0], m[..., 1]
    tap = torch.arange(K).view(1, 1, K, 1).expand_as(x)
    cells = []
    if interp == 0:
        xi = torch.where(x >= 0, (x + 0.5).floor(), (x - 0.5).ceil()).long()
        yi = torch.where(y >= 0, (y + 0.5).floor(), (y - 0.5).ceil()).long()
        corners = [(xi, yi, w)]
    else:
        x1, y1 = x.floor(), y.floor()
        corners = []
        for cx, cy, cw in ((x1, y1, (y1 + 1 - y) * (x1 + 1 - x)), (x1 + 1, y1, (y1 + 1 - y) * (x - x1)),
                           (x1, y1 + 1, (y - y1) * (x1 + 1 - x)), (x1 + 1, y1 + 1, (y - y1) * (x - x1))):
            corners.append((cx.long(), cy.long(), cw * w))
    for cx, cy, cw in corners:
        if interp == 2:
            cx = cx % dw
        ok = (cx >= 0) & (cx < dw) & (cy >= 0) & (cy < dh) & (cw != 0)
        cells.append(((cy * dw + cx) * K + tap)[ok])
    return torch.cat(cells)


def transposed_map_overflows(smap, iw, dh, dw, interp):
    """True when the convolution's slotted transposed map cannot hold this map: more
    contributions beyond the slots of their cells (4, or 8 for single-row maps) than the
    overflow list has room for (2 per map sample).  The product then runs through the
    scatter kernel with its LDS windows and atomics."""
    cells = map_contributions(smap, iw, dh, dw, interp)
    slots = 8 if smap.shape[0] == 1 else 4
    counts = torch.bincount(cells, minlength=dh * dw * smap.shape[2])
    spill = (counts - slots).clamp_min(0).sum().item()
    cap = smap[..., 0].numel() * 2
    return spill > cap
