"""The entry point that allocates nothing: mcx_conv_forward_static keeps its scratch in an array
inside the library (one per GPU) instead of a caller's workspace.  Called through the C ABI with
caller-owned inputs and outputs and compared with mcx_conv_forward on the same inputs: the same
kernels on the same data, so the same bits.  Two calls in a row, the second on a smaller problem
(whatever the first left in the array must not matter), then fp64 (no scratch at all), a weighted
nearest map, and a problem whose scratch exceeds the array."""
import pytest
import torch

import helpers
from mappedconvolutions_amd import _C, _lib
from mappedconvolutions_amd.util import synthetic

pytestmark = pytest.mark.gpu


def _static_forward(x, smap, iw, w, b, K, interp):
    lib = _lib.load()
    B, Ci, IH, IW = x.shape
    Co, (OH, OW) = w.shape[0], smap.shape[:2]
    P = 0 if iw is None else iw.shape[-1]
    y = torch.full((B, Co, OH, OW), float("nan"), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.mcx_conv_forward_static(
            x.data_ptr(), smap.data_ptr(), None if iw is None else iw.data_ptr(), w.data_ptr(),
            b.data_ptr(), y.data_ptr(), B, Ci, Co, IH, IW, OH, OW, K, P, interp,
            _C._DTYPES[x.dtype], torch.cuda.current_stream(x.device).cuda_stream)
    return rc, y


def _problem(seed, B, Ci, Co, H, W, radius, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    K = (2 * radius + 1) ** 2
    x = torch.randn(B, Ci, H, W, generator=g, dtype=torch.float64).to(dtype).cuda()
    w = (torch.randn(Co, Ci, K, generator=g, dtype=torch.float64) / (Ci * K) ** 0.5).to(dtype).cuda()
    b = torch.randn(Co, generator=g, dtype=torch.float64).to(dtype).cuda()
    smap = synthetic.latitude_map(H, W, radius, dtype=dtype if dtype != torch.bfloat16
                                  else torch.float32).cuda()
    return x, smap, w, b, K


def test_static_forward_matches_workspace_forward_twice(device):
    # first call: 2 x 40 -> 72 channels on 24 x 96, 5x5 taps; second: a smaller 3x3 problem
    for seed, shape in ((1, (2, 40, 72, 24, 96, 2)), (2, (1, 7, 9, 6, 33, 1))):
        x, smap, w, b, K = _problem(seed, *shape)
        for interp in (1, 0):
            want = _C.mapped_conv_forward(x, smap, w, b, K, interp)
            rc, got = _static_forward(x, smap, None, w, b, K, interp)
            assert rc == 0, _lib.load().mcx_error_string(rc)
            torch.cuda.synchronize()
            assert torch.equal(got, want), "shape %s interp %d" % (shape, interp)


def test_static_forward_weighted_and_fp64(device):
    g = torch.Generator().manual_seed(3)
    B, Ci, Co, IH, IW, OH, OW, K, P = 2, 5, 7, 9, 11, 6, 10, 5, 3
    for dtype in (torch.float32, torch.float64):
        x = torch.randn(B, Ci, IH, IW, generator=g, dtype=torch.float64).to(dtype).cuda()
        smap, iw = helpers.random_map(g, OH, OW, K, P, IH, IW, dtype)
        w = torch.randn(Co, Ci, K, generator=g, dtype=torch.float64).to(dtype).cuda()
        b = torch.randn(Co, generator=g, dtype=torch.float64).to(dtype).cuda()
        smap, iw = smap.cuda(), iw.cuda()
        for interp in (0, 2):
            want = _C.weighted_mapped_conv_forward(x, smap, iw, w, b, K, interp)
            rc, got = _static_forward(x, smap, iw, w, b, K, interp)
            assert rc == 0
            assert torch.equal(got, want)


def test_static_forward_rejects_what_does_not_fit(device):
    lib = _lib.load()
    # bf16 storage stages a copy of the input: far beyond the array at this size
    x, smap, w, b, K = _problem(4, 8, 64, 64, 256, 512, 1, torch.bfloat16)
    need = lib.mcx_conv_forward_workspace(8, 64, 64, 256, 512, 256, 512, K, 0, _lib.MCX_BF16)
    assert need > (8 << 20)
    rc, _ = _static_forward(x, smap, None, w, b, K, 1)
    assert rc == -5 and b"static" in lib.mcx_error_string(rc)
    # the headline fp32 shape fits
    x, smap, w, b, K = _problem(5, 1, 64, 64, 256, 512, 1)
    rc, got = _static_forward(x, smap, None, w, b, K, 1)
    assert rc == 0
    assert torch.equal(got, _C.mapped_conv_forward(x, smap, w, b, K, 1))
