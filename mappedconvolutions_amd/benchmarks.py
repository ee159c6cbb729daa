"""Secondary workloads of the mapped-convolution hot path, timed on one GPU.

    python -m mappedconvolutions_amd.benchmarks [name ...]

Each workload is one of the reference configurations other than the headline one
(which `bench.py` at the repository root measures): the weighted mesh convolution,
the cube-to-equirectangular resampling with pooling, KNN, the encoder-scale
bf16 convolution, and the sample-map builders.  For every op the script prints one JSON line with the time per
call (events on the launch stream, inputs resident in HBM), the algorithmic bytes
or flops of the call and the fraction of the MI355X roofline that bounds it.
"""
import json
import sys

import torch

from . import _C
from .util import synthetic

HBM_GBS = 8000.0
FP32_MFMA_TFLOPS = 157.3
BF16_MFMA_TFLOPS = 2500.0
FP32_VALU_TFLOPS = 157.3  # vector fp32 FMA peak (packed); KNN is bound by it


def _time(fn, iters=10, warmup=2):
    """ms per call: `warmup` calls, untimed loops of `iters` for at least 80 ms (after a change
    of workload the GPU runs at a lower clock for some tens of milliseconds: up to 10 % slower),
    then the timed loop."""
    import time
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    while True:
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 >= 0.08:
            break
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def _line(name, ms, nbytes=None, flops=None, peak_tflops=FP32_MFMA_TFLOPS, bound="mfma", **extra):
    out = {"workload": name, "ms": round(ms, 4)}
    if nbytes is not None:
        gbs = nbytes / (ms * 1e-3) / 1e9
        out.update(bound="hbm", algorithmic_MB=round(nbytes / 1e6, 1), achieved_GBs=round(gbs, 1),
                   frac=round(gbs / HBM_GBS, 4))
    if flops is not None:
        tf = flops / (ms * 1e-3) / 1e12
        out.update(bound=bound, peak_TFLOPs=peak_tflops, GFLOP=round(flops / 1e9, 2),
                   achieved_TFLOPs=round(tf, 2), frac=round(tf / peak_tflops, 4))
    out.update(extra)
    print(json.dumps(out), flush=True)


def config3(dev):
    """Weighted mesh convolution: [4, 64, 1, 40962] -> 128 channels, K=7, P=4, nearest."""
    B, Ci, Co, V, K, P = 4, 64, 128, 40962, 7, 4
    smap, iw = synthetic.mesh_weighted_map(V, K, P)
    smap, iw = smap.to(dev), iw.to(dev)
    g = torch.Generator().manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16):
        x = torch.randn(B, Ci, 1, V, generator=g).to(dev, dtype)
        w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dev, dtype)
        b = torch.zeros(Co, device=dev, dtype=dtype)
        gy = torch.randn(B, Co, 1, V, generator=g).to(dev, dtype)
        flop = 2.0 * B * V * Co * Ci * K
        tag = "config3 weighted mesh conv %s" % str(dtype).split(".")[-1]
        peak = BF16_MFMA_TFLOPS if dtype == torch.bfloat16 else FP32_MFMA_TFLOPS
        _line(tag + " forward",
              _time(lambda: _C.weighted_mapped_conv_forward(x, smap, iw, w, b, K, 0)), flops=flop,
              peak_tflops=peak)
        _line(tag + " backward",
              _time(lambda: _C.weighted_mapped_conv_backward(gy, smap, iw, x, w, b, K, 0)),
              flops=2 * flop, peak_tflops=peak)


def config4(dev):
    """Cube -> equirect resampling (scatter + gather), pools, unpools on 512x1024."""
    B, C, F, H, W = 4, 64, 256, 512, 1024
    g = torch.Generator().manual_seed(0)
    cube = torch.rand(B, C, F, 6 * F, generator=g).to(dev)
    cmap = synthetic.cube_to_equirect_map(F, H, W).to(dev)
    eq = torch.rand(B, C, H, W, generator=g).to(dev)
    lmap = synthetic.latitude_map(H, W, 1).to(dev)
    fb = 4
    n_cube, n_eq = cube.numel() * fb, eq.numel() * fb
    for name, code in (("bilinear", 1), ("bispherical", 2)):
        _line("config4 resample_to_map %s" % name,
              _time(lambda: _C.resample_to_map(cube, cmap, H, W, code)),
              nbytes=n_cube + n_eq + cmap.numel() * fb)
        _line("config4 resample_from_map %s (Unresample forward)" % name,
              _time(lambda: _C.resample_from_map(eq, cmap, code)),
              nbytes=n_cube + n_eq + cmap.numel() * fb)
    mbytes = lmap.numel() * fb
    _line("config4 mapped_avg_pool K9", _time(lambda: _C.mapped_avg_pool(eq, lmap, 9, 1)),
          nbytes=2 * n_eq + mbytes)
    _line("config4 mapped_max_pool K9", _time(lambda: _C.mapped_max_pool(eq, lmap, 9, 1)),
          nbytes=2 * n_eq + 2 * n_eq + mbytes)
    pooled, idx = _C.mapped_max_pool(eq, lmap, 9, 1)
    _line("config4 mapped_avg_unpool K9",
          _time(lambda: _C.mapped_avg_unpool(eq, lmap, H, W, 9, 1)), nbytes=2 * n_eq + mbytes)
    _line("config4 mapped_max_unpool K9",
          _time(lambda: _C.mapped_max_unpool(eq, idx, lmap, H, W, 9, 1)),
          nbytes=2 * n_eq + 2 * n_eq + mbytes)


def knn(dev):
    """k=8 nearest of 40962 reference points for 524288 queries on the unit sphere: the grid
    search `knn_forward` uses (bytes: points in, indices and distances out), and the walk over
    all reference points it replaces (8 flop per pair of points) through the C ABI."""
    import ctypes

    from . import _lib
    ref = synthetic.sphere_points(40962, seed=1).to(dev)
    qry = synthetic.sphere_points(524288, seed=2).to(dev)
    Q, R, k = 524288, 40962, 8
    _line("config4 knn k=8 Q=524288 R=40962 (grid search)",
          _time(lambda: _C.knn_forward(ref, qry, k), iters=5, warmup=1),
          nbytes=(Q + R) * 3 * 4 + Q * k * (8 + 4))
    lib = _lib.load()
    idx = torch.empty(1, k, Q, dtype=torch.int64, device=dev)
    dist = torch.empty(1, k, Q, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _line("config4 knn k=8 Q=524288 R=40962 (walk over all points, no workspace)",
          _time(lambda: lib.mcx_knn(ref.data_ptr(), qry.data_ptr(), idx.data_ptr(),
                                    dist.data_ptr(), None, 0, 1, 3, R, Q, k, 0, stream),
                iters=3, warmup=1),
          flops=8.0 * Q * R, peak_tflops=FP32_VALU_TFLOPS, bound="valu")


def config5(dev):
    """Encoder-scale convolution, bf16 storage: B=16, 128->128, 512x1024, 5x5 bilinear."""
    B, C, H, W, K = 16, 128, 512, 1024, 25
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, C, H, W, generator=g, dtype=torch.bfloat16).to(dev)
    gy = torch.randn(B, C, H, W, generator=g, dtype=torch.bfloat16).to(dev)
    w = (torch.randn(C, C, K, generator=g) / (C * K) ** 0.5).to(dev, torch.bfloat16)
    b = torch.zeros(C, device=dev, dtype=torch.bfloat16)
    smap = synthetic.latitude_map(H, W, 2).to(dev)
    flop = 2.0 * B * H * W * C * C * K
    _line("config5 bf16 conv forward (bf16 MFMA, fp32 accumulate)",
          _time(lambda: _C.mapped_conv_forward(x, smap, w, b, K, 1), iters=3, warmup=1), flops=flop,
          peak_tflops=BF16_MFMA_TFLOPS)
    _line("config5 bf16 conv backward (bf16 MFMA, fp32 accumulate)",
          _time(lambda: _C.mapped_conv_backward(gy, smap, x, w, b, K, 1), iters=3, warmup=1),
          flops=2 * flop, peak_tflops=BF16_MFMA_TFLOPS)


def maps(dev):
    """Map builders at the encoder scale (512x1024, 5x5) and cube2rect of config 4's cube."""
    from .util import (cube_to_rect, get_projection_map, get_reverse_cube_projection_map)
    H, W, ks = 512, 1024, (5, 5)
    out_bytes = H * W * 25 * 2 * 4
    for proj in ("gnomonic", "equirectangular"):
        _line("projection map %s 512x1024 5x5" % proj,
              _time(lambda: get_projection_map((H, W), ks, proj, device=dev)), nbytes=out_bytes)
    _line("cube projection map dim 256 3x3",
          _time(lambda: get_reverse_cube_projection_map(256, (3, 3), device=dev)),
          nbytes=256 * 1536 * 9 * 2 * 4)
    # the real maps of a mesh convolution at config 3's size: 7 taps at each of 40962 vertices
    from .util import gnomonic_kernel, convert_3d_to_spherical
    verts, faces = synthetic.subdivided_icosahedron(6)
    verts, faces = verts.to(dev), faces.to(dev)
    samples = gnomonic_kernel(convert_3d_to_spherical(verts), 1, 7, 0.02, 0.02).contiguous()
    n, f = samples.numel() // 2, faces.shape[0]
    _line("planar conv operator: %d samples x %d faces" % (n, f),
          _time(lambda: _C.planar_conv_operator_from_samples(samples, verts, faces, True, False),
                iters=3, warmup=1),
          flops=6.0 * n * f, peak_tflops=FP32_VALU_TFLOPS, bound="valu")
    cube = torch.rand(64, 256, 6 * 256, device=dev)
    for interp in ("nearest", "bilinear"):
        _line("cube2rect %s C=64 dim 256 -> 512x1024" % interp,
              _time(lambda: cube_to_rect(cube, H, W, interp)),
              nbytes=cube.numel() * 4 + 64 * H * W * 4)


def plans(dev):
    """The same calls with map plans (built once, outside the timed region): config 4's scatter
    ops through scatter_map_plan, the headline convolution through conv_map_plan."""
    B, C, F, H, W = 4, 64, 256, 512, 1024
    g = torch.Generator().manual_seed(0)
    cube = torch.rand(B, C, F, 6 * F, generator=g).to(dev)
    cmap = synthetic.cube_to_equirect_map(F, H, W).to(dev)
    eq = torch.rand(B, C, H, W, generator=g).to(dev)
    lmap = synthetic.latitude_map(H, W, 1).to(dev)
    fb = 4
    n_cube, n_eq = cube.numel() * fb, eq.numel() * fb
    plan = _C.scatter_map_plan(cmap, None, H, W, 1)
    _line("planned config4 resample_to_map bilinear",
          _time(lambda: _C.resample_to_map(cube, cmap, H, W, 1, plan=plan)),
          nbytes=n_cube + n_eq + plan.numel())
    _, idx = _C.mapped_max_pool(eq, lmap, 9, 1)
    plan_a = _C.scatter_map_plan(lmap, None, H, W, 1)
    plan_m = _C.scatter_map_plan(lmap, None, H, W, 1, for_max_unpool=True)
    _line("planned config4 mapped_avg_unpool K9",
          _time(lambda: _C.mapped_avg_unpool(eq, lmap, H, W, 9, 1, plan=plan_a)),
          nbytes=2 * n_eq + plan_a.numel())
    _line("planned config4 mapped_max_unpool K9",
          _time(lambda: _C.mapped_max_unpool(eq, idx, lmap, H, W, 9, 1, plan=plan_m)),
          nbytes=2 * n_eq + 2 * n_eq + plan_m.numel())
    del cube, eq, idx
    B, C, H, W, K = 8, 64, 256, 512, 9
    x = torch.randn(B, C, H, W, generator=g).to(dev)
    gy = torch.randn(B, C, H, W, generator=g).to(dev)
    w = (torch.randn(C, C, K, generator=g) / (C * K) ** 0.5).to(dev)
    b = torch.zeros(C, device=dev)
    smap = synthetic.latitude_map(H, W, 1).to(dev)
    cplan = _C.conv_map_plan(smap, None, H, W, 1)
    flop = 2.0 * B * H * W * C * C * K
    _line("planned headline conv forward fp32",
          _time(lambda: _C.mapped_conv_forward(x, smap, w, b, K, 1, plan=cplan)), flops=flop)
    _line("unplanned headline conv forward fp32",
          _time(lambda: _C.mapped_conv_forward(x, smap, w, b, K, 1)), flops=flop)
    _line("planned headline conv backward fp32",
          _time(lambda: _C.mapped_conv_backward(gy, smap, x, w, b, K, 1, plan=cplan)),
          flops=2 * flop)
    _line("unplanned headline conv backward fp32",
          _time(lambda: _C.mapped_conv_backward(gy, smap, x, w, b, K, 1)), flops=2 * flop)
    del x, gy, w, b, smap, cplan
    B, C, H, W, K = 16, 128, 512, 1024, 25
    bf = torch.bfloat16
    x = torch.randn(B, C, H, W, generator=g, dtype=bf).to(dev)
    gy = torch.randn(B, C, H, W, generator=g, dtype=bf).to(dev)
    w = (torch.randn(C, C, K, generator=g) / (C * K) ** 0.5).to(dev, bf)
    b = torch.zeros(C, device=dev, dtype=bf)
    smap = synthetic.latitude_map(H, W, 2).to(dev)
    cplan = _C.conv_map_plan(smap, None, H, W, 1, bf)
    flop = 2.0 * B * H * W * C * C * K
    _line("planned config5 bf16 conv forward",
          _time(lambda: _C.mapped_conv_forward(x, smap, w, b, K, 1, plan=cplan)),
          flops=flop, peak_tflops=BF16_MFMA_TFLOPS)
    _line("planned config5 bf16 conv backward",
          _time(lambda: _C.mapped_conv_backward(gy, smap, x, w, b, K, 1, plan=cplan)),
          flops=2 * flop, peak_tflops=BF16_MFMA_TFLOPS)


def _launches(fn):
    """Kernel launches of one call, counted by torch's profiler (0 when it cannot tell)."""
    try:
        from torch.profiler import ProfilerActivity, profile
        fn()
        torch.cuda.synchronize()
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            fn()
            torch.cuda.synchronize()
        return sum(1 for e in prof.events() if e.device_type.name == "CUDA" and
                   "memcpy" not in e.name.lower() and "memset" not in e.name.lower())
    except Exception:  # noqa: BLE001 - the count is an extra, the timing is the result
        return 0


def small(dev):
    """Latency at small shapes.  Configuration 1 (B=1, 16 -> 32 channels, 64 x 128, 3 x 3
    latitude map, bilinear, fp32) and the reference's own size sweep
    (profile/profile_mapped_convolution.py:45-57: B=1, 10 -> 1 channels, K=9, bilinear over a
    pixel-shuffle map, 10 x 10 ... 2000 x 2500) in the reference's float64 (scalar kernels
    here) and in float32 (matrix-core kernels), next to the library's plain 3 x 3 convolution
    the reference times beside it.  Microseconds per call and kernel launches per call."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(0)
    B, Ci, Co, H, W, K = 1, 16, 32, 64, 128, 9
    x = torch.randn(B, Ci, H, W, generator=g).to(dev)
    w = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dev)
    b = torch.zeros(Co, device=dev)
    gy = torch.randn(B, Co, H, W, generator=g).to(dev)
    smap = synthetic.latitude_map(H, W, 1).to(dev)
    plan = _C.conv_map_plan(smap, None, H, W, 1)
    for tag, pl in (("", None), (" with a map plan", plan)):
        fwd = lambda: _C.mapped_conv_forward(x, smap, w, b, K, 1, plan=pl)
        bwd = lambda: _C.mapped_conv_backward(gy, smap, x, w, b, K, 1, plan=pl)
        _line("config1 conv forward fp32 B1 16->32 64x128 K9" + tag, _time(fwd, iters=50),
              flops=2.0 * B * H * W * Co * Ci * K, launches=_launches(fwd))
        _line("config1 conv backward fp32" + tag, _time(bwd, iters=50),
              flops=4.0 * B * H * W * Co * Ci * K, launches=_launches(bwd))
    sizes = [(10, 10), (20, 25), (20, 50), (50, 100), (100, 100), (200, 250), (200, 500),
             (500, 1000), (1000, 1000), (2000, 2500)]
    Ci, Co = 10, 1
    for dtype in (torch.float64, torch.float32):
        name = str(dtype).split(".")[-1]
        wgt = (torch.randn(Co, Ci, K, generator=g) / (Ci * K) ** 0.5).to(dev, dtype)
        bias = torch.zeros(Co, device=dev, dtype=dtype)
        for (h, wd) in sizes:
            data = torch.randn(1, Ci, h, wd, generator=g).to(dev, dtype)
            gout = torch.rand(1, Co, h, wd, generator=g).to(dev, dtype)
            m = synthetic.pixel_shuffle_map(h, wd, 1, dtype).to(dev)
            w33 = wgt.view(Co, Ci, 3, 3)
            fwd = lambda: _C.mapped_conv_forward(data, m, wgt, bias, K, 1)
            bwd = lambda: _C.mapped_conv_backward(gout, m, data, wgt, bias, K, 1)
            it = 50 if h * wd <= 250000 else 10
            print(json.dumps({
                "workload": "sweep %s %dx%d B1 10->1 K9 bilinear pixel-shuffle map" % (name, h, wd),
                "mapped_forward_us": round(_time(fwd, iters=it) * 1e3, 1),
                "mapped_backward_us": round(_time(bwd, iters=it) * 1e3, 1),
                "plain_conv_forward_us": round(
                    _time(lambda: F.conv2d(data, w33, bias, padding=1), iters=it) * 1e3, 1),
                "launches_forward": _launches(fwd), "launches_backward": _launches(bwd)}),
                flush=True)


WORKLOADS = {"small": small, "config3": config3, "config4": config4, "knn": knn, "config5": config5,
             "maps": maps, "plans": plans}


def main(argv):
    names = argv or list(WORKLOADS)
    dev = torch.device("cuda:0")
    for n in names:
        WORKLOADS[n](dev)


if __name__ == "__main__":
    main(sys.argv[1:])
