"""The extension-op boundary of the mapped-convolution backend.

Same op names, argument order and return values as the reference's pybind
modules under `_mapped_convolution_ext` (one module per op family there, one
namespace here); each function checks its tensors like the reference's
include/nn/layers/*.h wrappers do, allocates the outputs with torch, and calls
the C ABI of libmcx_hip.so on the current HIP stream.  Tensors must live on the
GPU: there is no CPU implementation behind these names.
"""
import torch

from . import _lib
from ._lib import MCX_BF16, MCX_F32, MCX_F64

_DTYPES = {torch.float32: MCX_F32, torch.float64: MCX_F64, torch.bfloat16: MCX_BF16}


# Optional timing hook: when set to a list, every C-ABI call made by the convolution
# ops appends (label, start_event, end_event), recorded on the stream the kernels
# are enqueued on.  Used by the benchmark to time individual kernels.
profile_events = None
profile_pool = []  # pre-made (start, end) event pairs, see make_event_pool

# resample_to_map and the unpoolings run as gathers through a transposed map when
# given a workspace; False selects the library's atomic-scatter form instead.
scatter_as_gather = True


def make_event_pool(n, device):
    """n pairs of timing events whose underlying handles exist (an event gets its handle at
    its first record), for `profile_pool`."""
    stream = torch.cuda.current_stream(device)
    pool = []
    for _ in range(n):
        pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        for e in pair:
            e.record(stream)
        pool.append(pair)
    return pool


def _timed(label, device, fn):
    """Run one C-ABI call; with `profile_events` set and a pair left in `profile_pool`, ask
    the library to record the pair around the call's dominant kernel (the only cost inside
    a timed region: one extra C call and two event records)."""
    if profile_events is None or not profile_pool:
        return fn()
    start, end = profile_pool.pop()
    lib = _lib.load()
    lib.mcx_profile_dominant_kernel(start.cuda_event, end.cuda_event)
    rc = fn()
    lib.mcx_profile_dominant_kernel(None, None)
    profile_events.append((label, start, end))
    return rc


def _contig(**tensors):
    for name, t in tensors.items():
        if t is not None and not t.is_contiguous():
            raise RuntimeError("%s must be contiguous" % name)


def _on_gpu(ref_name, ref, **tensors):
    if not ref.is_cuda:
        raise RuntimeError(
            "%s must be a GPU tensor: this backend has no CPU implementation" % ref_name)
    for name, t in tensors.items():
        if t is not None and t.device != ref.device:
            raise RuntimeError("%s must be on the same device as %s" % (name, ref_name))


def _dtype(data, maps=(), same=()):
    """Data dtype code.  Maps share the data's dtype (the reference's rule,
    layers/nn/layer_utils.py:21-30), except bf16 data which takes fp32 maps
    because bf16 cannot hold pixel coordinates above 256 exactly."""
    if data.dtype not in _DTYPES:
        raise RuntimeError("unsupported dtype %s" % data.dtype)
    want_map = torch.float32 if data.dtype == torch.bfloat16 else data.dtype
    for m in maps:
        if m is not None and m.dtype != want_map:
            raise RuntimeError("sample_map / interp_weights must be %s for %s data (got %s)" %
                               (want_map, data.dtype, m.dtype))
    for t in same:
        if t is not None and t.dtype != data.dtype:
            raise RuntimeError("tensor dtypes differ: %s vs %s" % (t.dtype, data.dtype))
    return _DTYPES[data.dtype]


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _workspace(nbytes, device):
    """Scratch for one call (torch's caching allocator returns 512-byte aligned blocks)."""
    return torch.empty((max(int(nbytes), 1),), dtype=torch.uint8, device=device)


def _weighted_dims(sample_map, interp_weights, kernel):
    """Number of interpolation points P (0 = unweighted) after a shape check."""
    want = (4 if kernel else 3) + (0 if interp_weights is None else 1)
    if sample_map.dim() != want or sample_map.shape[-1] != 2:
        raise RuntimeError("sample_map has shape %s, expected %d dims ending in 2" %
                           (tuple(sample_map.shape), want))
    if interp_weights is None:
        return 0
    if tuple(interp_weights.shape) != tuple(sample_map.shape[:-1]):
        raise RuntimeError("interp_weights shape %s does not match sample_map %s" %
                           (tuple(interp_weights.shape), tuple(sample_map.shape)))
    return int(interp_weights.shape[-1])


# --------------------------------------------------------------------------- conv
def _conv_forward(input, sample_map, interp_weights, weight, bias, kernel_size, interpolation,
                  plan=None):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
            bias=bias)
    _on_gpu("input", input, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
            bias=bias)
    dt = _dtype(input, maps=(sample_map, interp_weights), same=(weight, bias))
    P = _weighted_dims(sample_map, interp_weights, True)
    B, Ci, IH, IW = input.shape
    Co = weight.shape[0]
    OH, OW, K = sample_map.shape[0], sample_map.shape[1], int(kernel_size)
    if weight.dim() != 3 or weight.shape[1] != Ci or weight.shape[2] != K or sample_map.shape[2] != K:
        raise RuntimeError("weight %s / sample_map %s do not match input channels %d, kernel %d" %
                           (tuple(weight.shape), tuple(sample_map.shape), Ci, K))
    if bias.numel() != Co:
        raise RuntimeError("bias must have %d elements" % Co)
    out = torch.empty((B, Co, OH, OW), dtype=input.dtype, device=input.device)
    lib = _lib.load()
    ws_bytes = lib.mcx_conv_forward_workspace(B, Ci, Co, IH, IW, OH, OW, K, P, dt)
    ws = _workspace(ws_bytes, input.device)
    if plan is None and map_plan_cache is not None:
        plan = _cached_plan(sample_map, interp_weights, IH, IW, interpolation, input.dtype)
    plan_ptr, plan_bytes, plan_desc = _plan_args(plan)
    with torch.cuda.device(input.device):
        rc = _timed("conv_forward", input.device, lambda: lib.mcx_conv_forward_planned(
            _ptr(input), _ptr(sample_map), _ptr(interp_weights), _ptr(weight), _ptr(bias),
            _ptr(out), _ptr(ws), ws_bytes, plan_ptr, plan_bytes, plan_desc, B, Ci, Co, IH, IW, OH,
            OW, K, P, int(interpolation), dt, _stream(input)))
    _lib.check(rc, "mapped_conv_forward")
    return out


# ---- map plans (no counterpart in the reference) ------------------------------------
# What the operators derive from sample_map alone can be built once and reused while the map
# does not change: for the (transposed) convolutions the transposed map of the scatter
# direction, the resolved taps of the gather direction and the masks of pairs in use
# (`conv_map_plan`); for resample_to_map and the unpoolings the sorted per-destination lists of
# contributions (`scatter_map_plan`).  With `map_plan_cache` set to a dict (see
# enable_map_plan_cache) the ops keep the plans of the maps they have seen, keyed by the
# tensors' storage and in-place version counters.  Off by default: every call then rebuilds
# what it needs, like the reference.
map_plan_cache = None
_MAP_PLAN_CACHE_ENTRIES = 16


class MapPlan:
    """A map plan: the device buffer, the host-side descriptor the library checks it by
    (mcx_plan_desc: op family, interpolation, sizes, the addresses of the plan and of the map it
    was built from) and the map tensors themselves, kept alive so that their addresses cannot
    pass to other tensors while the plan exists."""
    __slots__ = ("buffer", "desc", "tensors")

    def __init__(self, buffer, desc, tensors):
        self.buffer, self.desc, self.tensors = buffer, desc, tensors

    def numel(self):
        return self.buffer.numel()


def _plan_args(plan):
    """(device pointer, bytes, descriptor) of a MapPlan for the C ABI; NULLs for None."""
    if plan is None:
        return None, 0, None
    if not isinstance(plan, MapPlan):
        raise RuntimeError("plan must come from conv_map_plan / scatter_map_plan / pool_map_plan")
    import ctypes
    return plan.buffer.data_ptr(), plan.buffer.numel(), ctypes.byref(plan.desc)


def enable_map_plan_cache(enabled=True):
    """Keep (or stop keeping) the plans of the sample maps seen by the convolution backward."""
    global map_plan_cache
    map_plan_cache = {} if enabled else None


def conv_map_plan(sample_map, interp_weights, input_height, input_width, interpolation,
                  data_dtype=torch.float32):
    """Plan of one sample_map [MH, MW, K, (P,) 2] that samples an image of input_height x
    input_width: a MappedConvolution's input, or a MappedTransposedConvolution's OUTPUT.  None
    where the library has no plan for the case (float64 data, P > 4).  Pass it as `plan=` to
    the forward and backward ops of that layer for as long as the map's contents stay the
    same."""
    _contig(sample_map=sample_map, interp_weights=interp_weights)
    _on_gpu("sample_map", sample_map, interp_weights=interp_weights)
    P = _weighted_dims(sample_map, interp_weights, True)
    OH, OW, K = sample_map.shape[:3]
    dt = _DTYPES[data_dtype]
    want = torch.float32 if data_dtype == torch.bfloat16 else data_dtype
    if sample_map.dtype != want:
        raise RuntimeError("sample_map must be %s for %s data" % (want, data_dtype))
    lib = _lib.load()
    IH, IW = int(input_height), int(input_width)
    nbytes = lib.mcx_conv_plan_bytes(IH, IW, OH, OW, K, P, dt)
    if nbytes == 0:
        return None
    plan = torch.empty((nbytes,), dtype=torch.uint8, device=sample_map.device)
    desc = _lib.PlanDesc()
    with torch.cuda.device(sample_map.device):
        rc = lib.mcx_conv_plan_build(_ptr(sample_map), _ptr(interp_weights), _ptr(plan), nbytes,
                                     desc, IH, IW, OH, OW, K, P, int(interpolation), dt,
                                     _stream(sample_map))
    _lib.check(rc, "conv_map_plan")
    return MapPlan(plan, desc, (sample_map, interp_weights))


def _cached_plan(sample_map, interp_weights, IH, IW, interpolation, data_dtype, kind="conv",
                 **scatter_args):
    """Plan from the cache, rebuilt when a tensor was modified in place or replaced."""
    def ident(t):
        return None if t is None else (t.data_ptr(), t._version, tuple(t.shape))
    key = (kind, ident(sample_map), ident(interp_weights), IH, IW, int(interpolation), data_dtype,
           sample_map.device.index)
    hit = map_plan_cache.get(key)
    if hit is not None:
        return hit[0]
    if kind == "conv":
        plan = conv_map_plan(sample_map, interp_weights, IH, IW, interpolation, data_dtype)
    else:
        plan = scatter_map_plan(sample_map, interp_weights, IH, IW, interpolation,
                                for_max_unpool=kind == "max_unpool", **scatter_args)
    if len(map_plan_cache) >= _MAP_PLAN_CACHE_ENTRIES:
        map_plan_cache.pop(next(iter(map_plan_cache)))
    # the entry keeps the tensors alive, so their addresses cannot be handed to other maps
    map_plan_cache[key] = (plan, sample_map, interp_weights)
    return plan


def _conv_backward(grad_output, sample_map, interp_weights, input, weight, bias, kernel_size,
                   interpolation, plan=None, needs=(True, True, True)):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
            bias=bias)
    grad_output = grad_output.contiguous()  # the reference reads it raw without a check
    _on_gpu("grad_output", grad_output, input=input, sample_map=sample_map,
            interp_weights=interp_weights, weight=weight, bias=bias)
    dt = _dtype(input, maps=(sample_map, interp_weights), same=(weight, grad_output))
    P = _weighted_dims(sample_map, interp_weights, True)
    B, Ci, IH, IW = input.shape
    Co, OH, OW = grad_output.shape[1], grad_output.shape[2], grad_output.shape[3]
    K = int(kernel_size)
    if tuple(weight.shape) != (Co, Ci, K) or tuple(sample_map.shape[:3]) != (OH, OW, K):
        raise RuntimeError("shape mismatch in mapped_conv_backward")
    # `needs` (grad_input, grad_weight, grad_bias): a gradient nobody asked for is not
    # computed (the C ABI takes NULL for it) and comes back as None
    grad_input = torch.empty_like(input) if needs[0] else None
    grad_weight = torch.empty_like(weight) if needs[1] else None
    grad_bias = torch.empty((Co,), dtype=input.dtype, device=input.device) if needs[2] else None
    lib = _lib.load()
    ws_bytes = lib.mcx_conv_backward_workspace(B, Ci, Co, IH, IW, OH, OW, K, P, dt)
    ws = _workspace(ws_bytes, input.device)
    if plan is None and map_plan_cache is not None:
        plan = _cached_plan(sample_map, interp_weights, IH, IW, interpolation, input.dtype)
    plan_ptr, plan_bytes, plan_desc = _plan_args(plan)
    # Two C-ABI calls (NULL skips a gradient) so that the input gradient and the weight
    # gradient can be timed alone; the bias gradient rides on the weight gradient's pass
    # over grad_output.
    outs = {"conv_backward_input": (grad_input, None, None),
            "conv_backward_weight": (None, grad_weight, grad_bias)}
    with torch.cuda.device(input.device):
        for label, (gx, gw, gb) in outs.items():
            if gx is None and gw is None and gb is None:
                continue
            rc = _timed(label, input.device, lambda: lib.mcx_conv_backward_planned(
                _ptr(grad_output), _ptr(sample_map), _ptr(interp_weights), _ptr(input),
                _ptr(weight), _ptr(gx), _ptr(gw), _ptr(gb), _ptr(ws), ws_bytes, plan_ptr,
                plan_bytes, plan_desc, B, Ci, Co, IH, IW, OH, OW, K, P, int(interpolation), dt,
                _stream(input)))
            _lib.check(rc, "mapped_conv_backward")
    return [grad_input, grad_weight, grad_bias]


def mapped_conv_forward(input, sample_map, weight, bias, kernel_size, interpolation, plan=None):
    """include/nn/layers/mapped_convolution_layer.h:64-66.  `plan` (optional, not in the
    reference): see conv_map_plan."""
    return _conv_forward(input, sample_map, None, weight, bias, kernel_size, interpolation, plan)


def mapped_conv_backward(grad_output, sample_map, input, weight, bias, kernel_size, interpolation,
                         plan=None, needs=(True, True, True)):
    """include/nn/layers/mapped_convolution_layer.h:90-93 -> [grad_input, grad_weight, grad_bias].
    `plan` (optional, not in the reference): see conv_map_plan.  `needs` (optional, not in the
    reference): which of the three gradients to compute; the others come back as None."""
    return _conv_backward(grad_output, sample_map, None, input, weight, bias, kernel_size,
                          interpolation, plan, needs)


def weighted_mapped_conv_forward(input, sample_map, interp_weights, weight, bias, kernel_size,
                                 interpolation, plan=None):
    """include/nn/layers/weighted_mapped_convolution_layer.h:65-68.  `plan`: see conv_map_plan."""
    return _conv_forward(input, sample_map, interp_weights, weight, bias, kernel_size,
                         interpolation, plan)


def weighted_mapped_conv_backward(grad_output, sample_map, interp_weights, input, weight, bias,
                                  kernel_size, interpolation, plan=None,
                                  needs=(True, True, True)):
    """include/nn/layers/weighted_mapped_convolution_layer.h:97-100.  `plan`: see conv_map_plan;
    `needs`: see mapped_conv_backward."""
    return _conv_backward(grad_output, sample_map, interp_weights, input, weight, bias,
                          kernel_size, interpolation, plan, needs)


# ---------------------------------------------------------------- transposed conv
def _tconv_forward(input, sample_map, interp_weights, weight, bias, output_height, output_width,
                   kernel_size, interpolation, plan=None):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
            bias=bias)
    _on_gpu("input", input, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
            bias=bias)
    dt = _dtype(input, maps=(sample_map, interp_weights), same=(weight, bias))
    P = _weighted_dims(sample_map, interp_weights, True)
    B, Ci, IH, IW = input.shape
    Co, K = weight.shape[1], int(kernel_size)
    OH, OW = int(output_height), int(output_width)
    if tuple(weight.shape) != (Ci, Co, K) or tuple(sample_map.shape[:3]) != (IH, IW, K):
        raise RuntimeError("shape mismatch in mapped_transposed_conv_forward")
    out = torch.empty((B, Co, OH, OW), dtype=input.dtype, device=input.device)
    lib = _lib.load()
    ws_bytes = lib.mcx_tconv_forward_workspace(B, Ci, Co, IH, IW, OH, OW, K, P, dt)
    ws = _workspace(ws_bytes, input.device)
    if plan is None and map_plan_cache is not None:
        plan = _cached_plan(sample_map, interp_weights, OH, OW, interpolation, input.dtype)
    plan_ptr, plan_bytes, plan_desc = _plan_args(plan)
    with torch.cuda.device(input.device):
        rc = lib.mcx_tconv_forward_planned(_ptr(input), _ptr(sample_map), _ptr(interp_weights),
                                           _ptr(weight), _ptr(bias), _ptr(out), _ptr(ws),
                                           ws_bytes, plan_ptr, plan_bytes, plan_desc, B, Ci, Co,
                                           IH, IW, OH, OW, K, P, int(interpolation), dt,
                                           _stream(input))
    _lib.check(rc, "mapped_transposed_conv_forward")
    return out


def _tconv_backward(grad_output, sample_map, interp_weights, input, weight, bias, kernel_size,
                    interpolation, plan=None, needs=(True, True, True)):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
            bias=bias)
    grad_output = grad_output.contiguous()
    _on_gpu("grad_output", grad_output, input=input, sample_map=sample_map,
            interp_weights=interp_weights, weight=weight, bias=bias)
    dt = _dtype(input, maps=(sample_map, interp_weights), same=(weight, grad_output))
    P = _weighted_dims(sample_map, interp_weights, True)
    B, Ci, IH, IW = input.shape
    Co, OH, OW = grad_output.shape[1], grad_output.shape[2], grad_output.shape[3]
    K = int(kernel_size)
    if tuple(weight.shape) != (Ci, Co, K) or tuple(sample_map.shape[:3]) != (IH, IW, K):
        raise RuntimeError("shape mismatch in mapped_transposed_conv_backward")
    grad_input = torch.empty_like(input) if needs[0] else None
    grad_weight = torch.empty_like(weight) if needs[1] else None
    grad_bias = torch.empty((Co,), dtype=input.dtype, device=input.device) if needs[2] else None
    if not any(needs):
        return [None, None, None]
    lib = _lib.load()
    ws_bytes = lib.mcx_tconv_backward_workspace(B, Ci, Co, IH, IW, OH, OW, K, P, dt)
    ws = _workspace(ws_bytes, input.device)
    if plan is None and map_plan_cache is not None:
        plan = _cached_plan(sample_map, interp_weights, OH, OW, interpolation, input.dtype)
    plan_ptr, plan_bytes, plan_desc = _plan_args(plan)
    with torch.cuda.device(input.device):
        rc = lib.mcx_tconv_backward_planned(
            _ptr(grad_output), _ptr(sample_map), _ptr(interp_weights), _ptr(input), _ptr(weight),
            _ptr(grad_input), _ptr(grad_weight), _ptr(grad_bias), _ptr(ws), ws_bytes, plan_ptr,
            plan_bytes, plan_desc, B, Ci, Co, IH, IW, OH, OW, K, P, int(interpolation), dt,
            _stream(input))
    _lib.check(rc, "mapped_transposed_conv_backward")
    return [grad_input, grad_weight, grad_bias]


def mapped_transposed_conv_forward(input, sample_map, weight, bias, output_height, output_width,
                                   kernel_size, interpolation, plan=None):
    """include/nn/layers/mapped_transposed_convolution_layer.h:64-69.  `plan` (optional, not in
    the reference): conv_map_plan(sample_map, None, output_height, output_width, ...)."""
    return _tconv_forward(input, sample_map, None, weight, bias, output_height, output_width,
                          kernel_size, interpolation, plan)


def mapped_transposed_conv_backward(grad_output, sample_map, input, weight, bias, kernel_size,
                                    interpolation, plan=None, needs=(True, True, True)):
    """include/nn/layers/mapped_transposed_convolution_layer.h:97-100.  `needs`: see
    mapped_conv_backward."""
    return _tconv_backward(grad_output, sample_map, None, input, weight, bias, kernel_size,
                           interpolation, plan, needs)


def weighted_mapped_transposed_conv_forward(input, sample_map, interp_weights, weight, bias,
                                            output_height, output_width, kernel_size,
                                            interpolation, plan=None):
    """include/nn/layers/weighted_mapped_transposed_convolution_layer.h:64-67."""
    return _tconv_forward(input, sample_map, interp_weights, weight, bias, output_height,
                          output_width, kernel_size, interpolation, plan)


def weighted_mapped_transposed_conv_backward(grad_output, sample_map, interp_weights, input,
                                             weight, bias, kernel_size, interpolation, plan=None,
                                             needs=(True, True, True)):
    """include/nn/layers/weighted_mapped_transposed_convolution_layer.h:98-100."""
    return _tconv_backward(grad_output, sample_map, interp_weights, input, weight, bias,
                           kernel_size, interpolation, plan, needs)


def scatter_map_plan(sample_map, interp_weights, dest_height, dest_width, interpolation,
                     for_max_unpool=False, kernel=None):
    """Plan of resample_to_map (sample_map [IH, IW, (P,) 2]) or of an unpooling (sample_map
    [OH, OW, K, (P,) 2]) into an image of dest_height x dest_width: the transposed form of the
    map, built once.  `kernel`: whether the map has a tap axis (default: told from its number of
    dimensions).  A plan built with `for_max_unpool` serves mapped_max_unpool only, one built
    without it resample_to_map / mapped_avg_unpool.  Pass it as `plan=` to those ops."""
    _contig(sample_map=sample_map, interp_weights=interp_weights)
    _on_gpu("sample_map", sample_map, interp_weights=interp_weights)
    if kernel is None:
        kernel = sample_map.dim() == (4 if interp_weights is None else 5)
    P = _weighted_dims(sample_map, interp_weights, kernel)
    if sample_map.dtype not in (torch.float32, torch.float64):
        raise RuntimeError("unsupported dtype %s" % sample_map.dtype)
    dt = _DTYPES[sample_map.dtype]
    MH, MW = sample_map.shape[0], sample_map.shape[1]
    K = sample_map.shape[2] if kernel else 1
    DH, DW = int(dest_height), int(dest_width)
    lib = _lib.load()
    nbytes = lib.mcx_scatter_plan_bytes(MH, MW, DH, DW, K, P, int(interpolation), dt)
    if nbytes == 0:
        return None
    plan = torch.empty((nbytes,), dtype=torch.uint8, device=sample_map.device)
    desc = _lib.PlanDesc()
    with torch.cuda.device(sample_map.device):
        rc = lib.mcx_scatter_plan_build(_ptr(sample_map), _ptr(interp_weights), _ptr(plan), nbytes,
                                        desc, MH, MW, DH, DW, K, P, int(interpolation), dt,
                                        1 if for_max_unpool else 0, _stream(sample_map))
    _lib.check(rc, "scatter_map_plan")
    return MapPlan(plan, desc, (sample_map, interp_weights))


def _scatter_plan_for(kind, plan, sample_map, interp_weights, DH, DW, interpolation, kernel):
    if plan is None and map_plan_cache is not None and scatter_as_gather:
        plan = _cached_plan(sample_map, interp_weights, DH, DW, interpolation, sample_map.dtype,
                            kind=kind, kernel=kernel)
    return plan


# ------------------------------------------------------------------------ pooling
def _pool_dims(input, sample_map, interp_weights, kernel_size):
    if input.dim() != 4:
        raise RuntimeError("expected a 4-D [B, C, H, W] tensor, got %d dimensions" % input.dim())
    P = _weighted_dims(sample_map, interp_weights, True)
    K = int(kernel_size)
    if sample_map.shape[2] != K:
        raise RuntimeError("sample_map kernel dimension %d != kernel_size %d" %
                           (sample_map.shape[2], K))
    return P, K


def _max_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights)
    _on_gpu("input", input, sample_map=sample_map, interp_weights=interp_weights)
    dt = _dtype(input, maps=(sample_map, interp_weights))
    P, K = _pool_dims(input, sample_map, interp_weights, kernel_size)
    B, C, IH, IW = input.shape
    OH, OW = sample_map.shape[0], sample_map.shape[1]
    out = torch.empty((B, C, OH, OW), dtype=input.dtype, device=input.device)
    idx = torch.empty((B, C, OH, OW), dtype=torch.int64, device=input.device)
    with torch.cuda.device(input.device):
        rc = _lib.load().mcx_max_pool(_ptr(input), _ptr(sample_map), _ptr(interp_weights),
                                      _ptr(out), _ptr(idx), B, C, IH, IW, OH, OW, K, P,
                                      int(interpolation), dt, _stream(input))
    _lib.check(rc, "mapped_max_pool")
    return [out, idx]


def _max_unpool(grad_output, idx_mask, sample_map, interp_weights, input_height, input_width,
                kernel_size, interpolation, plan=None):
    _contig(grad_output=grad_output, idx_mask=idx_mask, sample_map=sample_map,
            interp_weights=interp_weights)
    _on_gpu("grad_output", grad_output, idx_mask=idx_mask, sample_map=sample_map,
            interp_weights=interp_weights)
    dt = _dtype(grad_output, maps=(sample_map, interp_weights))
    if idx_mask.dtype != torch.int64 or idx_mask.shape != grad_output.shape:
        raise RuntimeError("idx_mask must be int64 with grad_output's shape")
    P, K = _pool_dims(grad_output, sample_map, interp_weights, kernel_size)
    B, C, OH, OW = grad_output.shape
    if tuple(sample_map.shape[:2]) != (OH, OW):
        raise RuntimeError("sample_map spatial size must match grad_output")
    IH, IW = int(input_height), int(input_width)
    gin = torch.empty((B, C, IH, IW), dtype=grad_output.dtype, device=grad_output.device)
    lib = _lib.load()
    plan = _scatter_plan_for("max_unpool", plan, sample_map, interp_weights, IH, IW,
                             interpolation, True)
    if plan is not None:
        with torch.cuda.device(grad_output.device):
            rc = lib.mcx_max_unpool_planned(_ptr(grad_output), _ptr(idx_mask), *_plan_args(plan),
                                            _ptr(gin), B, C, IH, IW, OH, OW, K, P,
                                            int(interpolation), dt, _stream(grad_output))
        _lib.check(rc, "mapped_max_unpool")
        return gin
    ws_bytes = lib.mcx_unpool_workspace(IH, IW, OH, OW, K, P, int(interpolation), dt) \
        if scatter_as_gather else 0
    ws = _workspace(ws_bytes, grad_output.device)
    with torch.cuda.device(grad_output.device):
        rc = lib.mcx_max_unpool(_ptr(grad_output), _ptr(idx_mask), _ptr(sample_map),
                                _ptr(interp_weights), _ptr(gin), _ptr(ws), ws_bytes, B, C, IH, IW,
                                OH, OW, K, P, int(interpolation), dt, _stream(grad_output))
    _lib.check(rc, "mapped_max_unpool")
    return gin


def _avg_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights)
    _on_gpu("input", input, sample_map=sample_map, interp_weights=interp_weights)
    dt = _dtype(input, maps=(sample_map, interp_weights))
    P, K = _pool_dims(input, sample_map, interp_weights, kernel_size)
    B, C, IH, IW = input.shape
    OH, OW = sample_map.shape[0], sample_map.shape[1]
    out = torch.empty((B, C, OH, OW), dtype=input.dtype, device=input.device)
    with torch.cuda.device(input.device):
        rc = _lib.load().mcx_avg_pool(_ptr(input), _ptr(sample_map), _ptr(interp_weights),
                                      _ptr(out), B, C, IH, IW, OH, OW, K, P, int(interpolation),
                                      dt, _stream(input))
    _lib.check(rc, "mapped_avg_pool")
    return out


def _avg_unpool(grad_output, sample_map, interp_weights, input_height, input_width, kernel_size,
                interpolation, plan=None):
    _contig(grad_output=grad_output, sample_map=sample_map, interp_weights=interp_weights)
    _on_gpu("grad_output", grad_output, sample_map=sample_map, interp_weights=interp_weights)
    dt = _dtype(grad_output, maps=(sample_map, interp_weights))
    P, K = _pool_dims(grad_output, sample_map, interp_weights, kernel_size)
    B, C, OH, OW = grad_output.shape
    if tuple(sample_map.shape[:2]) != (OH, OW):
        raise RuntimeError("sample_map spatial size must match grad_output")
    IH, IW = int(input_height), int(input_width)
    gin = torch.empty((B, C, IH, IW), dtype=grad_output.dtype, device=grad_output.device)
    lib = _lib.load()
    plan = _scatter_plan_for("avg_unpool", plan, sample_map, interp_weights, IH, IW,
                             interpolation, True)
    if plan is not None:
        with torch.cuda.device(grad_output.device):
            rc = lib.mcx_avg_unpool_planned(_ptr(grad_output), *_plan_args(plan), _ptr(gin),
                                            B, C, IH, IW, OH, OW, K, P, int(interpolation), dt,
                                            _stream(grad_output))
        _lib.check(rc, "mapped_avg_unpool")
        return gin
    ws_bytes = lib.mcx_unpool_workspace(IH, IW, OH, OW, K, P, int(interpolation), dt) \
        if scatter_as_gather else 0
    ws = _workspace(ws_bytes, grad_output.device)
    with torch.cuda.device(grad_output.device):
        rc = lib.mcx_avg_unpool(_ptr(grad_output), _ptr(sample_map), _ptr(interp_weights),
                                _ptr(gin), _ptr(ws), ws_bytes, B, C, IH, IW, OH, OW, K, P,
                                int(interpolation), dt, _stream(grad_output))
    _lib.check(rc, "mapped_avg_unpool")
    return gin


def mapped_max_pool(input, sample_map, kernel_size, interpolation):
    """include/nn/layers/mapped_max_pooling_layer.h:46-49 -> [pooled, idx_mask]."""
    return _max_pool(input, sample_map, None, kernel_size, interpolation)


def mapped_max_unpool(grad_output, idx_mask, sample_map, input_height, input_width, kernel_size,
                      interpolation, plan=None):
    """include/nn/layers/mapped_max_pooling_layer.h:69-73.  `plan`: see scatter_map_plan."""
    return _max_unpool(grad_output, idx_mask, sample_map, None, input_height, input_width,
                       kernel_size, interpolation, plan)


def weighted_mapped_max_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    """include/nn/layers/weighted_mapped_max_pooling_layer.h:42-44."""
    return _max_pool(input, sample_map, interp_weights, kernel_size, interpolation)


def weighted_mapped_max_unpool(grad_output, idx_mask, sample_map, interp_weights, input_height,
                               input_width, kernel_size, interpolation, plan=None):
    """include/nn/layers/weighted_mapped_max_pooling_layer.h:67-70."""
    return _max_unpool(grad_output, idx_mask, sample_map, interp_weights, input_height,
                       input_width, kernel_size, interpolation, plan)


def mapped_avg_pool(input, sample_map, kernel_size, interpolation):
    """include/nn/layers/mapped_avg_pooling_layer.h:42-44."""
    return _avg_pool(input, sample_map, None, kernel_size, interpolation)


def mapped_avg_unpool(grad_output, sample_map, input_height, input_width, kernel_size,
                      interpolation, plan=None):
    """include/nn/layers/mapped_avg_pooling_layer.h:64-67.  `plan`: see scatter_map_plan."""
    return _avg_unpool(grad_output, sample_map, None, input_height, input_width, kernel_size,
                       interpolation, plan)


def weighted_mapped_avg_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    """include/nn/layers/weighted_mapped_avg_pooling_layer.h:48-52."""
    return _avg_pool(input, sample_map, interp_weights, kernel_size, interpolation)


def weighted_mapped_avg_unpool(grad_output, sample_map, interp_weights, input_height, input_width,
                               kernel_size, interpolation, plan=None):
    """include/nn/layers/weighted_mapped_avg_pooling_layer.h:75-78."""
    return _avg_unpool(grad_output, sample_map, interp_weights, input_height, input_width,
                       kernel_size, interpolation, plan)


# ----------------------------------------------------------------------- resample
def _resample_to_map(input, sample_map, interp_weights, output_height, output_width,
                     interpolation, plan=None):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights)
    _on_gpu("input", input, sample_map=sample_map, interp_weights=interp_weights)
    dt = _dtype(input, maps=(sample_map, interp_weights))
    P = _weighted_dims(sample_map, interp_weights, False)
    if input.dim() != 4:
        raise RuntimeError("expected a 4-D [B, C, H, W] tensor, got %d dimensions" % input.dim())
    B, C, IH, IW = input.shape
    if tuple(sample_map.shape[:2]) != (IH, IW):
        raise RuntimeError("sample_map spatial size must match the input")
    OH, OW = int(output_height), int(output_width)
    out = torch.empty((B, C, OH, OW), dtype=input.dtype, device=input.device)
    lib = _lib.load()
    plan = _scatter_plan_for("resample", plan, sample_map, interp_weights, OH, OW, interpolation,
                             False)
    if plan is not None:
        with torch.cuda.device(input.device):
            rc = lib.mcx_resample_to_map_planned(_ptr(input), *_plan_args(plan), _ptr(out),
                                                 B, C, IH, IW, OH, OW, P, int(interpolation), dt,
                                                 _stream(input))
        _lib.check(rc, "resample_to_map")
        return out
    ws_bytes = lib.mcx_resample_to_map_workspace(IH, IW, OH, OW, P, int(interpolation), dt) \
        if scatter_as_gather else 0
    ws = _workspace(ws_bytes, input.device)
    with torch.cuda.device(input.device):
        rc = lib.mcx_resample_to_map(_ptr(input), _ptr(sample_map), _ptr(interp_weights),
                                     _ptr(out), _ptr(ws), ws_bytes, B, C, IH, IW, OH, OW, P,
                                     int(interpolation), dt, _stream(input))
    _lib.check(rc, "resample_to_map")
    return out


def _resample_from_map(input, sample_map, interp_weights, interpolation):
    _contig(input=input, sample_map=sample_map, interp_weights=interp_weights)
    _on_gpu("input", input, sample_map=sample_map, interp_weights=interp_weights)
    dt = _dtype(input, maps=(sample_map, interp_weights))
    P = _weighted_dims(sample_map, interp_weights, False)
    if input.dim() != 4:
        raise RuntimeError("expected a 4-D [B, C, H, W] tensor, got %d dimensions" % input.dim())
    B, C, SH, SW = input.shape
    MH, MW = sample_map.shape[0], sample_map.shape[1]
    out = torch.empty((B, C, MH, MW), dtype=input.dtype, device=input.device)
    with torch.cuda.device(input.device):
        rc = _lib.load().mcx_resample_from_map(_ptr(input), _ptr(sample_map),
                                               _ptr(interp_weights), _ptr(out), B, C, SH, SW, MH,
                                               MW, P, int(interpolation), dt, _stream(input))
    _lib.check(rc, "resample_from_map")
    return out


def resample_to_map(input, sample_map, output_height, output_width, interpolation, plan=None):
    """include/nn/layers/resample_layer.h:38-40 (scatter).  `plan`: see scatter_map_plan."""
    return _resample_to_map(input, sample_map, None, output_height, output_width, interpolation,
                            plan)


def resample_from_map(input, sample_map, interpolation):
    """include/nn/layers/resample_layer.h:60-61 (gather)."""
    return _resample_from_map(input, sample_map, None, interpolation)


def weighted_resample_to_map(input, sample_map, interp_weights, output_height, output_width,
                             interpolation, plan=None):
    """include/nn/layers/weighted_resample_layer.h:49-54."""
    return _resample_to_map(input, sample_map, interp_weights, output_height, output_width,
                            interpolation, plan)


def weighted_resample_from_map(input, sample_map, interp_weights, interpolation):
    """include/nn/layers/weighted_resample_layer.h:78-81."""
    return _resample_from_map(input, sample_map, interp_weights, interpolation)


# ---------------------------------------------------------------------------- knn
def knn_forward(ref, query, k):
    """include/util/layers/knn_layer.h:25-35 -> [idx int64 [B,k,Q] (1-based), dist [B,k,Q]]."""
    _contig(ref=ref, query=query)
    _on_gpu("ref", ref, query=query)
    dt = _dtype(ref, same=(query,))
    if ref.dim() != 3 or query.dim() != 3 or ref.shape[:2] != query.shape[:2]:
        raise RuntimeError("ref and query must be [B, D, *] with equal B and D")
    B, D, R = ref.shape
    Q, k = query.shape[2], int(k)
    idx = torch.empty((B, k, Q), dtype=torch.int64, device=ref.device)
    dist = torch.empty((B, k, Q), dtype=ref.dtype, device=ref.device)
    lib = _lib.load()
    with torch.cuda.device(ref.device):
        # (the grid search's bins; 0 bytes where it does not apply and every point is walked)
        ws_bytes = lib.mcx_knn_workspace(B, D, R, dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=ref.device) if ws_bytes else None
        rc = lib.mcx_knn(_ptr(ref), _ptr(query), _ptr(idx), _ptr(dist),
                         _ptr(ws) if ws is not None else None, ws_bytes, B, D, R, Q, k, dt,
                         _stream(ref))
    _lib.check(rc, "knn_forward")
    return [idx, dist]


# ------------------------------------------------------- map builders, cube2rect
PROJECTIONS = {"grid": 0, "gnomonic": 1, "equirectangular": 2, "perspective": 3}


def projection_map(shape, kernel_size, proj, stride, dilation, device):
    """Sample map [ceil(H/stride), ceil(W/stride), kh*kw, 2] (float32, on `device`) of the
    reference's host-side builders, package/layers/util/spherical_projections.py:12-24,33-35;
    `proj` is a key of PROJECTIONS."""
    H, W = (int(v) for v in shape)
    kh, kw = (int(v) for v in kernel_size)
    stride, dilation = int(stride), int(dilation)
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("maps are built on the GPU: this backend has no CPU implementation")
    out = torch.empty((-(-H // stride), -(-W // stride), kh * kw, 2), dtype=torch.float32,
                      device=device)
    with torch.cuda.device(device):
        rc = _lib.load().mcx_projection_map(_ptr(out), H, W, kh, kw, PROJECTIONS[proj], stride,
                                            dilation, _stream(out))
    _lib.check(rc, "projection_map")
    return out


def cube_projection_map(cube_dim, kernel_size, stride, device):
    """spherical_projections.py:26-30 -> [ceil(dim/stride), ceil(6*dim/stride), kh*kw, 2]."""
    dim, stride = int(cube_dim), int(stride)
    kh, kw = (int(v) for v in kernel_size)
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("maps are built on the GPU: this backend has no CPU implementation")
    out = torch.empty((-(-dim // stride), -(-6 * dim // stride), kh * kw, 2),
                      dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        rc = _lib.load().mcx_cube_projection_map(_ptr(out), dim, kh, kw, stride, _stream(out))
    _lib.check(rc, "cube_projection_map")
    return out


def cube2rect(cubemap, rect_height, rect_width, interpolation):
    """include/util/layers/cube2rect_layer.h:29-43: cubemap [C, dim, 6*dim] with faces
    [-z, -x, +z, +x, +y, -y] -> equirectangular [C, rect_height, rect_width]."""
    _contig(cubemap=cubemap)
    _on_gpu("cubemap", cubemap)
    if cubemap.dtype not in (torch.float32, torch.float64):
        raise RuntimeError("unsupported dtype %s" % cubemap.dtype)
    if cubemap.dim() != 3 or cubemap.shape[2] != 6 * cubemap.shape[1]:
        raise RuntimeError("cubemap must be [C, dim, 6*dim], got %s" % (tuple(cubemap.shape),))
    C, dim = cubemap.shape[0], cubemap.shape[1]
    RH, RW = int(rect_height), int(rect_width)
    rect = torch.empty((C, RH, RW), dtype=cubemap.dtype, device=cubemap.device)
    with torch.cuda.device(cubemap.device):
        rc = _lib.load().mcx_cube2rect(_ptr(cubemap), _ptr(rect), C, dim, RH, RW,
                                       int(interpolation), _DTYPES[cubemap.dtype],
                                       _stream(cubemap))
    _lib.check(rc, "cube2rect")
    return rect


# ------------------------------------------------------------ icosphere map operators
def gnomonic_samples(centres, kh, kw, res_lat, res_lon):
    """gnomonic_kernel of package/layers/util/icosphere_functions.py:135-183 on the device:
    centres [V, 2] (longitude, latitude), float32 -> [1, V, kh*kw, 2]."""
    _contig(centres=centres)
    _on_gpu("spherical_coords", centres)
    if centres.dtype != torch.float32 or centres.dim() != 2 or centres.shape[1] != 2:
        raise RuntimeError("spherical_coords must be a float32 tensor [V, 2]")
    V = centres.shape[0]
    out = torch.empty((1, V, int(kh) * int(kw), 2), dtype=torch.float32, device=centres.device)
    with torch.cuda.device(centres.device):
        rc = _lib.load().mcx_gnomonic_samples(_ptr(centres), _ptr(out), V, int(kh), int(kw),
                                              float(res_lat), float(res_lon), _stream(centres))
    _lib.check(rc, "gnomonic_kernel")
    return out


def planar_conv_operator_from_samples(samples, vertices, faces, keepdim=True, nearest=False):
    """Sphere.get_planar_conv_operator_from_samples of the reference's `_sphere` module
    (package/ext_modules/src/util/cpp/sphere.cpp:1117-1270) over a caller-supplied mesh.

    samples [OH, OW, K, 2] or [OH, OW, 2] (longitude, latitude), float32, on the GPU;
    vertices [V, 3] float32 and faces [F, 3] int64 of a closed triangle mesh around the
    origin.  Returns [face_idx [OH, OW, K] int64, vertex_idx [OH, OW, K, 3] int64,
    weights [OH, OW, K, 3] float32]; a [OH, OW, 2] input without `keepdim` drops the K axis,
    as in the reference."""
    _contig(samples=samples, vertices=vertices, faces=faces)
    _on_gpu("samples", samples, vertices=vertices, faces=faces)
    if samples.dtype != torch.float32 or vertices.dtype != torch.float32:
        raise RuntimeError("samples and vertices must be float32")
    if faces.dtype != torch.int64:
        raise RuntimeError("faces must be int64")
    if samples.dim() not in (3, 4) or samples.shape[-1] != 2:
        raise RuntimeError("samples must be [OH, OW, K, 2] or [OH, OW, 2]")
    if vertices.dim() != 2 or vertices.shape[1] != 3 or faces.dim() != 2 or faces.shape[1] != 3:
        raise RuntimeError("vertices must be [V, 3] and faces [F, 3]")
    lead = tuple(samples.shape[:-1])
    if samples.dim() == 3 and keepdim:
        lead = lead + (1,)
    N, V, F = samples.numel() // 2, vertices.shape[0], faces.shape[0]
    dev = samples.device
    face_idx = torch.empty(lead, dtype=torch.int64, device=dev)
    vertex_idx = torch.empty(lead + (3,), dtype=torch.int64, device=dev)
    weights = torch.empty(lead + (3,), dtype=torch.float32, device=dev)
    lib = _lib.load()
    ws_bytes = lib.mcx_planar_conv_operator_workspace(F)
    ws = _workspace(ws_bytes, dev)
    with torch.cuda.device(dev):
        rc = lib.mcx_planar_conv_operator(_ptr(samples), _ptr(vertices), _ptr(faces),
                                          _ptr(face_idx), _ptr(vertex_idx), _ptr(weights),
                                          _ptr(ws), ws_bytes, N, V, F, 1 if nearest else 0,
                                          _stream(samples))
    _lib.check(rc, "planar_conv_operator_from_samples")
    return [face_idx, vertex_idx, weights]
