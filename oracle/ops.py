"""TEST INFRASTRUCTURE: the C oracle (oracle/mcx_oracle.c) behind the op names of
the shipped `_C` boundary, operating on CPU float32 / float64 tensors."""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmcx_oracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "libmcx_oracle.so"])


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
    return _lib


def _sfx(t):
    if t.dtype == torch.float32:
        return "_f32"
    if t.dtype == torch.float64:
        return "_f64"
    raise TypeError("oracle supports float32 / float64 only, got %s" % t.dtype)


def _p(t):
    return ctypes.c_void_p(None if t is None else t.data_ptr())


def _i(v):
    return ctypes.c_int64(int(v))


def _call(name, like, *args):
    fn = getattr(load(), name + _sfx(like))
    fn.restype = None
    fn(*args)


def _prep(*ts):
    out = []
    for t in ts:
        if t is not None:
            assert not t.is_cuda, "oracle runs on CPU tensors"
            t = t.contiguous()
        out.append(t)
    return out


def _P(iw):
    return 0 if iw is None else iw.shape[-1]


# ----------------------------------------------------------------------- resample
def weighted_resample_from_map(input, sample_map, interp_weights, interpolation):
    input, sample_map, interp_weights = _prep(input, sample_map, interp_weights)
    B, C, SH, SW = input.shape
    MH, MW = sample_map.shape[:2]
    out = torch.empty(B, C, MH, MW, dtype=input.dtype)
    _call("orc_resample_from_map", input, _p(input), _p(sample_map), _p(interp_weights), _p(out),
          _i(B), _i(C), _i(SH), _i(SW), _i(MH), _i(MW), _i(_P(interp_weights)),
          ctypes.c_int(interpolation))
    return out


def resample_from_map(input, sample_map, interpolation):
    return weighted_resample_from_map(input, sample_map, None, interpolation)


def weighted_resample_to_map(input, sample_map, interp_weights, output_height, output_width,
                             interpolation):
    input, sample_map, interp_weights = _prep(input, sample_map, interp_weights)
    B, C, IH, IW = input.shape
    out = torch.empty(B, C, output_height, output_width, dtype=input.dtype)
    _call("orc_resample_to_map", input, _p(input), _p(sample_map), _p(interp_weights), _p(out),
          _i(B), _i(C), _i(IH), _i(IW), _i(output_height), _i(output_width),
          _i(_P(interp_weights)), ctypes.c_int(interpolation))
    return out


def resample_to_map(input, sample_map, output_height, output_width, interpolation):
    return weighted_resample_to_map(input, sample_map, None, output_height, output_width,
                                    interpolation)


# ------------------------------------------------------------------------ pooling
def weighted_mapped_max_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    input, sample_map, interp_weights = _prep(input, sample_map, interp_weights)
    B, C, IH, IW = input.shape
    OH, OW = sample_map.shape[:2]
    out = torch.empty(B, C, OH, OW, dtype=input.dtype)
    idx = torch.empty(B, C, OH, OW, dtype=torch.int64)
    _call("orc_max_pool", input, _p(input), _p(sample_map), _p(interp_weights), _p(out), _p(idx),
          _i(B), _i(C), _i(IH), _i(IW), _i(OH), _i(OW), _i(kernel_size), _i(_P(interp_weights)),
          ctypes.c_int(interpolation))
    return [out, idx]


def mapped_max_pool(input, sample_map, kernel_size, interpolation):
    return weighted_mapped_max_pool(input, sample_map, None, kernel_size, interpolation)


def weighted_mapped_max_unpool(grad_output, idx_mask, sample_map, interp_weights, input_height,
                               input_width, kernel_size, interpolation):
    grad_output, idx_mask, sample_map, interp_weights = _prep(grad_output, idx_mask, sample_map,
                                                              interp_weights)
    B, C, OH, OW = grad_output.shape
    gin = torch.empty(B, C, input_height, input_width, dtype=grad_output.dtype)
    _call("orc_max_unpool", grad_output, _p(grad_output), _p(idx_mask), _p(sample_map),
          _p(interp_weights), _p(gin), _i(B), _i(C), _i(input_height), _i(input_width), _i(OH),
          _i(OW), _i(kernel_size), _i(_P(interp_weights)), ctypes.c_int(interpolation))
    return gin


def mapped_max_unpool(grad_output, idx_mask, sample_map, input_height, input_width, kernel_size,
                      interpolation):
    return weighted_mapped_max_unpool(grad_output, idx_mask, sample_map, None, input_height,
                                      input_width, kernel_size, interpolation)


def weighted_mapped_avg_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    input, sample_map, interp_weights = _prep(input, sample_map, interp_weights)
    B, C, IH, IW = input.shape
    OH, OW = sample_map.shape[:2]
    out = torch.empty(B, C, OH, OW, dtype=input.dtype)
    _call("orc_avg_pool", input, _p(input), _p(sample_map), _p(interp_weights), _p(out), _i(B),
          _i(C), _i(IH), _i(IW), _i(OH), _i(OW), _i(kernel_size), _i(_P(interp_weights)),
          ctypes.c_int(interpolation))
    return out


def mapped_avg_pool(input, sample_map, kernel_size, interpolation):
    return weighted_mapped_avg_pool(input, sample_map, None, kernel_size, interpolation)


def weighted_mapped_avg_unpool(grad_output, sample_map, interp_weights, input_height, input_width,
                               kernel_size, interpolation):
    grad_output, sample_map, interp_weights = _prep(grad_output, sample_map, interp_weights)
    B, C, OH, OW = grad_output.shape
    gin = torch.empty(B, C, input_height, input_width, dtype=grad_output.dtype)
    _call("orc_avg_unpool", grad_output, _p(grad_output), _p(sample_map), _p(interp_weights),
          _p(gin), _i(B), _i(C), _i(input_height), _i(input_width), _i(OH), _i(OW),
          _i(kernel_size), _i(_P(interp_weights)), ctypes.c_int(interpolation))
    return gin


def mapped_avg_unpool(grad_output, sample_map, input_height, input_width, kernel_size,
                      interpolation):
    return weighted_mapped_avg_unpool(grad_output, sample_map, None, input_height, input_width,
                                      kernel_size, interpolation)


# --------------------------------------------------------------------------- conv
def weighted_mapped_conv_forward(input, sample_map, interp_weights, weight, bias, kernel_size,
                                 interpolation):
    input, sample_map, interp_weights, weight, bias = _prep(input, sample_map, interp_weights,
                                                            weight, bias)
    B, Ci, IH, IW = input.shape
    Co = weight.shape[0]
    OH, OW = sample_map.shape[:2]
    out = torch.empty(B, Co, OH, OW, dtype=input.dtype)
    _call("orc_conv_forward", input, _p(input), _p(sample_map), _p(interp_weights), _p(weight),
          _p(bias), _p(out), _i(B), _i(Ci), _i(Co), _i(IH), _i(IW), _i(OH), _i(OW),
          _i(kernel_size), _i(_P(interp_weights)), ctypes.c_int(interpolation))
    return out


def mapped_conv_forward(input, sample_map, weight, bias, kernel_size, interpolation):
    return weighted_mapped_conv_forward(input, sample_map, None, weight, bias, kernel_size,
                                        interpolation)


def weighted_mapped_conv_backward(grad_output, sample_map, interp_weights, input, weight, bias,
                                  kernel_size, interpolation):
    grad_output, sample_map, interp_weights, input, weight = _prep(grad_output, sample_map,
                                                                   interp_weights, input, weight)
    B, Ci, IH, IW = input.shape
    Co, OH, OW = grad_output.shape[1:]
    P = _P(interp_weights)
    gx = torch.empty_like(input)
    gw = torch.empty_like(weight)
    gb = torch.empty(Co, dtype=input.dtype)
    dims = (_i(B), _i(Ci), _i(Co), _i(IH), _i(IW), _i(OH), _i(OW), _i(kernel_size), _i(P),
            ctypes.c_int(interpolation))
    _call("orc_conv_backward_input", input, _p(grad_output), _p(sample_map), _p(interp_weights),
          _p(weight), _p(gx), *dims)
    _call("orc_conv_backward_weight", input, _p(grad_output), _p(sample_map), _p(interp_weights),
          _p(input), _p(gw), _p(gb), *dims)
    return [gx, gw, gb]


def mapped_conv_backward(grad_output, sample_map, input, weight, bias, kernel_size, interpolation):
    return weighted_mapped_conv_backward(grad_output, sample_map, None, input, weight, bias,
                                         kernel_size, interpolation)


def weighted_mapped_transposed_conv_forward(input, sample_map, interp_weights, weight, bias,
                                            output_height, output_width, kernel_size,
                                            interpolation):
    input, sample_map, interp_weights, weight, bias = _prep(input, sample_map, interp_weights,
                                                            weight, bias)
    B, Ci, IH, IW = input.shape
    Co = weight.shape[1]
    out = torch.empty(B, Co, output_height, output_width, dtype=input.dtype)
    _call("orc_tconv_forward", input, _p(input), _p(sample_map), _p(interp_weights), _p(weight),
          _p(bias), _p(out), _i(B), _i(Ci), _i(Co), _i(IH), _i(IW), _i(output_height),
          _i(output_width), _i(kernel_size), _i(_P(interp_weights)), ctypes.c_int(interpolation))
    return out


def mapped_transposed_conv_forward(input, sample_map, weight, bias, output_height, output_width,
                                   kernel_size, interpolation):
    return weighted_mapped_transposed_conv_forward(input, sample_map, None, weight, bias,
                                                   output_height, output_width, kernel_size,
                                                   interpolation)


def weighted_mapped_transposed_conv_backward(grad_output, sample_map, interp_weights, input,
                                             weight, bias, kernel_size, interpolation):
    grad_output, sample_map, interp_weights, input, weight = _prep(grad_output, sample_map,
                                                                   interp_weights, input, weight)
    B, Ci, IH, IW = input.shape
    Co, OH, OW = grad_output.shape[1:]
    P = _P(interp_weights)
    gx = torch.empty_like(input)
    gw = torch.empty_like(weight)
    gb = torch.empty(Co, dtype=input.dtype)
    dims = (_i(B), _i(Ci), _i(Co), _i(IH), _i(IW), _i(OH), _i(OW), _i(kernel_size), _i(P),
            ctypes.c_int(interpolation))
    _call("orc_tconv_backward_input", input, _p(grad_output), _p(sample_map), _p(interp_weights),
          _p(weight), _p(gx), *dims)
    _call("orc_tconv_backward_weight", input, _p(grad_output), _p(sample_map), _p(interp_weights),
          _p(input), _p(gw), _p(gb), *dims)
    return [gx, gw, gb]


def mapped_transposed_conv_backward(grad_output, sample_map, input, weight, bias, kernel_size,
                                    interpolation):
    return weighted_mapped_transposed_conv_backward(grad_output, sample_map, None, input, weight,
                                                    bias, kernel_size, interpolation)


def im2col(image, sample_map, interp_weights, kernel_size, interpolation):
    """Column buffer [C*K, OH*OW] of ONE image [C, H, W]."""
    image, sample_map, interp_weights = _prep(image, sample_map, interp_weights)
    C, H, W = image.shape
    N = sample_map.shape[0] * sample_map.shape[1]
    col = torch.empty(C * kernel_size, N, dtype=image.dtype)
    _call("orc_im2col", image, _p(image), _p(sample_map), _p(interp_weights), _p(col), _i(C),
          _i(H), _i(W), _i(N), _i(kernel_size), _i(_P(interp_weights)),
          ctypes.c_int(interpolation))
    return col


def col2im(col, sample_map, interp_weights, channels, height, width, kernel_size, interpolation):
    col, sample_map, interp_weights = _prep(col, sample_map, interp_weights)
    N = sample_map.shape[0] * sample_map.shape[1]
    im = torch.empty(channels, height, width, dtype=col.dtype)
    _call("orc_col2im", col, _p(col), _p(sample_map), _p(interp_weights), _p(im), _i(channels),
          _i(height), _i(width), _i(N), _i(kernel_size), _i(_P(interp_weights)),
          ctypes.c_int(interpolation))
    return im


# ---------------------------------------------------------------------------- knn
def knn_forward(ref, query, k):
    ref, query = _prep(ref, query)
    B, D, R = ref.shape
    Q = query.shape[2]
    idx = torch.empty(B, k, Q, dtype=torch.int64)
    dist = torch.empty(B, k, Q, dtype=ref.dtype)
    _call("orc_knn", ref, _p(ref), _p(query), _p(idx), _p(dist), _i(B), _i(D), _i(R), _i(Q),
          _i(k))
    return [idx, dist]
