"""MI355X-native backend for mapped convolutions.

`mappedconvolutions_amd.nn` mirrors the reference's `mapped_convolution.nn`
layer API; `mappedconvolutions_amd._C` mirrors its extension ops; both run on
hand-written gfx950 HIP kernels in libmcx_hip.so (C ABI: include/mcx.h).

`install_aliases()` registers the reference's import names
(`mapped_convolution`, `mapped_convolution.nn`, `mapped_convolution.util`,
`_mapped_convolution_ext._<op family>`) so code written against the reference
imports unchanged.
"""
import sys
import types

from . import _C, nn, util  # noqa: F401

__version__ = "0.1.0"

# pybind module of the reference (package/setup.py:52-84) -> op names it exports
_EXT_MODULES = {
    "_mapped_convolution": ["mapped_conv_forward", "mapped_conv_backward"],
    "_weighted_mapped_convolution": ["weighted_mapped_conv_forward",
                                     "weighted_mapped_conv_backward"],
    "_mapped_transposed_convolution": ["mapped_transposed_conv_forward",
                                       "mapped_transposed_conv_backward"],
    "_weighted_mapped_transposed_convolution": ["weighted_mapped_transposed_conv_forward",
                                                "weighted_mapped_transposed_conv_backward"],
    "_mapped_max_pooling": ["mapped_max_pool", "mapped_max_unpool"],
    "_weighted_mapped_max_pooling": ["weighted_mapped_max_pool", "weighted_mapped_max_unpool"],
    "_mapped_avg_pooling": ["mapped_avg_pool", "mapped_avg_unpool"],
    "_weighted_mapped_avg_pooling": ["weighted_mapped_avg_pool", "weighted_mapped_avg_unpool"],
    "_resample": ["resample_to_map", "resample_from_map"],
    "_weighted_resample": ["weighted_resample_to_map", "weighted_resample_from_map"],
    "_knn": ["knn_forward"],
    "_cube2rect": ["cube2rect"],
}


# Modules of the reference's extension package that lie outside this backend's path.  The
# plain convolution pair is the reference's timing baseline, a re-implementation of the library
# convolution (package/ext_modules/include/nn/layers/convolution_layer.h:64-143,
# transposed_convolution_layer.h): registered as thin calls of that library routine so that
# the reference's `nn/__init__` imports and its baseline layers run.  `_sphere` is a host-side
# half-edge mesh class (include/util/cpp/sphere.h:131-175): its name resolves, its use raises.
def _plain_conv_module():
    import torch
    import torch.nn.functional as F
    m = types.ModuleType("_mapped_convolution_ext._convolution")

    def conv_forward(input, weight, bias, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,
                     dilation_h, dilation_w):
        return F.conv2d(input, weight, bias, (stride_h, stride_w), (pad_h, pad_w),
                        (dilation_h, dilation_w))

    def conv_backward(grad_output, input, weight, bias, kernel_h, kernel_w, stride_h, stride_w,
                      pad_h, pad_w, dilation_h, dilation_w):
        gi, gw, gb = torch.ops.aten.convolution_backward(
            grad_output, input, weight, [bias.numel()], [stride_h, stride_w], [pad_h, pad_w],
            [dilation_h, dilation_w], False, [0, 0], 1, [True, True, True])
        return [gi, gw, gb]

    m.conv_forward, m.conv_backward = conv_forward, conv_backward
    return m


def _plain_transposed_conv_module():
    import torch
    import torch.nn.functional as F
    m = types.ModuleType("_mapped_convolution_ext._transposed_convolution")

    def transposed_conv_forward(input, weight, bias, kernel_h, kernel_w, stride_h, stride_w,
                                pad_h, pad_w, dilation_h, dilation_w):
        return F.conv_transpose2d(input, weight, bias, (stride_h, stride_w), (pad_h, pad_w), 0,
                                  1, (dilation_h, dilation_w))

    def transposed_conv_backward(grad_output, input, weight, bias, kernel_h, kernel_w, stride_h,
                                 stride_w, pad_h, pad_w, dilation_h, dilation_w):
        gi, gw, gb = torch.ops.aten.convolution_backward(
            grad_output, input, weight, [bias.numel()], [stride_h, stride_w], [pad_h, pad_w],
            [dilation_h, dilation_w], True, [0, 0], 1, [True, True, True])
        return [gi, gw, gb]

    m.transposed_conv_forward = transposed_conv_forward
    m.transposed_conv_backward = transposed_conv_backward
    return m


class _HostOnlyModule(types.ModuleType):
    def __getattr__(self, name):
        if name.startswith("__"):
            raise AttributeError(name)
        raise RuntimeError(
            "%s.%s: the reference's host-side mesh tools are not part of this GPU backend; "
            "pass mesh tensors to mappedconvolutions_amd.util.vertex_to_vertex_kernel_map / "
            "_C.planar_conv_operator_from_samples instead" % (self.__name__, name))


def install_aliases(ext_only=False):
    """Make `import mapped_convolution.nn` and
    `import _mapped_convolution_ext._mapped_convolution` resolve to this package.
    With `ext_only` only the extension-module names are registered, for use under
    the reference's own pure-Python layer files."""
    if not ext_only:
        pkg = types.ModuleType("mapped_convolution")
        pkg.nn, pkg.util = nn, util
        pkg.__path__ = []
        sys.modules.setdefault("mapped_convolution", pkg)
        sys.modules.setdefault("mapped_convolution.nn", nn)
        sys.modules.setdefault("mapped_convolution.util", util)
        sys.modules.setdefault("mapped_convolutions", sys.modules["mapped_convolution"])
        sys.modules.setdefault("mapped_convolutions.nn", nn)
    ext = types.ModuleType("_mapped_convolution_ext")
    ext.__path__ = []
    sys.modules.setdefault("_mapped_convolution_ext", ext)
    for mod_name, ops in _EXT_MODULES.items():
        m = types.ModuleType("_mapped_convolution_ext." + mod_name)
        for op in ops:
            setattr(m, op, getattr(_C, op))
        sys.modules.setdefault(m.__name__, m)
        setattr(sys.modules["_mapped_convolution_ext"], mod_name, m)
    for m in (_plain_conv_module(), _plain_transposed_conv_module(),
              _HostOnlyModule("_mapped_convolution_ext._sphere")):
        sys.modules.setdefault(m.__name__, m)
        setattr(sys.modules["_mapped_convolution_ext"], m.__name__.rsplit(".", 1)[1], m)
