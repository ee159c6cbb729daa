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
