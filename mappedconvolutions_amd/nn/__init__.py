"""Mapped layers with the reference's `mapped_convolution.nn` names
(layers/nn/__init__.py:6-10).  The plain `Convolution` / `TransposedConvolution` that the
reference also exports re-implement torch.nn.Conv2d and are no part of the mapped hot path:
the layer classes are not defined here; `mappedconvolutions_amd.install_aliases()` registers
the extension modules behind them (`_convolution`, `_transposed_convolution`) as calls of the
library convolution, so that the reference's own layer files import."""
from .mapped_convolution_layer import MappedConvolution
from .mapped_transposed_convolution_layer import MappedTransposedConvolution
from .mapped_max_pooling_layer import MappedMaxPool
from .mapped_avg_pooling_layer import MappedAvgPool, MappedAvgUnpool
from .resample_layer import Resample, Unresample

__all__ = ['MappedConvolution', 'MappedTransposedConvolution', 'MappedMaxPool', 'MappedAvgPool',
           'MappedAvgUnpool', 'Resample', 'Unresample']
