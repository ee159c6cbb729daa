"""Mapped layers with the reference's `mapped_convolution.nn` names
(layers/nn/__init__.py:6-10).  The plain `Convolution` / `TransposedConvolution`
re-implementations of torch.nn.Conv2d that the reference also exports are not
part of the mapped hot path and are not provided."""
from .mapped_convolution_layer import MappedConvolution
from .mapped_transposed_convolution_layer import MappedTransposedConvolution
from .mapped_max_pooling_layer import MappedMaxPool
from .mapped_avg_pooling_layer import MappedAvgPool, MappedAvgUnpool
from .resample_layer import Resample, Unresample

__all__ = ['MappedConvolution', 'MappedTransposedConvolution', 'MappedMaxPool', 'MappedAvgPool',
           'MappedAvgUnpool', 'Resample', 'Unresample']
