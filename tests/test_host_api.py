"""CPU tests of the host side: the C-ABI library loads and exports every symbol
include/mcx.h declares, the layer API mirrors the reference's, argument checks
raise the reference's error types, and nothing silently falls back to a CPU path."""
import ctypes
import os
import re

import pytest
import torch

import mappedconvolutions_amd as mca
from mappedconvolutions_amd import _C, _lib, nn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mcx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mcx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "libmcx_hip.so has not been built"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), "missing symbol " + n
    assert set(names) == set(_lib.SIGNATURES), "ctypes table and header disagree"
    assert _lib.load().mcx_abi_version() >= 1
    assert b"dtype" in _lib.load().mcx_error_string(-1)


def test_rejected_arguments_return_codes_without_a_gpu():
    lib = _lib.load()
    # NULL pointers / bad sizes are rejected before any launch
    assert lib.mcx_conv_forward(None, None, None, None, None, None, None, 0, 1, 1, 1, 4, 4, 4, 4,
                                1, 0, 1, 0, None) == -3
    # a matrix-core path without its scratch buffer is refused, not run
    assert lib.mcx_conv_forward(1, 1, None, 1, 1, 1, None, 0, 1, 1, 1, 4, 4, 4, 4, 1, 0, 1, 0,
                                None) == -4
    assert lib.mcx_conv_forward_workspace(1, 64, 64, 8, 8, 8, 8, 9, 0, 0) > 0
    assert lib.mcx_conv_forward_workspace(1, 64, 64, 8, 8, 8, 8, 9, 0, 1) == 0  # fp64: scalar kernels
    assert lib.mcx_resample_from_map(1, 1, None, 1, 0, 1, 4, 4, 4, 4, 0, 1, 0, None) == -2
    assert lib.mcx_resample_from_map(1, 1, None, 1, 1, 1, 4, 4, 4, 4, 0, 1, 7, None) == -1
    assert lib.mcx_knn(1, 1, 1, 1, None, 0, 1, 3, 10, 10, 65, 0, None) == -2
    # map builders: NULL output, a spherical grid of one row (divides by H - 1), unknown projection
    assert lib.mcx_projection_map(None, 8, 16, 3, 3, 1, 1, 1, None) == -3
    assert lib.mcx_projection_map(1, 1, 16, 3, 3, 1, 1, 1, None) == -2
    assert lib.mcx_projection_map(1, 8, 16, 3, 3, 9, 1, 1, None) == -2
    assert lib.mcx_cube2rect(1, 1, 3, 8, 16, 32, 1, 2, None) == -1  # no bf16 cube2rect
    # map plans: sized for the matrix-core paths only; too small a buffer is refused
    need = lib.mcx_conv_plan_bytes(8, 8, 8, 8, 9, 0, 0)
    assert need > 0 and lib.mcx_conv_plan_bytes(8, 8, 8, 8, 9, 0, 1) == 0
    desc = _lib.PlanDesc()
    assert lib.mcx_conv_plan_build(1, None, 1, need - 1, desc, 8, 8, 8, 8, 9, 0, 1, 0, None) == -4
    assert lib.mcx_conv_plan_build(1, None, None, need, desc, 8, 8, 8, 8, 9, 0, 1, 0, None) == -3
    assert lib.mcx_conv_plan_build(1, None, 1, need, None, 8, 8, 8, 8, 9, 0, 1, 0, None) == -3
    assert lib.mcx_conv_plan_build(1, None, 1, need, desc, 8, 8, 8, 8, 9, 0, 1, 1, None) == -1
    assert lib.mcx_conv_backward_planned(1, 1, None, 1, 1, 1, 1, 1, 1, 1 << 30, 1, need - 1, desc,
                                         1, 4, 4, 8, 8, 8, 8, 9, 0, 1, 0, None) == -4
    # a plan without a descriptor, or with one that no build call filled in, is refused
    assert lib.mcx_conv_backward_planned(1, 1, None, 1, 1, 1, 1, 1, 1, 1 << 30, 1, need, None,
                                         1, 4, 4, 8, 8, 8, 8, 9, 0, 1, 0, None) == -3
    assert lib.mcx_conv_backward_planned(1, 1, None, 1, 1, 1, 1, 1, 1, 1 << 30, 1, need, desc,
                                         1, 4, 4, 8, 8, 8, 8, 9, 0, 1, 0, None) == -6
    assert lib.mcx_avg_unpool_planned(1, 1, 1 << 20, desc, 1, 1, 1, 8, 8, 8, 8, 9, 0, 1, 0,
                                      None) == -6
    assert b"plan" in lib.mcx_error_string(-6)


def test_layer_api_and_parameter_shapes():
    conv = nn.MappedConvolution(4, 6, kernel_size=9)
    assert tuple(conv.weight.shape) == (6, 4, 9) and tuple(conv.bias.shape) == (6,)
    assert conv.interp == 1
    bound = 1.0 / (4 * 9) ** 0.5
    assert conv.weight.abs().max() <= bound and conv.bias.abs().max() <= bound
    nb = nn.MappedConvolution(4, 6, 9, interpolation='nearest', bias=False)
    assert nb.interp == 0 and isinstance(nb.bias, torch.nn.Parameter) and nb.bias.abs().sum() == 0
    t = nn.MappedTransposedConvolution(4, 6, 9, interpolation='bispherical')
    assert tuple(t.weight.shape) == (4, 6, 9) and t.interp == 2
    assert nn.MappedMaxPool(4, return_indices=True).return_indices
    assert set(conv.state_dict()) == {"weight", "bias"}
    with pytest.raises(AssertionError):
        nn.MappedConvolution(1, 1, 1, interpolation='cubic')
    for name in ('MappedConvolution', 'MappedTransposedConvolution', 'MappedMaxPool',
                 'MappedAvgPool', 'MappedAvgUnpool', 'Resample', 'Unresample'):
        assert hasattr(nn, name)


def test_argument_checks_raise_like_the_reference():
    conv = nn.MappedConvolution(2, 3, kernel_size=4)
    x = torch.zeros(1, 2, 4, 5)
    good = torch.zeros(4, 5, 4, 2)
    with pytest.raises(AssertionError):   # wrong number of input dims
        conv(x[0], good)
    with pytest.raises(AssertionError):   # dtype mismatch between input and map
        conv(x, good.double())
    with pytest.raises(AssertionError):   # channel mismatch
        conv(torch.zeros(1, 3, 4, 5), good)
    with pytest.raises(AssertionError):   # kernel size mismatch
        conv(x, torch.zeros(4, 5, 3, 2))
    with pytest.raises(AssertionError):   # last map dim must be 2
        conv(x, torch.zeros(4, 5, 4, 3))
    with pytest.raises(AssertionError):   # weighted map needs 5 dims
        conv(x, good, torch.zeros(4, 5, 4, 3))
    with pytest.raises(AssertionError):   # Resample: input and map must share H x W
        nn.Resample()(x, torch.zeros(3, 5, 2), (4, 4))


def test_no_cpu_fallback():
    """CPU tensors are refused: the ops exist only as HIP kernels."""
    conv = nn.MappedConvolution(2, 3, kernel_size=4)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        conv(torch.zeros(1, 2, 4, 5), torch.zeros(4, 5, 4, 2))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        _C.resample_from_map(torch.zeros(1, 1, 2, 2), torch.zeros(2, 2, 2), 1)
    with pytest.raises(RuntimeError, match="contiguous"):
        _C.resample_from_map(torch.zeros(1, 1, 2, 4)[..., ::2], torch.zeros(2, 2, 2), 1)


def test_shipped_package_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "mappedconvolutions_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, "%s mentions the oracle" % f


def test_reference_import_names_resolve():
    mca.install_aliases()
    import mapped_convolution.nn as rnn
    import _mapped_convolution_ext._mapped_convolution as ext
    import _mapped_convolution_ext._knn as knn_ext
    assert rnn.MappedConvolution is nn.MappedConvolution
    assert ext.mapped_conv_forward is _C.mapped_conv_forward
    assert knn_ext.knn_forward is _C.knn_forward
