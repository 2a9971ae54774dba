"""CPU-side checks of the native build: the C-ABI library loads and exports every symbol
include/geo_sc.h declares, the PyTorch modules export the reference's op names, host-side
argument validation answers without a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    with open(os.path.join(ROOT, "include", "geo_sc.h")) as f:
        text = f.read()
    return sorted(set(re.findall(r"GEO_SC_API\s+[\w\s\*]+?\b(geo_sc_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from geo_amd import _native
    names = declared_symbols()
    assert len(names) >= 9
    lib = ctypes.CDLL(_native.lib_path())
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_native.C_API) == names   # the ctypes table and the header agree
    assert _native.lib().geo_sc_version() == 1


def test_host_side_validation_without_gpu():
    from geo_amd import capi
    d = capi.make_desc((2, 3, 8, 8), (4, 3, 3, 3), 64, (1, 1))
    assert capi.output_shape(d) == (2, 4, 8, 8)
    assert capi.workspace_size(d) > 0
    # padding convention: first entry pads the last dim
    d = capi.make_desc((1, 1, 4, 6), (1, 1, 3, 3), 32, (2, 0))
    assert (d.pad_h, d.pad_w) == (2, 0) and capi.output_shape(d) == (1, 1, 2, 8)
    for sx, sw, L, status in (((2, 3, 8, 8), (4, 3, 3, 3), 100, 2), ((2, 3, 2, 2), (4, 3, 3, 3), 64, 1)):
        with pytest.raises(capi.GeoScError) as e:
            capi.workspace_size(capi.make_desc(sx, sw, L))
        assert e.value.status == status
    with pytest.raises(capi.GeoScError):
        capi.workspace_size(capi.make_desc((2, 3, 8, 8), (4, 3, 3, 3), 64, load_width=0))
    # stream layout query: single-row outputs of 1/3/5-wide kernels with several items are item-innermost
    import ctypes as ct
    from geo_amd import _native
    inner = ct.c_int(-1)
    for sx, sw, want in (((5, 4, 3, 6), (2, 4, 3, 3), 1), ((5, 4, 8, 6), (2, 4, 3, 3), 0), ((1, 4, 3, 6), (2, 4, 3, 3), 0)):
        assert _native.lib().geo_sc_act_stream_layout(ct.byref(capi.make_desc(sx, sw, 64)), ct.byref(inner)) == 0
        assert inner.value == want, (sx, sw)
    # workspace of the headline shape: tables + weight streams + activation streams
    d = capi.make_desc((256, 128, 16, 16), (128, 128, 3, 3), 128, (1, 1))
    assert capi.workspace_size(d) >= 4 * (256 * 4 * 128 * 18 * 18 + 2 * 4 * 3 * 384 * 128)


def test_torch_modules_export_reference_names():
    from geo_amd import _native
    cuda = _native.module("sc_extension_cuda")
    for n in ("conv2d_add_partial_variable_acc", "conv2d_add_yz_variable_acc", "conv2d_add_partial_acc_acc",
              "conv2d_or_acc"):
        assert callable(getattr(cuda, n))
    assert callable(_native.module("sc_extension").conv2d_add_partial_new)
    import sys
    _native.register_reference_module_names()
    import sc_extension
    import sc_extension_cuda
    assert sc_extension_cuda is cuda and sc_extension is sys.modules["sc_extension"]


def test_host_entry_point_raises_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from geo_amd import _native
    x = torch.zeros(1, 1, 4, 4)
    w = torch.zeros(1, 1, 3, 3)
    with pytest.raises(RuntimeError, match="needs a GPU"):
        _native.module("sc_extension").conv2d_add_partial_new(x, w, 64, (0, 0), (1, 1))
    with pytest.raises(RuntimeError):
        _native.module("sc_extension_cuda").conv2d_add_partial_variable_acc(x, w, 64, (0, 0), (1, 1), 7, 8, 1,
                                                                            False, 2)
