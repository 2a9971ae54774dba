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
    assert _native.lib().geo_sc_version() == 2


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
    # workspace of the headline shape: weight streams + activation streams (170 MB: inside the default budget)
    d = capi.make_desc((256, 128, 16, 16), (128, 128, 3, 3), 128, (1, 1))
    assert capi.workspace_size(d) >= 4 * (256 * 4 * 128 * 18 * 18 + 2 * 4 * 3 * 384 * 128)
    assert capi.forward_chunk(d) == 256


def test_forward_scratch_is_bounded_by_the_stream_budget():
    """A batch whose activation streams exceed geo_sc_options.forward_stream_bytes runs in chunks: the workspace
    stops growing with the batch (the reference keeps streams for 128 blocks whatever the batch,
    sc_cuda_kernel.cu:1787-1789)."""
    from geo_amd import capi
    # the ResNet-style layer: 0.88 GB of streams for the batch of 128
    sx, sw = (128, 64, 56, 56), (64, 64, 3, 3)
    d = capi.make_desc(sx, sw, 256, (1, 1))
    item = 4 * 8 * 64 * 58 * 58
    nc = capi.forward_chunk(d)
    assert 1 <= nc < 128 and 2 * nc * item <= 256 << 20
    assert capi.workspace_size(d) <= 300 << 20
    big = capi.make_desc((4096,) + sx[1:], sw, 256, (1, 1))
    assert capi.workspace_size(big) <= 300 << 20 and capi.forward_chunk(big) * item <= 256 << 20
    # the caller's budget: one item is always held, whatever the budget
    tiny = capi.make_options(forward_stream_bytes=1)
    assert capi.forward_chunk(d, tiny) == 1 and capi.workspace_size(d, tiny) >= item
    whole = capi.make_options(forward_stream_bytes=1 << 40)
    assert capi.forward_chunk(d, whole) == 128 and capi.workspace_size(d, whole) >= 128 * item
    # a cut batch uses the budget as two buffers: a chunk fits half of it
    for budget in (3 * item, 5 * item + 17, 40 * item):
        o = capi.make_options(forward_stream_bytes=budget)
        c = capi.forward_chunk(d, o)
        most = max(1, budget // 2 // item)
        assert (most + 1) // 2 <= c <= most
        assert capi.workspace_size(d, o) < capi.workspace_size(d, whole)
        assert capi.workspace_size(d, o) == capi.workspace_size(d, capi.make_options(budget, 0, True))


def test_descriptors_around_four_gib_of_activation_streams():
    """Stage entry points hold the streams of the whole batch.  From 4 GiB on the kernels with 32-bit byte offsets
    are not used: the layout query stops answering item-innermost.  The whole-op forward never gets there: it
    cuts the batch, so its workspace and its kernels are those of one chunk."""
    import ctypes as ct
    from geo_amd import _native, capi
    sw = (4096, 16, 1, 256)                     # the SC linear mapping: 64 KiB of stream words per item
    item = 4 * 4 * 16 * 256
    inner = ct.c_int(-1)
    words = ct.c_size_t(0)
    for n, want in ((65535, 1), (65536, 0), (70000, 0)):
        d = capi.make_desc((n, 16, 1, 256), sw, 128)
        assert _native.lib().geo_sc_act_stream_layout(ct.byref(d), ct.byref(inner)) == 0
        assert inner.value == want, n
        assert _native.lib().geo_sc_act_stream_words(ct.byref(d), ct.byref(words)) == 0
        assert words.value * 4 == n * item
        assert capi.skips_zero_rail(d)          # the weight buffer's format depends on the kernel's shape only
        nc = capi.forward_chunk(d)
        assert nc * item <= 256 << 20
        # a chunk of the forward is itself a geometry below the limit, with the fast layout
        dc = capi.make_desc((nc, 16, 1, 256), sw, 128)
        assert _native.lib().geo_sc_act_stream_layout(ct.byref(dc), ct.byref(inner)) == 0 and inner.value == 1
    sizes = {capi.workspace_size(capi.make_desc((n, 16, 1, 256), sw, 128)) for n in (65535, 65536, 70000)}
    assert max(sizes) - min(sizes) <= 8 * item  # chunk sizes may differ by a few items, not by the batch


def test_stream_tables_are_constants_of_the_library():
    """The comparison tables the generators read (evaluated at compile time) against the oracle's register:
    posp1 inverts the cycle from state 1, thr[code] holds [code > state] along the doubled cycle."""
    import ctypes as ct
    import numpy as np
    from geo_amd import _native
    from oracle import sc_oracle as so
    lib = _native.lib()
    nbytes = ct.c_size_t(99)
    assert lib.geo_sc_stream_tables_size(64, ct.byref(nbytes)) == 0 and nbytes.value == 0
    assert lib.geo_sc_stream_table_copy(100, None, 0, None) == 2
    for L in (8, 16, 32, 64, 128, 256):
        n = ct.c_size_t(0)
        assert lib.geo_sc_stream_table_copy(L, None, 0, ct.byref(n)) == 0
        wpc = (2 * L + 31) // 32 + 2
        assert n.value == L + L * wpc
        buf = np.zeros(n.value, dtype=np.uint32)
        assert lib.geo_sc_stream_table_copy(L, buf.ctypes.data_as(ct.c_void_p), 3, None) == 1
        assert lib.geo_sc_stream_table_copy(L, buf.ctypes.data_as(ct.c_void_p), n.value, None) == 0
        nb = so.nbits_for_length(L)
        cyc = [1]
        for _ in range(L - 2):
            cyc.append(so.lfsr_step(nb, cyc[-1]))
        assert so.lfsr_step(nb, cyc[-1]) == 1 and sorted(cyc) == list(range(1, L))
        for j, state in enumerate(cyc):
            assert buf[state - 1] == j + 1
        thr = buf[L:].reshape(L, wpc)
        bits = ((thr[:, :, None] >> (31 - np.arange(32, dtype=np.uint32))) & 1).reshape(L, wpc * 32)
        states = np.array([cyc[j % (L - 1)] for j in range(wpc * 32)])
        assert np.array_equal(bits, (np.arange(L)[:, None] > states[None, :]).astype(bits.dtype))


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
