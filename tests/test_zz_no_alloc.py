"""The forward entry point that allocates nothing (geo_sc_conv2d_add_partial_forward_static: tables and
stream buffers in a static device array of the library) against the workspace-taking entry point it is
a variant of: same counts, bit for bit, on two calls in a row of which the second is smaller, so that
the first call's streams are still in the array when the second runs."""
import numpy as np
import pytest
import torch

from geo_amd import workloads as wl

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from geo_amd import capi as m
    return m


CASES = [
    # larger first: 4-layer-CNN-sized layer (two packs, 5-wide kernel, progressive loading) ...
    ((16, 32, 16, 16), (32, 32, 5, 5), (2, 2), 64, dict(total_width=7, load_width=2, load_wait_w=2, load_wait_a=2)),
    # ... then a smaller problem with other strides, one pack, partial c_out tile
    ((3, 5, 9, 7), (6, 5, 3, 3), (1, 1), 32, {}),
]


def test_static_workspace_forward_equals_workspace_forward(capi):
    from oracle import sc_oracle as so
    for shape_x, shape_w, pad, L, loading in CASES:
        x, w = wl.make_inputs(shape_x, shape_w, "prescribed", seed=L)
        xd, wd = x.cuda(), w.cuda()
        d = capi.make_desc(xd.shape, wd.shape, L, pad, **loading)
        assert capi.workspace_size(d) <= capi.STATIC_WORKSPACE_BYTES
        expect = capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d)
        out = torch.full(capi.output_shape(d), -7, dtype=torch.int32, device="cuda")
        capi.conv2d_add_partial_forward_static(xd, wd, out, d)
        torch.cuda.synchronize()
        assert torch.equal(out, expect), (shape_x, shape_w)
        oracle = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, **loading)
        assert np.array_equal(out.cpu().numpy(), oracle), (shape_x, shape_w)


def test_static_workspace_forward_rejects_problems_beyond_its_limit(capi):
    x = torch.zeros((256, 128, 16, 16), device="cuda")
    w = torch.zeros((128, 128, 3, 3), device="cuda")
    d = capi.make_desc(x.shape, w.shape, 128, (1, 1))
    assert capi.workspace_size(d) > capi.STATIC_WORKSPACE_BYTES
    out = torch.zeros(capi.output_shape(d), dtype=torch.int32, device="cuda")
    with pytest.raises(capi.GeoScError) as e:
        capi.conv2d_add_partial_forward_static(x, w, out, d)
    assert e.value.status == 3   # GEO_SC_ERR_WORKSPACE
