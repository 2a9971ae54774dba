"""The forward entry point that allocates nothing (geo_sc_conv2d_add_partial_forward_static: both
stream buffers in a static device array of the library) against the workspace-taking entry point it is
a variant of: same counts, bit for bit, on two calls in a row of which the second is smaller, so that
the first call's streams are still in the array when the second runs; that it leaves the device's free
memory as it found it; a batch larger than the array holds at once (chunks); a HIP graph of it, replayed."""
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
        assert capi.workspace_size(d) <= capi.static_workspace_bytes()
        expect = capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d)
        out = torch.full(capi.output_shape(d), -7, dtype=torch.int32, device="cuda")
        capi.conv2d_add_partial_forward_static(xd, wd, out, d)
        torch.cuda.synchronize()
        assert torch.equal(out, expect), (shape_x, shape_w)
        oracle = so.conv2d_add_partial(x.numpy(), w.numpy(), L, pad, **loading)
        assert np.array_equal(out.cpu().numpy(), oracle), (shape_x, shape_w)


def test_static_workspace_forward_allocates_nothing_and_cuts_large_batches(capi):
    """Free device memory is the same before and after (the caller's tensors exist beforehand), also for a
    batch whose streams are several times the array: those run in chunks behind the weight streams."""
    assert capi.static_workspace_bytes() == 32 << 20
    x, w = wl.make_inputs((512, 32, 16, 16), (32, 32, 3, 3), "sparse", seed=5)
    xd, wd = x.cuda(), w.cuda()
    L, pad = 128, (1, 1)
    d = capi.make_desc(xd.shape, wd.shape, L, pad)
    whole = capi.make_options(forward_stream_bytes=1 << 40)
    assert capi.workspace_size(d, whole) > 2 * capi.static_workspace_bytes()
    expect = capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d, options=whole)
    out = torch.full(capi.output_shape(d), -7, dtype=torch.int32, device="cuda")
    capi.conv2d_add_partial_forward_static(xd, wd, out, d)   # first call on the device: symbol lookup
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    out.fill_(-7)
    capi.conv2d_add_partial_forward_static(xd, wd, out, d)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.equal(out, expect)
    assert int(expect.abs().max()) > 0


def test_static_workspace_forward_in_a_hip_graph(capi):
    """Captured after geo_sc_init, replayed three times with the program's own eager calls (which overwrite the
    shared array) and synchronisations in between: every replay gives the eager counts."""
    capi.init()
    x, w = wl.make_inputs((8, 16, 12, 12), (24, 16, 3, 3), "sparse", seed=9)
    xd, wd = x.cuda(), w.cuda()
    L, pad = 64, (1, 1)
    d = capi.make_desc(xd.shape, wd.shape, L, pad)
    expect = capi.conv2d_add_partial_forward(xd, wd, L, pad, desc=d)
    out = torch.zeros(capi.output_shape(d), dtype=torch.int32, device="cuda")
    x2, w2 = wl.make_inputs((3, 5, 9, 7), (6, 5, 3, 3), "prescribed", seed=2)
    x2d, w2d = x2.cuda(), w2.cuda()
    d2 = capi.make_desc(x2d.shape, w2d.shape, 32, (1, 1))
    out2 = torch.zeros(capi.output_shape(d2), dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        capi.conv2d_add_partial_forward_static(xd, wd, out, d)   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        capi.conv2d_add_partial_forward_static(xd, wd, out, d)
    for _ in range(3):
        out.fill_(-1)
        capi.conv2d_add_partial_forward_static(x2d, w2d, out2, d2)   # eager work on the same array
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, expect)


def test_static_workspace_forward_rejects_problems_beyond_its_limit(capi):
    # weight streams alone larger than the array: the SC linear layer (403 MB of rail-packed lines)
    x = torch.zeros((4, 16, 1, 256), device="cuda")
    w = torch.zeros((4096, 16, 1, 256), device="cuda")
    d = capi.make_desc(x.shape, w.shape, 128, (0, 0))
    assert capi.workspace_size(d) > capi.static_workspace_bytes()
    out = torch.zeros(capi.output_shape(d), dtype=torch.int32, device="cuda")
    with pytest.raises(capi.GeoScError) as e:
        capi.conv2d_add_partial_forward_static(x, w, out, d)
    assert e.value.status == 3   # GEO_SC_ERR_WORKSPACE
