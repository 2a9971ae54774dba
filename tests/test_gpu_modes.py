"""GPU parity of the z and yz accumulation modes (conv2d_add_partial_variable_acc with dim=0,
conv2d_add_yz_variable_acc) against the CPU oracle, through the C ABI and through the
PyTorch module with the reference's op names.  Bit-exact."""
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


@pytest.fixture(scope="module")
def so():
    from oracle import sc_oracle
    return sc_oracle


def run(capi, x, w, L, pad, mode, zu=1, loading=(7, 8, 1, 1)):
    y = capi.conv2d_add_partial_forward(x.cuda(), w.cuda(), L, pad, *loading, accumulate=mode, z_unit=zu)
    torch.cuda.synchronize()
    return y.cpu().numpy()


CASES = [
    # x shape, w shape, pad (last dim, the one before)
    ((2, 7, 6, 7), (19, 7, 3, 3), (1, 1)),     # ragged channel blocks, two c_out tiles
    ((3, 4, 5, 9), (5, 4, 1, 3), (0, 0)),      # w_k = 1 (three channels per trip + tail)
    ((2, 5, 8, 6), (40, 5, 5, 2), (0, 2)),     # w_k = 5, three c_out tiles
    ((2, 3, 6, 6), (4, 3, 2, 4), (1, 0)),      # run-time kernel extent
    ((5, 6, 3, 8), (3, 6, 3, 3), (0, 0)),      # single output row
    ((70, 8, 1, 1), (33, 8, 1, 1), (0, 0)),    # SC-linear mapping
]


@pytest.mark.parametrize("case", range(len(CASES)))
@pytest.mark.parametrize("L", [8, 64, 256])
def test_z_mode_matches_oracle(capi, so, case, L):
    sx, sw, pad = CASES[case]
    x, w = wl.make_inputs(sx, sw, "prescribed", seed=300 + case)
    print(f"z-mode case {sx} {sw} pad {pad} L {L}", flush=True)
    exp = so.conv2d_modes(x.numpy(), w.numpy(), L, pad, "z")
    assert np.array_equal(run(capi, x, w, L, pad, "z"), exp)


@pytest.mark.parametrize("case", range(len(CASES)))
@pytest.mark.parametrize("L,zu", [(8, 2), (64, 3), (128, 1), (256, 4), (32, 100)])
def test_yz_mode_matches_oracle(capi, so, case, L, zu):
    sx, sw, pad = CASES[case]
    x, w = wl.make_inputs(sx, sw, "prescribed", seed=400 + case)
    print(f"yz-mode case {sx} {sw} pad {pad} L {L} z_unit {zu}", flush=True)
    exp = so.conv2d_modes(x.numpy(), w.numpy(), L, pad, "yz", zu)
    assert np.array_equal(run(capi, x, w, L, pad, "yz", zu), exp)


@pytest.mark.parametrize("mode,zu", [("z", 1), ("yz", 2)])
@pytest.mark.parametrize("loading", [(7, 2, 2, 3), (7, 1, 3, 5), (7, 3, 40, 7)])
def test_modes_progressive_loading(capi, so, mode, zu, loading):
    x, w = wl.make_inputs((2, 5, 7, 6), (6, 5, 3, 3), "prescribed", seed=77)
    for L in (16, 128):
        exp = so.conv2d_modes(x.numpy(), w.numpy(), L, (1, 1), mode, zu, *loading)
        assert np.array_equal(run(capi, x, w, L, (1, 1), mode, zu, loading), exp), (L, loading)


def test_yz_is_sum_of_y_over_channel_blocks_at_layer_size(capi):
    """Size-independent property at a training-size layer (no CPU oracle run): the yz result
    equals the sum over channel blocks of y-mode results of the blocks."""
    x, w = wl.make_inputs((64, 32, 16, 16), (32, 32, 3, 3), "kaiming", seed=5)
    xd, wd = x.cuda(), w.cuda()
    got = capi.conv2d_add_partial_forward(xd, wd, 128, (1, 1), accumulate="yz", z_unit=8)
    exp = torch.zeros_like(got)
    for c0 in range(0, 32, 8):
        exp += capi.conv2d_add_partial_forward(xd[:, c0:c0 + 8].contiguous(), wd[:, c0:c0 + 8].contiguous(), 128,
                                               (1, 1))
    assert torch.equal(got, exp)


def test_torch_module_ops(so):
    import geo_amd  # noqa: F401  (puts the modules on the path)
    from geo_amd import _native
    ext = _native.module("sc_extension_cuda")
    x, w = wl.make_inputs((3, 6, 6, 6), (10, 6, 3, 3), "prescribed", seed=88)
    xd, wd = x.cuda(), w.cuda()
    yz = ext.conv2d_add_partial_variable_acc(xd, wd, 64, (1, 1), (1, 1), 7, 2, 3, True, 0)
    assert yz.dtype == torch.int32
    assert np.array_equal(yz.cpu().numpy(), so.conv2d_modes(x.numpy(), w.numpy(), 64, (1, 1), "z", 1, 7, 2, 3, 3))
    yy = ext.conv2d_add_partial_variable_acc(xd, wd, 64, (1, 1), (1, 1), 7, 2, 3, True, 1)
    assert np.array_equal(yy.cpu().numpy(), so.conv2d_add_partial(x.numpy(), w.numpy(), 64, (1, 1), 7, 2, 3, 3))
    for zu in (1, 4, 6, 64):
        y = ext.conv2d_add_yz_variable_acc(xd, wd, 64, (1, 1), (1, 1), 7, 2, 3, 5, True, zu)
        assert np.array_equal(y.cpu().numpy(),
                              so.conv2d_modes(x.numpy(), w.numpy(), 64, (1, 1), "yz", zu, 7, 2, 3, 5)), zu
    with pytest.raises(RuntimeError):
        ext.conv2d_add_yz_variable_acc(xd, wd, 64, (1, 1), (1, 1), 7, 2, 3, 5, True, 0)


# ------------------------------------------------------------------ surrogate backward
RTOL = 1e-5  # fp32 gradients: max|got - ref| <= 1e-5 * max|ref| against the float64 oracle


def rel_err(got, ref):
    ref = ref.double().cpu()
    return ((got.double().cpu() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()


BWD_CASES = [
    # shape_x, shape_w, pad, input kind, weight scale
    ((2, 7, 5, 6), (4, 7, 3, 2), (1, 1), "q7", 3.0),
    ((3, 8, 9, 9), (10, 8, 3, 3), (1, 1), "q7", 4.0),
    ((1, 4, 7, 8), (3, 4, 2, 3), (2, 0), "prescribed", 0.5),
    ((6, 16, 1, 8), (40, 16, 1, 8), (0, 0), "prescribed", 0.3),
    ((3, 70, 6, 6), (140, 70, 3, 3), (1, 1), "kaiming", 3.0),
]


@pytest.mark.parametrize("case", range(len(BWD_CASES)))
@pytest.mark.parametrize("mode,zu", [("z", 1), ("yz", 1), ("yz", 3), ("yz", 4), ("yz", 64)])
def test_backward_modes_match_float64_oracle(capi, case, mode, zu):
    from oracle import surrogate
    shape_x, shape_w, pad, kind, scale = BWD_CASES[case]
    print(f"backward {mode} z_unit {zu} case {shape_x} {shape_w} pad {pad}", flush=True)
    x, w = wl.make_inputs(shape_x, shape_w, kind, seed=shape_x[1])
    w = (w * scale).contiguous()
    w.view(-1)[::7] = 0.0
    d = capi.make_desc(x.shape, w.shape, 128, pad)
    g = torch.randn(capi.output_shape(d), generator=torch.Generator().manual_seed(1))
    gx, gw = capi.conv2d_add_partial_backward(x.cuda(), w.cuda(), g.cuda(), 128, pad, accumulate=mode, z_unit=zu)
    torch.cuda.synchronize()
    rx, rw, _ = surrogate.surrogate_autograd(x, w, g, pad, mode=mode, z_unit=min(zu, shape_x[1]))
    assert rel_err(gx, rx) <= RTOL, ("grad_x", rel_err(gx, rx))
    assert rel_err(gw, rw) <= RTOL, ("grad_w", rel_err(gw, rw))
    gx2, none = capi.conv2d_add_partial_backward(x.cuda(), w.cuda(), g.cuda(), 128, pad, need_grad_w=False,
                                                 accumulate=mode, z_unit=zu)
    none2, gw2 = capi.conv2d_add_partial_backward(x.cuda(), w.cuda(), g.cuda(), 128, pad, need_grad_x=False,
                                                  accumulate=mode, z_unit=zu)
    assert none is None and none2 is None
    assert torch.equal(gx2, gx) and rel_err(gw2, gw) <= 1e-6 and rel_err(gw2, rw) <= RTOL


@pytest.mark.parametrize("forward,kw", [("z_bin", {}), ("yz_bin", {"z_unit": 4, "load_wait_a": 3}),
                                        ("yz_bin", {})])
def test_conv2d_generic_modes(so, forward, kw):
    """The functional layer: SC value from the kernels, gradient of the matching surrogate."""
    from geo_amd import utils_functional as uf
    from oracle import surrogate
    x, w = wl.make_inputs((3, 6, 6, 6), (8, 6, 3, 3), "prescribed", seed=5)
    w = (w * 2).contiguous()
    xd = x.cuda().requires_grad_(True)
    wd = w.cuda().requires_grad_(True)
    y = uf.conv2d_generic(xd, wd, (1, 1), (1, 1), bit_length=64, forward=forward, generator="lfsr", load_unit=2,
                          load_wait_w=2, **kw)
    mode = "z" if forward == "z_bin" else "yz"
    zu = min(kw.get("z_unit", 1024), 6)
    wa = kw.get("load_wait_a", 1) if mode == "yz" else 2
    exp = so.conv2d_modes(x.numpy(), w.numpy(), 64, (1, 1), mode, zu, 7, 2, 2, wa)
    assert np.array_equal((y.detach().cpu() * 64).round().int().numpy(), exp)
    g = torch.randn(y.shape, generator=torch.Generator().manual_seed(3))
    y.backward(g.cuda())
    rx, rw, _ = surrogate.surrogate_autograd(x, w, g, (1, 1), mode=mode, z_unit=zu)
    assert rel_err(xd.grad, rx) <= RTOL and rel_err(wd.grad, rw) <= RTOL
    with pytest.raises(NotImplementedError):
        uf.conv2d_generic(x, w, (1, 1), (1, 1), bit_length=64, forward=forward, generator="lfsr")
