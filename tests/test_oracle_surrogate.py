"""Pins the gradient oracle (oracle/surrogate.py): autograd restatement == closed form ==
central finite differences, including weights that are exactly zero, and the value
overwrite leaving gradients untouched."""
import numpy as np
import pytest
import torch

from geo_amd import workloads as wl
from oracle import surrogate


def _case(seed, shape_x=(2, 3, 5, 6), shape_w=(4, 3, 3, 2)):
    x, w = wl.make_inputs(shape_x, shape_w, "q7", seed=seed)
    w = w * 3
    w.view(-1)[::5] = 0.0           # exact zeros: both clamp branches pass gradient
    g = torch.randn((shape_x[0], shape_w[0], shape_x[2] + 2 - shape_w[2] + 1, shape_x[3] + 2 - shape_w[3] + 1),
                    generator=torch.Generator().manual_seed(seed))
    return x.double(), w.double(), g.double()


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_autograd_matches_closed_form(seed):
    x, w, g = _case(seed)
    gx, gw, val = surrogate.surrogate_autograd(x, w, g, (1, 1))
    gx2, gw2, val2 = surrogate.surrogate_closed_form(x.numpy(), w.numpy(), g.numpy(), (1, 1))
    assert np.allclose(val.numpy(), val2, rtol=1e-12, atol=1e-12)
    assert np.allclose(gx.numpy(), gx2, rtol=1e-11, atol=1e-12)
    assert np.allclose(gw.numpy(), gw2, rtol=1e-11, atol=1e-12)
    # at w == 0 the gradient is the sum of both rails' terms, not zero
    zero = (w == 0).numpy()
    assert zero.any() and np.abs(gw.numpy()[zero]).max() > 0


def test_value_overwrite_does_not_change_gradients():
    x, w, g = _case(3)
    gx, gw, val = surrogate.surrogate_autograd(x, w, g, (1, 1))
    fake = torch.full_like(val, 0.25)
    gx2, gw2, _ = surrogate.surrogate_autograd(x, w, g, (1, 1), sc_value=fake)
    assert torch.equal(gx, gx2) and torch.equal(gw, gw2)


def test_asymmetric_padding_and_rectangular_kernels():
    x, w = wl.make_inputs((1, 2, 4, 7), (3, 2, 2, 3), "prescribed", seed=4)
    g = torch.randn((1, 3, 4 + 0 - 2 + 1, 7 + 4 - 3 + 1), generator=torch.Generator().manual_seed(4))
    gx, gw, val = surrogate.surrogate_autograd(x, w, g, (2, 0))
    gx2, gw2, val2 = surrogate.surrogate_closed_form(x.numpy(), w.numpy(), g.numpy(), (2, 0))
    assert val.shape == g.shape
    assert np.allclose(gx.numpy(), gx2, atol=1e-12) and np.allclose(gw.numpy(), gw2, atol=1e-12)


def test_central_finite_differences():
    x, w, g = _case(5, (1, 2, 4, 4), (2, 2, 3, 3))
    w = w + 0.013                     # keep away from the clamp kink for the FD check
    gx, gw, _ = surrogate.surrogate_autograd(x, w, g, (1, 1))

    def loss(xv, wv):
        _, _, val = surrogate.surrogate_closed_form(xv, wv, g.numpy(), (1, 1))
        return float((val * g.numpy()).sum())

    eps = 1e-6
    xn, wn = x.numpy().copy(), w.numpy().copy()
    rng = np.random.default_rng(0)
    for _ in range(12):
        idx = tuple(rng.integers(0, s) for s in xn.shape)
        xp, xm = xn.copy(), xn.copy()
        xp[idx] += eps
        xm[idx] -= eps
        fd = (loss(xp, wn) - loss(xm, wn)) / (2 * eps)
        assert abs(fd - gx[idx].item()) <= 1e-6 * max(1.0, abs(fd))
        idx = tuple(rng.integers(0, s) for s in wn.shape)
        wp, wm = wn.copy(), wn.copy()
        wp[idx] += eps
        wm[idx] -= eps
        fd = (loss(xn, wp) - loss(xn, wm)) / (2 * eps)
        assert abs(fd - gw[idx].item()) <= 1e-6 * max(1.0, abs(fd))


# ------------------------------------------------------------------ z / yz accumulation modes
@pytest.mark.parametrize("mode,zu", [("y", 1), ("z", 1), ("yz", 1), ("yz", 2), ("yz", 3)])
def test_modes_autograd_matches_closed_form(mode, zu):
    x, w, g = _case(11, (2, 5, 5, 6), (4, 5, 3, 2))
    gx, gw, val = surrogate.surrogate_autograd(x, w, g, (1, 1), mode=mode, z_unit=zu)
    gx2, gw2, val2 = surrogate.surrogate_closed_form_modes(x.numpy(), w.numpy(), g.numpy(), (1, 1), mode, zu)
    assert np.allclose(val.numpy(), val2, rtol=1e-12, atol=1e-12)
    assert np.allclose(gx.numpy(), gx2, rtol=1e-11, atol=1e-12)
    assert np.allclose(gw.numpy(), gw2, rtol=1e-11, atol=1e-12)
    if mode == "y":
        gx3, gw3, val3 = surrogate.surrogate_closed_form(x.numpy(), w.numpy(), g.numpy(), (1, 1))
        assert np.allclose(gx2, gx3, atol=1e-12) and np.allclose(gw2, gw3, atol=1e-12)


def test_modes_reduce_to_y_mode():
    x, w, g = _case(12, (2, 4, 5, 6), (3, 4, 3, 2))
    ref = surrogate.surrogate_autograd(x, w, g, (1, 1))
    # one channel block = y-mode
    got = surrogate.surrogate_autograd(x, w, g, (1, 1), mode="yz", z_unit=4)
    assert all(torch.equal(a, b) for a, b in zip(ref, got))
    # yz = sum over channel blocks of y-mode on the blocks
    got = surrogate.surrogate_autograd(x, w, g, (1, 1), mode="yz", z_unit=3)
    val = 0
    gxs, gws = [], []
    for c0, c1 in ((0, 3), (3, 4)):
        gx, gw, v = surrogate.surrogate_autograd(x[:, c0:c1], w[:, c0:c1], g, (1, 1))
        val = val + v
        gxs.append(gx)
        gws.append(gw)
    assert torch.allclose(got[2], val, atol=1e-12)
    assert torch.allclose(got[0], torch.cat(gxs, 1), atol=1e-12)
    assert torch.allclose(got[1], torch.cat(gws, 1), atol=1e-12)


@pytest.mark.parametrize("mode,zu", [("z", 1), ("yz", 2)])
def test_modes_central_finite_differences(mode, zu):
    x, w, g = _case(13, (1, 3, 4, 4), (2, 3, 3, 3))
    w = w + 0.013
    gx, gw, _ = surrogate.surrogate_autograd(x, w, g, (1, 1), mode=mode, z_unit=zu)

    def loss(xv, wv):
        _, _, val = surrogate.surrogate_closed_form_modes(xv, wv, g.numpy(), (1, 1), mode, zu)
        return float((val * g.numpy()).sum())

    eps = 1e-6
    rng = np.random.default_rng(0)
    for _ in range(12):
        idx = tuple(rng.integers(0, s) for s in x.shape)
        xp, xm = x.numpy().copy(), x.numpy().copy()
        xp[idx] += eps
        xm[idx] -= eps
        assert abs((loss(xp, w.numpy()) - loss(xm, w.numpy())) / (2 * eps) - gx.numpy()[idx]) < 1e-6
        idx = tuple(rng.integers(0, s) for s in w.shape)
        wp_, wm_ = w.numpy().copy(), w.numpy().copy()
        wp_[idx] += eps
        wm_[idx] -= eps
        assert abs((loss(x.numpy(), wp_) - loss(x.numpy(), wm_)) / (2 * eps) - gw.numpy()[idx]) < 1e-6
