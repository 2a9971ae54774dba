"""Gradient oracle of the SC convolution layer: TEST INFRASTRUCTURE, never on the product
path.

The reference has no native backward.  It builds a floating-point surrogate of the layer
with ordinary torch ops and lets autograd differentiate it (utils_functional.py:611-634
with conv2d_or_bin_1d, utils_functional.py:235-252).  ``surrogate_autograd`` restates
exactly that composition (pad -> clamp -> per-row W x 1 convolutions -> 1 - exp(-z) ->
stack/sum -> value overwrite -> pos - neg) in double precision; ``surrogate_closed_form``
is an independent numpy evaluation of the derivative formulas, used to pin the first on
small shapes together with finite differences (tests/test_oracle_surrogate.py).

Pinning status: pinned by closed form + central finite differences; the reference's Python
modules are not imported.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F


def _groups(act, w_pos, w_neg, mode, z_unit):
    """(activation section, w_pos section, w_neg section) per add group, as the reference
    slices them: conv2d_or_bin_1d (utils_functional.py:235-252), conv2d_or_bin_z (:254-270),
    conv2d_or_bin_yz (:272-299)."""
    c_in, i_y, f_y = act.size(1), act.size(3), w_pos.size(3)
    if mode == "full":  # conv2d_or_approx (utils_functional.py:189-210): one group, everything OR-ed
        yield act, w_pos, w_neg
    elif mode == "z":
        for c in range(c_in):
            yield act[:, c:c + 1].clone(), w_pos[:, c:c + 1].clone(), w_neg[:, c:c + 1].clone()
    elif mode == "yz":
        for c in range(0, c_in, z_unit):
            c_end = c + z_unit if c + z_unit <= c_in else c_in
            for j in range(f_y):
                yield (act[:, c:c_end, :, j:i_y - f_y + j + 1].clone(), w_pos[:, c:c_end, :, j:j + 1].clone(),
                       w_neg[:, c:c_end, :, j:j + 1].clone())
    else:
        for j in range(f_y):
            yield act[..., j:i_y - f_y + j + 1].clone(), w_pos[..., j:j + 1].clone(), w_neg[..., j:j + 1].clone()


def surrogate_rails(act, w_pos, w_neg, mode="y", z_unit=1):
    """(positive rail, negative rail) of the surrogate on an already padded activation, as torch
    tensors that carry the autograd graph: per add group one convolution per rail, 1 - exp(-z),
    stacked and summed (conv2d_or_bin_1d utils_functional.py:235-252, conv2d_or_bin_z :254-270,
    conv2d_or_bin_yz :272-299, conv2d_or_approx :189-210 for mode "full").  Any dtype / device."""
    pos, neg = [], []
    for a_sec, wp_sec, wn_sec in _groups(act, w_pos, w_neg, mode, z_unit):
        pos.append(1 - torch.exp(-F.conv2d(a_sec, wp_sec)))
        neg.append(1 - torch.exp(-F.conv2d(a_sec, wn_sec)))
    return torch.stack(pos, 0).sum(0), torch.stack(neg, 0).sum(0)


def surrogate_autograd(x, w, grad_out, padding=(0, 0), sc_value=None, dtype=torch.float64, mode="y", z_unit=1):
    """(grad_x, grad_w, surrogate_value) as torch tensors of ``dtype``.

    ``padding=(p0,p1)``: p0 pads the last dim, p1 the one before (utils_functional.py:496).
    ``sc_value`` (optional) is written over the surrogate's value the way the reference does
    (utils_functional.py:632-633) to show that the overwrite does not reach the gradients.
    """
    x = torch.as_tensor(x).detach().to(dtype).requires_grad_(True)
    w = torch.as_tensor(w).detach().to(dtype).requires_grad_(True)
    g = torch.as_tensor(grad_out).detach().to(dtype)
    act = F.pad(x, (padding[0], padding[0], padding[1], padding[1]))
    w_pos = w.clamp(0, 100)
    w_neg = -(w.clamp(-100, 0))
    pos_v, neg_v = surrogate_rails(act, w_pos, w_neg, mode, z_unit)
    value = (pos_v - neg_v).detach().clone()
    if sc_value is not None:
        pos_v.data = torch.as_tensor(sc_value).to(dtype)
        neg_v.data = torch.zeros_like(neg_v)
    out = pos_v - neg_v
    out.backward(g)
    return x.grad.detach(), w.grad.detach(), value


def surrogate_closed_form_modes(x, w, grad_out, padding=(0, 0), mode="y", z_unit=1):
    """(grad_x, grad_w, value) in float64 numpy for any accumulation mode, written per add
    group from a dense product tensor (tiny shapes only):
        T[n,o,a,b,c,u,v] = xp[n,c,a+u,b+v]            (window view)
        z+-_G            = sum_{(c,u,v) in G} T * w+-[o,c,u,v]
        value            = sum_G (1-exp(-z+_G)) - (1-exp(-z-_G))
    with G the add groups: y {(c,u)} per v; z {(u,v)} per c; yz {(c in block,u)} per (block, v)."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    g = np.asarray(grad_out, dtype=np.float64)
    p0, p1 = int(padding[0]), int(padding[1])
    xp = np.pad(x, ((0, 0), (0, 0), (p1, p1), (p0, p0)))
    N, Cin, Wi, Hi = xp.shape
    Cout, _, W, H = w.shape
    Wo, Ho = Wi - W + 1, Hi - H + 1
    if mode == "y":
        groups = [[(c, u, v) for c in range(Cin) for u in range(W)] for v in range(H)]
    elif mode == "z":
        groups = [[(c, u, v) for u in range(W) for v in range(H)] for c in range(Cin)]
    elif mode == "full":
        groups = [[(c, u, v) for c in range(Cin) for u in range(W) for v in range(H)]]
    else:
        groups = [[(c, u, v) for c in range(c0, min(c0 + z_unit, Cin)) for u in range(W)]
                  for c0 in range(0, Cin, z_unit) for v in range(H)]
    wp = np.clip(w, 0, 100)
    wn = -np.clip(w, -100, 0)
    value = np.zeros((N, Cout, Wo, Ho))
    gxp = np.zeros_like(xp)
    gwp = np.zeros_like(w)
    gwn = np.zeros_like(w)
    for G in groups:
        zp = np.zeros((N, Cout, Wo, Ho))
        zn = np.zeros((N, Cout, Wo, Ho))
        for (c, u, v) in G:
            patch = xp[:, c, u:u + Wo, v:v + Ho]
            zp += patch[:, None] * wp[None, :, c, u, v, None, None]
            zn += patch[:, None] * wn[None, :, c, u, v, None, None]
        value += (1 - np.exp(-zp)) - (1 - np.exp(-zn))
        dzp = g * np.exp(-zp)
        dzn = -g * np.exp(-zn)
        for (c, u, v) in G:
            patch = xp[:, c, u:u + Wo, v:v + Ho]
            gwp[:, c, u, v] = np.einsum("noab,nab->o", dzp, patch)
            gwn[:, c, u, v] = np.einsum("noab,nab->o", dzn, patch)
            gxp[:, c, u:u + Wo, v:v + Ho] += np.einsum("noab,o->nab", dzp, wp[:, c, u, v])
            gxp[:, c, u:u + Wo, v:v + Ho] += np.einsum("noab,o->nab", dzn, wn[:, c, u, v])
    gw = gwp * ((w >= 0) & (w <= 100)) - gwn * ((w >= -100) & (w <= 0))
    gx = gxp[:, :, p1:Wi - p1, p0:Hi - p0]
    return gx, gw, value


def surrogate_closed_form(x, w, grad_out, padding=(0, 0)):
    """(grad_x, grad_w, value) in float64 numpy from the written-out derivative:
        z+-_v[n,co,a,b] = sum_{ci,u} xp[n,ci,a+u,b+v] * w+-[co,ci,u,v]
        value           = sum_v (1-exp(-z+_v)) - (1-exp(-z-_v))
        dL/dz+_v = g exp(-z+_v),  dL/dz-_v = -g exp(-z-_v)
        dL/dw    = [0<=w<=100] dL/dw+  -  [-100<=w<=0] dL/dw-
    """
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    g = np.asarray(grad_out, dtype=np.float64)
    p0, p1 = int(padding[0]), int(padding[1])
    xp = np.pad(x, ((0, 0), (0, 0), (p1, p1), (p0, p0)))
    N, Cin, Wi, Hi = xp.shape
    Cout, _, W, H = w.shape
    Wo, Ho = Wi - W + 1, Hi - H + 1
    wp = np.clip(w, 0, 100)
    wn = -np.clip(w, -100, 0)
    value = np.zeros((N, Cout, Wo, Ho))
    gxp = np.zeros_like(xp)
    gwp = np.zeros_like(w)
    gwn = np.zeros_like(w)
    for v in range(H):
        zp = np.zeros((N, Cout, Wo, Ho))
        zn = np.zeros((N, Cout, Wo, Ho))
        for u in range(W):
            patch = xp[:, :, u:u + Wo, v:v + Ho]
            zp += np.einsum("ncab,oc->noab", patch, wp[:, :, u, v])
            zn += np.einsum("ncab,oc->noab", patch, wn[:, :, u, v])
        value += (1 - np.exp(-zp)) - (1 - np.exp(-zn))
        dzp = g * np.exp(-zp)
        dzn = -g * np.exp(-zn)
        for u in range(W):
            patch = xp[:, :, u:u + Wo, v:v + Ho]
            gwp[:, :, u, v] = np.einsum("noab,ncab->oc", dzp, patch)
            gwn[:, :, u, v] = np.einsum("noab,ncab->oc", dzn, patch)
            gxp[:, :, u:u + Wo, v:v + Ho] += np.einsum("noab,oc->ncab", dzp, wp[:, :, u, v])
            gxp[:, :, u:u + Wo, v:v + Ho] += np.einsum("noab,oc->ncab", dzn, wn[:, :, u, v])
    gw = gwp * ((w >= 0) & (w <= 100)) - gwn * ((w >= -100) & (w <= 0))
    gx = gxp[:, :, p1:Wi - p1, p0:Hi - p0]
    return gx, gw, value
