"""Functional SC layer with the reference's interface (utils_functional.py), for the
configurations this build accelerates, all with the LFSR generators and ``legacy=False``:
``forward='1d_bin'`` (OR over input channels and kernel dim 2, binary add over kernel dim 3),
``forward='z_bin'`` (OR over the kernel window, add over input channels) and
``forward='yz_bin'`` (OR over ``z_unit`` input channels and kernel dim 2, add over kernel dim 3
and channel blocks).

Forward values come from the HIP SC kernels (integer counts / stream length); gradients
are those of the reference's floating-point surrogates ``conv2d_or_bin_1d`` / ``_z`` / ``_yz``
(utils_functional.py:235-299), computed by the HIP backward kernels instead of autograd
over two dense convolutions per add group.  The surrogate's own forward is never evaluated: the
reference overwrites its value with the SC result anyway (utils_functional.py:631-634).
"""
from __future__ import annotations

import torch

from . import capi

# Default precision is 8-bit integer, one bit is the sign (utils_functional.py:28)
prec_default = 7


def quantize(input, prec=8):
    """round(x * 2^prec) clamped to +-(2^prec - 1), scaled back (utils_functional.py:33-39)."""
    if input.is_cuda and input.dtype == torch.float32 and input.is_contiguous() and isinstance(prec, int) \
            and 1 <= prec <= 23 and not (torch.is_grad_enabled() and input.requires_grad):
        return capi.quantize(input, prec)   # the same values from one kernel instead of four
    prec_2 = 2 ** prec
    return (input * prec_2).round().clamp(-prec_2 + 1, prec_2 - 1) / prec_2


def quantize_shift(tensor, scale=None, scale_only=False):
    """Power-of-two scale, then 8-bit quantisation of tensor/scale (utils_functional.py:41-57)."""
    if scale_only:
        scale = 2 ** torch.ceil(torch.log2(torch.mean(tensor) * 2))
        return torch.ones_like(tensor) * scale, scale
    if scale is None:
        scale = 2 ** torch.ceil(torch.log2(torch.mean(tensor) * 3))
    q = ((tensor / scale) * 128).round().clamp(-127, 127) / 128
    return q * scale, scale


class _SCConv2dAddPartial(torch.autograd.Function):
    """value: SC count / L  (HIP forward);  gradient: surrogate (HIP backward)."""

    @staticmethod
    def forward(ctx, activation, weight, bit_length, padding, load_unit, load_wait, accumulate="y", z_unit=1,
                load_wait_a=None, generator="lfsr", seed=0):
        origin = activation.device
        dev = origin if activation.is_cuda else torch.device("cuda", torch.cuda.current_device())
        x = activation.detach().to(dev, torch.float32).contiguous()
        w = weight.detach().to(dev, torch.float32).contiguous()
        pad = (int(padding[0]), int(padding[1]))
        if activation.is_cuda:
            # sc_extension_cuda.conv2d_add_partial_variable_acc(..., prec_default, load_unit,
            # load_wait_w, False, 2): one wait for both generators (utils_functional.py:497)
            # (:504), and conv2d_add_yz_variable_acc(..., load_wait_w, load_wait_a, False, z_unit) (:508)
            loading = dict(total_width=prec_default, load_width=int(load_unit), load_wait_w=int(load_wait),
                           load_wait_a=int(load_wait if load_wait_a is None else load_wait_a))
        else:
            # host tensors take the reference's CPU entry point, which has no progressive
            # loading (utils_functional.py:493)
            loading = dict(capi.NEUTRAL_LOADING)
        z_unit = max(1, min(int(z_unit), x.shape[1]))
        if generator != "lfsr":
            loading = dict(capi.NEUTRAL_LOADING)  # the random generators have no progressive loading
        counts = capi.conv2d_add_partial_forward(x, w, int(bit_length), pad, accumulate=accumulate, z_unit=z_unit,
                                                 generator=generator, seed=seed, **loading)
        ctx.save_for_backward(x, w)
        ctx.accumulate = accumulate
        ctx.z_unit = z_unit
        ctx.pad = pad
        ctx.origin = origin
        ctx.bit_length = int(bit_length)
        ctx.act_dtype = activation.dtype
        ctx.w_dtype = weight.dtype
        ctx.w_device = weight.device
        # int32 * python float -> float32 in one kernel; exact, the length is a power of two
        return (counts * (1.0 / bit_length)).to(origin)

    @staticmethod
    def backward(ctx, grad_out):
        x, w = ctx.saved_tensors
        g = grad_out.detach().to(x.device, torch.float32).contiguous()
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        gx = gw = None
        if need_x or need_w:
            gx, gw = capi.conv2d_add_partial_backward(x, w, g, ctx.bit_length, ctx.pad, need_x, need_w,
                                                      accumulate=ctx.accumulate, z_unit=ctx.z_unit)
        if gx is not None:
            gx = gx.to(ctx.origin, ctx.act_dtype)
        if gw is not None:
            gw = gw.to(ctx.w_device, ctx.w_dtype)
        return gx, gw, None, None, None, None, None, None, None, None, None


def conv2d_generic(activation, weight, padding, stride, **kwargs):
    """Generic SC conv2d layer, same call as the reference's (utils_functional.py:406-634).

    Keyword arguments read: bit_length (128), generator (None), forward ('full_or'), legacy
    (False), load_unit (8), load_wait_w (1), load_wait_a (1), z_unit (1024); prec/acc/share are
    accepted and unused on these paths.  Implemented: forward='1d_bin' with generator='lfsr' or,
    on GPU tensors, 'acc'; forward='z_bin' / 'yz_bin' on GPU tensors (the reference sends those to
    its LFSR GPU ops whatever the generator, utils_functional.py:503-510); forward='full_or' on GPU
    tensors (random Bernoulli streams, :511-514); all with legacy=False; anything else raises
    NotImplementedError.
    """
    bit_length = kwargs.get("bit_length", 128)
    generator = kwargs.get("generator", None)
    forward = kwargs.get("forward", "full_or")
    legacy = kwargs.get("legacy", False)
    load_unit = kwargs.get("load_unit", 8)
    load_wait_w = kwargs.get("load_wait_w", 1)
    load_wait_a = kwargs.get("load_wait_a", 1)
    z_unit = kwargs.get("z_unit", 1024)
    ok_1d = forward == "1d_bin" and (generator == "lfsr" or (generator == "acc" and activation.is_cuda))
    ok_zyz = forward in ("z_bin", "yz_bin", "full_or") and activation.is_cuda
    if legacy or not (ok_1d or ok_zyz):
        raise NotImplementedError(
            f"conv2d_generic(forward={forward!r}, generator={generator!r}, legacy={legacy}, "
            f"cuda={activation.is_cuda}): this build implements forward='1d_bin' with generator='lfsr' and "
            "(on GPU tensors also 'acc'), and forward='z_bin'/'yz_bin'/'full_or' on GPU tensors, legacy=False")
    if isinstance(stride, int):
        stride = (stride, stride)
    if tuple(stride) != (1, 1):
        raise NotImplementedError("the SC kernels compute stride 1 only (the reference's native code ignores stride)")
    if isinstance(padding, int):
        padding = (padding, padding)
    if forward == "full_or":
        # sc_extension_cuda.conv2d_or_acc: Bernoulli random streams, OR over everything
        # (utils_functional.py:511-514); surrogate conv2d_or_approx (:616-617)
        return _SCConv2dAddPartial.apply(activation, weight, bit_length, tuple(padding), 8, 1, "full", 1, None, "rand",
                                         0)
    if forward == "1d_bin" and generator == "acc":
        # sc_extension_cuda.conv2d_add_partial_acc_acc (utils_functional.py:499-502)
        return _SCConv2dAddPartial.apply(activation, weight, bit_length, tuple(padding), 8, 1, "y", 1, None, "acc", 37)
    if forward == "z_bin":
        return _SCConv2dAddPartial.apply(activation, weight, bit_length, tuple(padding), load_unit, load_wait_w, "z")
    if forward == "yz_bin":
        return _SCConv2dAddPartial.apply(activation, weight, bit_length, tuple(padding), load_unit, load_wait_w,
                                         "yz", z_unit, load_wait_a)
    return _SCConv2dAddPartial.apply(activation, weight, bit_length, tuple(padding), load_unit, load_wait_w)


def sc_counts(activation, weight, bit_length, padding, forward="1d_bin", load_unit=8, load_wait_w=1, load_wait_a=1,
              z_unit=1024):
    """int32 SC counts of one layer without autograd (inference).  ``activation`` is fp32, or
    uint8 holding the 7-bit integers round(x * 128) that the fused layer epilogue emits.  Same
    argument meaning as ``conv2d_generic``'s keywords (utils_functional.py:406-510)."""
    if forward not in ("1d_bin", "z_bin", "yz_bin"):
        raise NotImplementedError(f"sc_counts(forward={forward!r})")
    mode = {"1d_bin": "y", "z_bin": "z", "yz_bin": "yz"}[forward]
    wait_a = load_wait_a if mode == "yz" else load_wait_w
    kw = dict(total_width=prec_default, load_width=int(load_unit), load_wait_w=int(load_wait_w),
              load_wait_a=int(wait_a), accumulate=mode, z_unit=max(1, min(int(z_unit), activation.shape[1])))
    pad = (int(padding[0]), int(padding[1]))
    w = weight.detach().float().contiguous()
    if activation.dtype == torch.uint8:
        return capi.conv2d_add_partial_forward_q7(activation.contiguous(), w, int(bit_length), pad, **kw)
    return capi.conv2d_add_partial_forward(activation.detach().float().contiguous(), w, int(bit_length), pad, **kw)
