"""SC layer modules with the reference's interface (utils_class.py)."""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import utils_functional


class Conv2d_Add_Partial(nn.Conv2d):
    """SC Conv2d with partial binary accumulation (utils_class.py:11-35): keeps a
    full-precision ``weight_org`` buffer, quantises input and weight in place to ``prec``
    bits, then runs the SC convolution at stream length 2**err."""

    def __init__(self, *kargs, **kwargs):
        super().__init__(*kargs, **kwargs)
        self.register_buffer("weight_org", self.weight.data.clone())

    def forward(self, input, prec=7, err=7, forward="1d_bin", generator="lfsr", z_unit=8, legacy=False, load_unit=8,
                load_wait_w=2, load_wait_a=2):
        input.data = utils_functional.quantize(input.data, prec=prec)
        self.weight.data = utils_functional.quantize(self.weight_org, prec=prec)
        return utils_functional.conv2d_generic(
            input, self.weight, bit_length=2 ** err, padding=self.padding, stride=self.stride, forward=forward,
            generator=generator, legacy=legacy, z_unit=z_unit, load_unit=load_unit, load_wait_w=load_wait_w,
            load_wait_a=load_wait_a)


def _fixed_affine(module, x, mean, var):
    """Batch-norm folded to y = x*w_n + b_n with w_n, b_n quantised to 8 bits under a shared
    power-of-two scale (utils_class.py:52-64)."""
    if module.affine:
        weight, bias = module.weight.data, module.bias.data
    else:
        weight, bias = 1, 0
    inv = torch.sqrt(var + module.eps)
    w_n = weight / inv
    b_n = bias - mean * weight / inv
    w_n, module.scale = utils_functional.quantize_shift(w_n.detach())
    b_n, _ = utils_functional.quantize_shift(b_n.detach(), module.scale)
    return w_n, b_n


class BatchNorm2d_fixed(nn.BatchNorm2d):
    """2-d batch norm whose value is the fixed-point affine; gradients are those of the
    ordinary batch norm (utils_class.py:37-65)."""

    def __init__(self, *kargs, **kwargs):
        super().__init__(*kargs, **kwargs)
        self.register_buffer("scale", None)

    def forward(self, x):
        out = F.batch_norm(x, self.running_mean, self.running_var, self.weight, self.bias, training=self.training)
        if self.training:
            mean, var = x.mean(dim=(0, 2, 3)), x.var(dim=(0, 2, 3), unbiased=False)
        else:
            mean, var = self.running_mean, self.running_var
        w_n, b_n = _fixed_affine(self, x, mean, var)
        out.data = (x.data * w_n.reshape(-1, 1, 1) + b_n.reshape(-1, 1, 1)).to(out.dtype)
        return out


class BatchNorm1d_fixed(nn.BatchNorm1d):
    """1-d counterpart (utils_class.py:67-93)."""

    def __init__(self, *kargs, **kwargs):
        super().__init__(*kargs, **kwargs)
        self.register_buffer("scale", None)

    def forward(self, x):
        out = F.batch_norm(x, self.running_mean, self.running_var, self.weight, self.bias, training=self.training)
        if self.training:
            mean, var = x.mean(dim=0), x.var(dim=0, unbiased=False)
        else:
            mean, var = self.running_mean, self.running_var
        w_n, b_n = _fixed_affine(self, x, mean, var)
        out.data = (x.data * w_n + b_n).to(out.dtype)
        return out
