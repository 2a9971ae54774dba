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


class _SCConvBlock(torch.autograd.Function):
    """One block of the reference's networks in training mode as a single autograd node:
    SC convolution -> BatchNorm*_fixed on the batch statistics -> [relu] -> [AvgPool2d(2)] ->
    [Hardtanh(0, 1)] -> [7-bit quantisation of the next layer's input] (network.py:165-170).
    Forward: the HIP SC kernels, the batch statistics and the fixed-point affine exactly as
    BatchNorm*_fixed computes them (utils_class.py:49-62), then one fused epilogue kernel.
    Backward: the fused tail backward (gradient of an ordinary batch norm, masks from the
    fixed-point values), then the HIP surrogate backward of the convolution."""

    @staticmethod
    def forward(ctx, activation, weight, gamma, beta, bn, conv_kw, relu, pool, hardtanh, quant7):
        from . import capi
        x = activation.detach().float().contiguous()
        w = weight.detach().float().contiguous()
        torch_stats = conv_kw.get("torch_stats", False)
        conv_kw = {k: v for k, v in conv_kw.items() if k != "torch_stats"}
        L = conv_kw["bit_length"]
        counts = capi.conv2d_add_partial_forward(x, w, **conv_kw)
        gm = gamma.detach().float().contiguous() if gamma is not None else None
        bt = beta.detach().float().contiguous() if beta is not None else None
        # One launch for what BatchNorm*_fixed computes per channel (utils_class.py:52-62) and for what
        # its F.batch_norm(x, running_mean, running_var, weight, bias, training=True) call
        # (utils_class.py:49) does to the running statistics: that function's default momentum 0.1
        # and, for the gradient, its default eps 1e-5; the batch counter is not touched.
        if torch_stats:
            # the two PyTorch reductions BatchNorm*_fixed itself runs (utils_class.py:52-56)
            y = counts * (1.0 / L)   # exact: L is a power of two
            mean, var = y.mean(dim=(0, 2, 3)), y.var(dim=(0, 2, 3), unbiased=False)
            w_n, b_n, invstd, bn.scale = capi.bn_fixed_affine(mean, var, gm, bt, bn.eps,
                                                              counts.numel() // counts.shape[1], bn.running_mean,
                                                              bn.running_var)
        else:
            # the same statistics from exact integer sums: no y in memory, no dependence on a reduction order
            mean, var, w_n, b_n, invstd, bn.scale = capi.bn_fixed_from_counts(counts, L, gm, bt, bn.eps,
                                                                              bn.running_mean, bn.running_var)
        act, _ = capi.layer_epilogue(counts, L, w_n, b_n, relu=relu, pool=pool, hardtanh=hardtanh, quant7=quant7)
        ctx.save_for_backward(x, w, counts, w_n, b_n, mean, invstd,
                              gamma.detach() if gamma is not None else torch.empty(0, device=x.device))
        ctx.conv_kw, ctx.flags = conv_kw, (relu, pool, hardtanh)
        ctx.has_gamma = gamma is not None
        return act

    @staticmethod
    def backward(ctx, grad_out):
        from . import capi
        x, w, counts, w_n, b_n, mean, invstd, gamma = ctx.saved_tensors
        relu, pool, hardtanh = ctx.flags
        kw = ctx.conv_kw
        gy, gg, gb = capi.layer_tail_backward(counts, grad_out.detach().float().contiguous(), kw["bit_length"], w_n,
                                              b_n, mean, invstd, gamma if ctx.has_gamma else None, relu, pool,
                                              hardtanh)
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        gx = gw = None
        if need_x or need_w:
            gx, gw = capi.conv2d_add_partial_backward(x, w, gy, kw["bit_length"], kw["padding"], need_x, need_w,
                                                      accumulate=kw["accumulate"], z_unit=kw["z_unit"])
        return (gx, gw, gg if ctx.has_gamma else None, gb if ctx.has_gamma else None, None, None, None, None, None,
                None)


def quantize_weights(convs, prec=7):
    """``conv.weight.data = quantize(conv.weight_org, prec)`` (utils_class.py:33) for several layers in one launch;
    ``sc_conv_block(..., weight_ready=True)`` then skips its own."""
    if all(c.weight_org.is_cuda and c.weight_org.dtype == torch.float32 and c.weight_org.is_contiguous() for c in convs):
        from . import capi
        for c, q in zip(convs, capi.quantize_many([c.weight_org for c in convs], prec)):
            c.weight.data = q
    else:
        for c in convs:
            c.weight.data = utils_functional.quantize(c.weight_org, prec=prec)


def sc_conv_block(conv, bn, input, *, err=7, forward="1d_bin", z_unit=8, load_unit=8, load_wait_w=2, load_wait_a=2,
                  prec=7, relu=False, pool=True, hardtanh=True, quant7=True, torch_stats=False, weight_ready=False):
    """``hardtanh(pool(relu(bn(conv(input)))))`` of a ``Conv2d_Add_Partial`` and a
    ``BatchNorm2d_fixed`` / ``BatchNorm1d_fixed`` in training mode, fused (LFSR generators, GPU
    tensors).  Same in-place quantisation of ``input.data`` and ``conv.weight.data`` as
    ``Conv2d_Add_Partial.forward`` (utils_class.py:32-33).  The output is already quantised to 7
    bits (the next layer would do that to its input anyway) unless ``quant7=False``.  The batch statistics are
    the correctly rounded mean and variance of ``counts / L`` (exact integer sums, one HIP kernel);
    ``torch_stats=True`` takes them from PyTorch's float reductions as the module chain does (the two can differ
    in the last bit, which the 8-bit rounding of the affine hides except at a rounding boundary)."""
    if forward not in ("1d_bin", "z_bin", "yz_bin") or not input.is_cuda:
        raise NotImplementedError("sc_conv_block: LFSR modes 1d_bin / z_bin / yz_bin on GPU tensors")
    if tuple(conv.stride) != (1, 1):
        raise NotImplementedError("the SC kernels compute stride 1 only")
    # an input that is the untouched 7-bit output of a fused block already holds quantize(input, 7)
    if not (prec == 7 and getattr(input, "_geo_q7_version", None) == input._version):
        input.data = utils_functional.quantize(input.data, prec=prec)
    if not weight_ready:   # (quantize_weights has done it for all layers of the network)
        conv.weight.data = utils_functional.quantize(conv.weight_org, prec=prec)
    mode = {"1d_bin": "y", "z_bin": "z", "yz_bin": "yz"}[forward]
    kw = dict(bit_length=2 ** err, padding=(int(conv.padding[0]), int(conv.padding[1])),
              total_width=utils_functional.prec_default, load_width=int(load_unit), load_wait_w=int(load_wait_w),
              load_wait_a=int(load_wait_a if mode == "yz" else load_wait_w), accumulate=mode,
              z_unit=max(1, min(int(z_unit), conv.weight.shape[1])), torch_stats=bool(torch_stats))
    gamma, beta = (bn.weight, bn.bias) if bn.affine else (None, None)
    out = _SCConvBlock.apply(input, conv.weight, gamma, beta, bn, kw, relu, pool, hardtanh, quant7)
    if quant7 and hardtanh:
        out._geo_q7_version = out._version   # values k / 128, 0 <= k <= 127, until somebody writes to the tensor
    return out
