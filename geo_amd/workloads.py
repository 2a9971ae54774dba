"""Synthetic inputs for the SC convolution workloads used by the tests and the benchmark.

The draws follow one fixed recipe so that every consumer (oracle, GPU path, compiled
reference) sees identical tensors: ``g = torch.Generator().manual_seed(0)``, then
``x = rand(shape_x)``, then ``w = rand(shape_w)*2-1``, then the optional masks.
"""
from __future__ import annotations

import math

import torch

# name -> (shape_x, shape_w, pad, L, view_x, view_w)
SHAPES = {
    # reference CPU-runnable case: 3->32 3x3 at 32x32, batch 32, L=64
    "C1": ((32, 3, 32, 32), (32, 3, 3, 3), 1, 64, None, None),
    # headline: 128->128 3x3 at 16x16, batch 256
    "C3": ((256, 128, 16, 16), (128, 128, 3, 3), 1, 128, None, None),
    # SC linear 4096->4096, batch 1024, OR groups of 16 inputs, written as a conv:
    # x (N,16,1,256), w (4096,16,1,256): OR over Cin*W=16, binary add over H=256 groups
    "C4": ((1024, 4096), (4096, 4096), 0, 128, (1024, 16, 1, 256), (4096, 16, 1, 256)),
    # ResNet-18-style 64->64 3x3 at 56x56, batch 128
    "C5": ((128, 64, 56, 56), (64, 64, 3, 3), 1, 256, None, None),
    # tiny shapes
    "T1": ((2, 3, 6, 6), (4, 3, 3, 3), 1, 64, None, None),
    "T2": ((2, 5, 9, 9), (7, 5, 5, 5), 2, 64, None, None),
    "T3": ((1, 4, 8, 11), (5, 4, 3, 5), 0, 64, None, None),
    "T4": ((3, 16, 1, 8), (9, 16, 1, 8), 0, 128, None, None),
}


def q7(t: torch.Tensor) -> torch.Tensor:
    return (t * 128).round().clamp(-127, 127) / 128


def make_inputs(shape_x, shape_w, mode: str = "prescribed", seed: int = 0, view_x=None, view_w=None):
    """(x, w) fp32 CPU tensors.  modes: prescribed | kaiming | q7 | sparse."""
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(shape_x, generator=g)
    w = torch.rand(shape_w, generator=g) * 2 - 1
    fan_in = 1
    for d in shape_w[1:]:
        fan_in *= d
    if mode == "prescribed":
        pass
    elif mode == "kaiming":
        w = w / math.sqrt(fan_in)
    elif mode == "q7":
        x = q7(x)
        w = q7(w / math.sqrt(fan_in))
    elif mode == "sparse":
        x = x * (torch.rand(shape_x, generator=g) < 0.1)
        w = w * (torch.rand(shape_w, generator=g) < 0.05)
    else:
        raise ValueError(mode)
    if view_x is not None:
        x = x.view(view_x)
    if view_w is not None:
        w = w.view(view_w)
    return x.contiguous(), w.contiguous()


def named(name: str, mode: str = "prescribed", seed: int = 0):
    """(x, w, pad, default_L) of a named shape."""
    sx, sw, pad, L, vx, vw = SHAPES[name]
    x, w = make_inputs(sx, sw, mode, seed, vx, vw)
    return x, w, pad, L


def bit_macs(x_shape, w_shape, pad, L) -> int:
    """Bipolar SC bit-MACs of one forward: N*Cout*Wo*Ho*Cin*W*H*L."""
    N, Cin, Wx, Hx = x_shape
    Cout, _, W, H = w_shape
    Wo = Wx + 2 * pad - W + 1
    Ho = Hx + 2 * pad - H + 1
    return N * Cout * Wo * Ho * Cin * W * H * L
